"""The CPU oracle against the committed golden vectors (outputs of the
reference's ``monarch_attention_torch`` for seeded inputs, written by
``tests/golden/make_golden.py`` in the build container)."""
import pytest
import torch

from helpers import assert_parity, golden_names, load_golden
from oracle.ma_oracle import monarch_attention_oracle

NAMES = golden_names()


def test_fixtures_present():
    assert len(NAMES) >= 60
    assert "c1_f32_N256_B16_T1" in NAMES


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_reference_output(name):
    g = load_golden(name)
    out = monarch_attention_oracle(g["q"], g["k"], g["v"], g["mask"], g["T"], g["B"], g["pre"])
    assert out.shape == g["out"].shape and out.dtype == g["out"].dtype
    # same ops, same machine arithmetic: the restatement is expected to be
    # bit-identical; allow the last place of the output dtype in case a BLAS
    # build orders an accumulation differently.
    if not torch.equal(out, g["out"]):
        ulp = {"f32": 2e-6, "f16": 2e-3, "bf16": 1.6e-2}[g["vdt"]]
        assert torch.allclose(out.float(), g["out"].float(), atol=ulp, rtol=ulp)


@pytest.mark.parametrize("name", NAMES)
def test_upcast_variant_within_gate(name):
    """The fp32-accumulate spelling of the low-precision matmuls (used for the
    timed CPU baseline and the large parity cases) stays within the parity
    gate of the reference's output."""
    g = load_golden(name)
    out = monarch_attention_oracle(g["q"], g["k"], g["v"], g["mask"], g["T"], g["B"], g["pre"],
                                   upcast=True)
    assert_parity(out, g["out"], g["vdt"] if g["dt"] == g["vdt"] else g["dt"], name)
