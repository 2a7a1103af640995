"""``ma_fwd_static``: the forward entry point that allocates nothing (its state
lives in an array the library holds on the GPU) against ``ma_fwd`` with a
caller-provided workspace, through the C ABI.

Both run the same kernels on the same inputs, so the gate is the strictest one:
bit-identical outputs (and, as a cross-check of the test itself, parity with the
CPU oracle at the usual tolerance).  Two calls in a row share the array, the
second on a smaller problem; problems beyond the array's size are refused.
"""
import pytest
import torch

from helpers import DT, assert_parity, block_safe_mask, seeded_qkv
from ma import _hip_lib as L
from ma.ma_hip import make_params
from oracle.ma_oracle import monarch_attention_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(lib, q, k, v, mask, T, B, pre, variant):
    """(ma_fwd output, ma_fwd_static output) for one problem."""
    outs = []
    stream = torch.cuda.current_stream().cuda_stream
    for static in (False, True):
        out = torch.full(v.shape, float("nan"), dtype=v.dtype, device=DEV)
        p = make_params(q, k, v, mask, out, T, B, pre, variant)
        if static:
            st = lib.ma_fwd_static(p, stream)
        else:
            nbytes = lib.ma_fwd_workspace_bytes(p)
            ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
            p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
            st = lib.ma_fwd(p, stream)
        L.check(st, "ma_fwd_static" if static else "ma_fwd")
        torch.cuda.synchronize()
        outs.append(out)
    return outs


CASES = [  # two calls in a row per case: (E, H, N, D, B, T, pre, dtype, masked), the second smaller than the first
    ((1, 16, 4096, 64, 64, 1, False, "f16", False), (1, 4, 1000, 64, 32, 2, True, "f16", True)),      # the metric workload first
    ((2, 3, 512, 64, 32, 3, False, "bf16", True), (1, 2, 197, 64, 16, 2, True, "bf16", False)),
    ((1, 2, 300, 48, 16, 2, False, "f32", True), (1, 1, 64, 48, 16, 1, False, "f32", False)),
    ((2, 12, 512, 64, 128, 2, False, "f16", True), (1, 3, 200, 64, 96, 2, True, "f16", False)),          # heads of 4 and 3 blocks
]


@pytest.mark.parametrize("variant", ["auto", "staged", "generic", "chained", "fused"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_static_matches_workspace_entry_point(case, variant):
    lib = L.load()
    for (E, H, N, D, B, T, pre, dt, masked) in CASES[case]:
        q, k, v = (t.to(DEV) for t in seeded_qkv(E, H, N, D, DT[dt], seed=case))
        mask = None
        if masked:
            mask = block_safe_mask(E, N, B, seed=7 + case).to(torch.uint8).to(DEV)
        try:
            ref, got = _both(lib, q, k, v, mask, T, B, pre, variant)
        except NotImplementedError as ex:
            pytest.skip(f"variant {variant}: {ex}")
        assert torch.equal(ref.view(torch.uint8), got.view(torch.uint8)), f"case {case} {variant} N={N}: outputs differ"
        want = monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None if mask is None else mask.cpu().bool(), T, B, pre)
        assert_parity(got.cpu(), want, dt, f"static case {case} {variant} N={N}")


def test_static_refuses_what_does_not_fit():
    lib = L.load()
    E, H, N, D = 1, 16, 16384, 64   # needs ~107 MiB of state
    q = torch.zeros(E, H, N, D, dtype=torch.float16, device=DEV)
    out = torch.full_like(q, float("nan"))
    p = make_params(q, q, q, None, out, 3, 128, False, "auto")
    assert lib.ma_fwd_workspace_bytes(p) > L.MA_STATIC_WORKSPACE_BYTES
    assert lib.ma_fwd_static(p, None) == L.MA_ERR_STATIC_LIMIT
    torch.cuda.synchronize()
    assert torch.isnan(out).all()   # nothing was launched
    assert "MA_STATIC_WORKSPACE_BYTES" in L.strerror(L.MA_ERR_STATIC_LIMIT)
