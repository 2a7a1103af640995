"""Parity of the HIP path (through the C ABI) with the CPU oracle and with the
committed golden vectors.  Runs on a MI355X only (``-m gpu``).

Gate: fp32 max-abs <= 1e-5; fp16/bf16 <= 2e-2 relative (max-norm and Frobenius)
plus the reference's own ``allclose(atol = rtol = 1e-2 | 5e-2)``
(ma/tests/test_ma.py:64-65).  Every variant of the library is checked; a
variant that does not support a problem must say so (NotImplementedError), it
must not fall back silently.
"""
import pytest
import torch

from helpers import (DT, assert_parity, block_safe_mask, err_metrics, golden_names, load_golden, seeded_qkv)
from ma import _hip_lib as L
from ma.ma_hip import make_params, monarch_attention_hip, monarch_matrix_hip, sync_status
from ma.monarch_attention import MonarchAttention, PadType
from oracle.ma_oracle import OracleTrace, monarch_attention_oracle, monarch_matrix_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
VARIANTS = ["generic", "staged", "fused", "resident", "chained", "auto"]


def run_hip(q, k, v, mask, T, B, pre, variant):
    try:
        out = monarch_attention_hip(q, k, v, mask, T, B, pre, variant=variant)
    except NotImplementedError as ex:
        if variant in ("auto", "generic"):
            raise
        pytest.skip(f"variant {variant}: {ex}")
    torch.cuda.synchronize()
    return out


def to_dev(*ts):
    return tuple(None if t is None else t.to(DEV) for t in ts)


# ---------------------------------------------------------------- golden vectors
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("name", golden_names())
def test_golden_vectors(name, variant):
    g = load_golden(name)
    q, k, v, mask = to_dev(g["q"], g["k"], g["v"], g["mask"])
    out = run_hip(q, k, v, mask, g["T"], g["B"], g["pre"], variant)
    assert out.shape == g["out"].shape and out.dtype == g["out"].dtype and out.is_contiguous()
    assert_parity(out.cpu(), g["out"], g["dt"], f"{name}/{variant}")


# ---------------------------------------------------------------- the reference's parameter tables, against the oracle
MATCH = [  # (E, H, N, D, B, T, pre_pad, dtype)   ma/tests/test_ma.py:34-48
    (1, 1, 16, 16, 4, 2, False, "f16"), (1, 1, 16, 16, 4, 2, True, "f16"), (1, 4, 16, 16, 8, 3, False, "f16"),
    (1, 1, 19, 16, 4, 2, False, "f16"), (1, 1, 19, 16, 4, 2, True, "f16"), (2, 4, 32, 32, 8, 2, False, "f16"),
    (2, 1, 24, 16, 8, 3, False, "f16"), (2, 4, 16, 32, 4, 2, False, "bf16"), (1, 1, 16, 32, 4, 2, True, "bf16"),
    (1, 1, 24, 16, 8, 2, False, "bf16"),
]
MASKED = [  # ma/tests/test_ma.py:70-80
    (1, 1, 16, 16, 4, 2, False, "f16"), (1, 1, 16, 16, 4, 2, True, "f16"), (1, 1, 19, 16, 4, 2, False, "f16"),
    (1, 4, 19, 16, 4, 3, True, "f16"), (1, 1, 32, 16, 8, 2, False, "f16"), (2, 4, 32, 32, 8, 2, False, "f16"),
    (1, 1, 16, 16, 4, 2, True, "bf16"), (2, 4, 16, 32, 4, 2, False, "bf16"),
]
T1 = [  # (E, H, N, D, B, pre_pad, dtype)   ma/tests/test_ma.py:105-109,125-133
    (1, 1, 16, 16, 4, False, "f16"), (2, 4, 19, 32, 8, True, "bf16"), (1, 1, 16, 16, 4, True, "f16"),
    (2, 4, 32, 32, 8, False, "f16"), (1, 1, 19, 16, 4, False, "f16"), (1, 1, 19, 16, 4, True, "f16"),
    (2, 4, 16, 32, 4, False, "bf16"),
]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt", MATCH)
def test_reference_match_table(E, H, N, D, B, T, pre, dt, variant):
    q, k, v = seeded_qkv(E, H, N, D, DT[dt])
    ref = monarch_attention_oracle(q, k, v, None, T, B, pre)
    out = run_hip(*to_dev(q, k, v), None, T, B, pre, variant)
    assert_parity(out.cpu(), ref, dt)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt", MASKED)
def test_reference_mask_table(E, H, N, D, B, T, pre, dt, variant):
    q, k, v = seeded_qkv(E, H, N, D, DT[dt])
    mask = block_safe_mask(E, N, B)
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre)
    out = run_hip(*to_dev(q, k, v, mask), T, B, pre, variant)
    assert not torch.isnan(out).any()
    assert_parity(out.cpu(), ref, dt)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("E,H,N,D,B,pre,dt", T1)
def test_reference_t1_table(E, H, N, D, B, pre, dt, variant):
    q, k, v = seeded_qkv(E, H, N, D, DT[dt])
    ref = monarch_attention_oracle(q, k, v, None, 1, B, pre)
    out = run_hip(*to_dev(q, k, v), None, 1, B, pre, variant)
    assert out.shape == (E, H, N, D)
    assert_parity(out.cpu(), ref, dt)


# ---------------------------------------------------------------- benchmark configurations (reduced batch where the CPU oracle is slow)
CONFIGS = [  # name, E, H, N, D, B, T, pre, dt, scale
    ("c1", 1, 1, 256, 64, 16, 1, False, "f32", 1.0),
    ("c2a_pre", 4, 12, 197, 64, 16, 2, True, "f16", 0.125),
    ("c2a_post", 4, 12, 197, 64, 16, 2, False, "f16", 0.125),
    ("c2b", 4, 12, 256, 64, 16, 2, False, "f16", 0.125),
    ("c3", 4, 12, 512, 64, 32, 2, False, "bf16", 1.0),
    ("c4", 2, 16, 1024, 72, 32, 3, False, "f16", 1.0),
    ("cM_T1", 1, 16, 4096, 64, 64, 1, False, "f16", 1.0),
    ("cM_T2", 1, 16, 4096, 64, 64, 2, False, "f16", 1.0),
    ("cM_T3", 1, 16, 4096, 64, 64, 3, False, "f16", 1.0),
    ("c5", 1, 4, 16384, 64, 128, 3, False, "f16", 1.0),
    ("c3_f32", 1, 4, 512, 64, 32, 2, False, "f32", 1.0),
    ("bart8k", 1, 2, 8192, 64, 64, 2, False, "bf16", 1.0),
    ("gps", 1, 2, 7600, 48, 128, 2, False, "f32", 1.0),
    ("vit_b14", 2, 12, 197, 64, 14, 2, True, "f16", 0.125),
    ("roberta_b24", 2, 12, 384, 64, 24, 1, False, "f16", 1.0),
    ("b48_m40", 2, 4, 1900, 64, 48, 2, False, "f16", 1.0),         # 3-strip problems in both kinds of phases
    ("b96_m90", 1, 2, 8600, 64, 96, 2, True, "bf16", 1.0),         # 6-strip problems (per-stage launches; 8-strip class in one launch)
    ("b40_m6_d72", 2, 3, 230, 72, 40, 3, False, "f16", 1.0),       # 3 strips of keys, one of blocks, head dim 72
    ("big_block", 1, 2, 600, 64, 200, 2, False, "f16", 1.0),       # B > 128: the 16-strip class of the stage kernels (AUTO -> staged)
    ("many_blocks", 1, 2, 4096, 32, 16, 2, False, "bf16", 1.0),    # M = 256 > 128: likewise, 16 strips of blocks
    ("one_block", 2, 2, 100, 64, 128, 3, True, "f16", 1.0),        # M = 1: dense softmax attention
    ("unit_blocks", 1, 2, 96, 32, 1, 1, False, "f16", 1.0),        # B = 1, M = N
    ("many_heads", 40, 64, 64, 32, 16, 2, False, "f16", 1.0),      # more heads than co-resident workgroups
    ("many_heads_odd", 3, 7, 80, 32, 16, 3, True, "bf16", 1.0),    # odd head count, ragged N
]


_ORACLE_CACHE = {}


def _config_case(name, E, H, N, D, B, T, pre, dt, scale):
    """Seeded inputs and the oracle's output for a named configuration (the
    oracle runs once per configuration, not once per variant)."""
    if name not in _ORACLE_CACHE:
        q, k, v = seeded_qkv(E, H, N, D, DT[dt], scale=scale)
        _ORACLE_CACHE[name] = (q, k, v, monarch_attention_oracle(q, k, v, None, T, B, pre, upcast=True))
    return _ORACLE_CACHE[name]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("name,E,H,N,D,B,T,pre,dt,scale", CONFIGS)
def test_benchmark_shapes_against_oracle(name, E, H, N, D, B, T, pre, dt, scale, variant):
    q, k, v, ref = _config_case(name, E, H, N, D, B, T, pre, dt, scale)
    out = run_hip(*to_dev(q, k, v), None, T, B, pre, variant)
    assert_parity(out.cpu(), ref, dt, f"{name}/{variant}")


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("B", [24, 48, 96, 128])
def test_roberta_block_sizes_with_tokenizer_mask(B, variant):
    """The block sizes the reference's RoBERTa evaluation sweeps (experiments/roberta/benchmark.py:67-89):
    N = 384 (max_length padding), T = 1, post-pad, the tokenizer's int64 attention mask with the tail
    of every sequence masked out."""
    E, H, N, D, T = 3, 12, 384, 64, 1
    q, k, v = seeded_qkv(E, H, N, D, torch.float16, seed=B)
    lengths = torch.tensor([384, 201, 77])
    mask = (torch.arange(N)[None] < lengths[:, None]).long()
    ref = monarch_attention_oracle(q, k, v, mask != 0, T, B, False, upcast=True)
    out = run_hip(*to_dev(q, k, v, mask), T, B, False, variant)
    assert_parity(out.cpu(), ref, "f16", f"roberta B={B}/{variant}")


FEW_BLOCKS = [  # E, H, N, D, B, T, pre, dt, masked: 1, 2, 3, 4, 5, 7 and 8 blocks per head, ragged last blocks
    (2, 3, 90, 32, 90, 2, False, "f16", False), (1, 2, 100, 64, 64, 2, True, "bf16", True),
    (2, 2, 384, 64, 128, 1, False, "f16", True), (1, 4, 512, 64, 128, 2, False, "f16", False),
    (1, 2, 333, 40, 67, 3, True, "f16", True), (2, 1, 140, 128, 20, 2, False, "bf16", False),
    (1, 12, 512, 64, 64, 2, False, "bf16", True), (1, 2, 17, 16, 3, 2, True, "f16", False),
]


@pytest.mark.parametrize("variant", ["staged", "chained", "auto"])
@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked", FEW_BLOCKS)
def test_heads_of_few_blocks(E, H, N, D, B, T, pre, dt, masked, variant):
    """At most 8 blocks per head: the per-stage and chained L and Z problems lay 16, 8, 4 or 2 in-block
    positions side by side in one 16-row tile and keep them apart with a block-diagonal mask."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    out = run_hip(*to_dev(q, k, v, mask), T, B, pre, variant)
    assert_parity(out.cpu(), ref, dt, f"few blocks {(E, H, N, D, B, T, pre, dt, masked)}/{variant}")


LARGE_TILES = [  # E, H, N, D, B, T, pre, dt, masked: blocks and / or block counts of 129 .. 256 rows
    (1, 2, 4096, 64, 256, 2, False, "f16", False), (2, 1, 3000, 64, 20, 2, True, "bf16", True),       # one side only
    (1, 2, 2100, 72, 130, 3, False, "f16", True), (1, 3, 2571, 32, 150, 1, True, "f16", False),
    (1, 1, 32768, 64, 181, 2, False, "f16", False), (1, 1, 40000, 128, 200, 2, True, "bf16", True),   # both sides
    (1, 1, 65536, 64, 256, 1, False, "bf16", False), (1, 2, 20000, 40, 129, 3, False, "f16", True),
]


@pytest.mark.parametrize("variant", ["staged", "auto"])
@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked", LARGE_TILES)
def test_blocks_and_block_counts_up_to_256(E, H, N, D, B, T, pre, dt, masked, variant):
    """Heads of up to 65536 tokens: block problems of 129 .. 256 rows run in the stage kernels' 16-strip
    class; AUTO must pick those kernels (not the FMA path), the one-launch variants must refuse."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    out = run_hip(*dev, T, B, pre, variant)
    assert_parity(out.cpu(), ref, dt, f"large tiles {(E, H, N, D, B, T, pre, dt, masked)}/{variant}")
    if variant == "auto":
        for other in ("fused", "chained", "resident"):
            with pytest.raises(NotImplementedError):
                monarch_attention_hip(*dev, T, B, pre, variant=other)


TEAM_SHAPES = [  # E, H, N, D, B, T, pre, dt, masked: 8 or 16 heads whose phases fill the device, more than one step
    (1, 8, 8000, 64, 64, 2, True, "f16", True), (1, 8, 8192, 72, 128, 3, False, "f16", False),
    (1, 16, 4096, 64, 32, 2, False, "bf16", True), (2, 4, 5000, 32, 128, 3, True, "f16", True),
    (1, 16, 4000, 64, 128, 2, True, "bf16", False), (1, 8, 4096, 80, 64, 2, False, "f16", True),
]


@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked", TEAM_SHAPES)
def test_few_long_heads_run_in_the_team_kernel(E, H, N, D, B, T, pre, dt, masked, monkeypatch):
    """For a caller that owns the device (MA_FLAG_DEVICE_EXCLUSIVE; the module's DEVICE_EXCLUSIVE switch) AUTO
    sends 8 or 16 heads of 64 .. 128 tasks per phase to the team kernel when T > 1 (teams larger than the
    workgroups the device holds per head loop over their tasks): parity, and the bounded waits all met.
    Without that statement the same call stays away from the team kernel and gives the same result to tolerance."""
    from ma import ma_hip
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    out = torch.empty_like(dev[2])
    p = make_params(*dev[:3], None, out, T, B, pre, "auto")
    assert L.VARIANT_NAMES[L.load().ma_fwd_select_variant(p)] in ("chained", "staged")
    p.flags = L.MA_FLAG_DEVICE_EXCLUSIVE
    assert L.VARIANT_NAMES[L.load().ma_fwd_select_variant(p)] == "fused"
    shared = monarch_attention_hip(*dev, T, B, pre, variant="auto")
    monkeypatch.setattr(ma_hip, "DEVICE_EXCLUSIVE", True)
    got = monarch_attention_hip(*dev, T, B, pre, variant="auto")
    fused = monarch_attention_hip(*dev, T, B, pre, variant="fused")
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.uint8), fused.view(torch.uint8)), "with DEVICE_EXCLUSIVE 'auto' must run the team kernel"
    assert_parity(got.cpu(), ref, dt, f"team shapes {(E, H, N, D, B, T, pre, dt, masked)}")
    assert_parity(shared.cpu(), ref, dt, f"team shapes, shared device {(E, H, N, D, B, T, pre, dt, masked)}")
    assert sync_status() == 0


TWO_TILE = [  # E, H, N, D, B, T, pre, dt, masked: heads too long for Q, K, V and the state in LDS, short enough for the state and one input tile
    (2, 3, 512, 64, 32, 2, False, "bf16", False), (1, 4, 500, 64, 32, 3, True, "f16", True),
    (1, 2, 384, 64, 24, 1, False, "f16", True), (2, 2, 448, 64, 16, 2, True, "bf16", False),
    (1, 3, 300, 72, 20, 2, False, "f16", True), (1, 2, 900, 32, 32, 2, False, "f16", False),
    (1, 2, 512, 64, 64, 2, False, "f16", True), (1, 2, 384, 64, 48, 2, True, "bf16", False),
    (1, 2, 272, 128, 16, 3, False, "f16", True), (1, 2, 480, 40, 27, 1, True, "bf16", True), (1, 1, 300, 64, 10, 2, False, "f16", False),
    (30, 12, 400, 64, 25, 2, False, "f16", True),   # more heads than workgroups: a workgroup walks several heads
    (16, 12, 512, 64, 32, 2, False, "bf16", False), (16, 16, 512, 64, 32, 1, True, "f16", True),   # what 'auto' sends there
]

PACKED = [  # E, H, N, D, B, T, pre, dt, masked, kernel: more short heads than compute units: a head-resident form in workgroups of 8 or 4 waves
    # four tiles (head dims of up to 80, heads whose four tiles fit half or a quarter of the LDS)
    (65, 4, 64, 64, 16, 1, False, "f16", False, "resident_head_mfma"), (130, 6, 64, 64, 16, 2, True, "bf16", True, "resident_head_mfma"),
    (200, 4, 96, 32, 16, 3, False, "f16", True, "resident_head_mfma"), (80, 4, 90, 40, 30, 1, True, "bf16", True, "resident_head_mfma"),
    (200, 4, 64, 32, 32, 2, False, "f16", False, "resident_head_mfma"), (210, 4, 100, 32, 5, 2, True, "f16", True, "resident_head_mfma"),
    (300, 4, 33, 64, 11, 3, False, "bf16", True, "resident_head_mfma"), (300, 4, 96, 64, 16, 2, False, "f16", True, "resident_head_mfma"),
    (100, 4, 128, 32, 32, 1, True, "bf16", False, "resident_head_mfma"), (70, 4, 80, 72, 16, 3, False, "f16", True, "resident_head_mfma"),
    (200, 4, 40, 80, 8, 2, True, "f16", False, "resident_head_mfma"),
    # two tiles (longer heads, and every head dim above 80)
    (70, 4, 197, 64, 16, 2, False, "f16", True, "resident_head2_mfma"), (192, 4, 197, 64, 16, 2, True, "f16", False, "resident_head2_mfma"),   # (the second: the ViT shape)
    (66, 4, 100, 72, 10, 2, False, "f16", True, "resident_head2_mfma"), (65, 4, 60, 128, 12, 3, True, "bf16", True, "resident_head2_mfma"),
    (260, 4, 50, 128, 10, 1, False, "f16", False, "resident_head2_mfma"), (65, 5, 130, 48, 26, 2, False, "f16", True, "resident_head2_mfma"),
]

ONE_TILE = [  # heads beyond that whose aL / aR / Y do not fit in LDS as three (or two) tiles either
    (1, 2, 1000, 32, 32, 2, False, "f16", False), (2, 3, 768, 64, 32, 2, False, "bf16", True), (1, 2, 640, 64, 40, 3, True, "f16", True),
    (1, 2, 600, 64, 64, 1, False, "f16", False), (1, 3, 420, 72, 30, 2, True, "bf16", True),
    (30, 12, 700, 64, 28, 2, False, "f16", True),   # more heads than workgroups
]


def resident_kernel_name(dev, T, B, pre):
    p = make_params(*dev[:3], dev[3], torch.empty_like(dev[2]), T, B, pre, "resident")
    return L.load().ma_fwd_kernel_name(p).decode()


@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked", TWO_TILE)
def test_resident_kernel_with_the_state_and_one_input_tile(E, H, N, D, B, T, pre, dt, masked):
    """Heads of ~260 .. 540 tokens (D = 64) in the resident kernel: the state tile and one input tile in LDS, the
    tile swapped at every phase boundary, V and Y in place of the K rows in the last R phase."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    assert resident_kernel_name(dev, T, B, pre) == "resident_head2_mfma"
    out = monarch_attention_hip(*dev, T, B, pre, variant="resident")   # the variant must take these shapes
    assert_parity(out.cpu(), ref, dt, f"two-tile resident {(E, H, N, D, B, T, pre, dt, masked)}")
    again = monarch_attention_hip(*dev, T, B, pre, variant="resident")
    assert torch.equal(out, again)
    if E * H >= 192:
        auto = monarch_attention_hip(*dev, T, B, pre, variant="auto")
        p = make_params(*dev[:3], dev[3], torch.empty_like(dev[2]), T, B, pre, "auto")
        assert L.VARIANT_NAMES[L.load().ma_fwd_select_variant(p)] == "resident"
        assert torch.equal(out, auto)


@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked,kernel", PACKED)
def test_resident_kernel_in_narrow_workgroups(E, H, N, D, B, T, pre, dt, masked, kernel):
    """Many short heads: the head-resident forms of the resident kernel in workgroups of 4 or 8 waves that share a
    compute unit (and walk several heads each)."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    assert resident_kernel_name(dev, T, B, pre) == kernel
    out = monarch_attention_hip(*dev, T, B, pre, variant="resident")
    assert_parity(out.cpu(), ref, dt, f"narrow-workgroup resident {(E, H, N, D, B, T, pre, dt, masked)}")
    again = monarch_attention_hip(*dev, T, B, pre, variant="resident")
    assert torch.equal(out, again)


@pytest.mark.parametrize("E,H,N,D,B,T,pre,dt,masked", ONE_TILE)
def test_resident_kernel_with_one_state_tile(E, H, N, D, B, T, pre, dt, masked):
    """Heads of ~550 .. 1000 tokens in the resident kernel: aL and aR share one LDS tile in place, the inputs are
    streamed and Y goes through the workspace."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    assert resident_kernel_name(dev, T, B, pre) == "resident_fwd_mfma"
    out = monarch_attention_hip(*dev, T, B, pre, variant="resident")   # the variant must take these shapes
    assert_parity(out.cpu(), ref, dt, f"one-tile resident {(E, H, N, D, B, T, pre, dt, masked)}")
    again = monarch_attention_hip(*dev, T, B, pre, variant="resident")
    assert torch.equal(out, again)


SMALL_F32 = [  # E, H, N, D, B, T, pre, masked: fp32 heads of at most 16 blocks of at most 16 rows
    (1, 1, 256, 64, 16, 1, False, False),      # the reference's CPU-sized case
    (2, 3, 197, 64, 16, 1, True, True), (1, 4, 100, 32, 8, 1, False, True), (3, 2, 250, 48, 16, 1, True, False),   # a single step, few heads
    (2, 2, 37, 20, 5, 1, False, True), (1, 2, 16, 64, 16, 1, False, False), (1, 2, 33, 4, 3, 1, True, True), (1, 16, 241, 64, 16, 1, False, True),
    (4, 5, 197, 64, 16, 1, False, True),       # ... 320 workgroups would be too many: the one-workgroup-per-head kernel
    (1, 1, 256, 64, 16, 3, True, True), (2, 3, 197, 64, 16, 2, True, True), (1, 4, 100, 32, 8, 3, False, True),
    (3, 2, 250, 48, 16, 2, True, False), (2, 2, 37, 20, 5, 2, False, True), (1, 2, 16, 64, 16, 2, False, False),
    (1, 3, 49, 64, 7, 1, True, True), (1, 2, 33, 4, 3, 2, False, False), (40, 8, 197, 64, 16, 2, False, True),   # 320 heads: workgroups walk several
]


@pytest.mark.parametrize("E,H,N,D,B,T,pre,masked", SMALL_F32)
def test_small_fp32_heads_in_one_launch(E, H, N, D, B, T, pre, masked):
    """fp32 heads of up to 256 tokens run whole in one workgroup each (variant 'resident', what 'auto' picks from
    64 heads on and for very small heads): parity with the oracle at the fp32 gate, and - the arithmetic being
    that of the fp32 stage kernels, operation for operation - bit-identical to the per-stage launches."""
    q, k, v = seeded_qkv(E, H, N, D, torch.float32, seed=N + B)
    mask = block_safe_mask(E, N, B, seed=B) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre)
    dev = to_dev(q, k, v, mask)
    out = monarch_attention_hip(*dev, T, B, pre, variant="resident")   # the variant must take these shapes
    staged = monarch_attention_hip(*dev, T, B, pre, variant="staged")
    auto = monarch_attention_hip(*dev, T, B, pre, variant="auto")
    torch.cuda.synchronize()
    assert_parity(out.cpu(), ref, "f32", f"fp32 head kernel {(E, H, N, D, B, T, pre, masked)}")
    assert_parity(auto.cpu(), ref, "f32", f"fp32 auto {(E, H, N, D, B, T, pre, masked)}")
    p = make_params(*dev[:3], None, torch.empty_like(dev[2]), T, B, pre, "resident")
    single_step = L.load().ma_fwd_kernel_name(p) == b"head_t1_f32"
    assert single_step == (T == 1 and E * H * B <= 256)
    if single_step:   # few heads, one step: a workgroup per (head, position) with plain FMAs - the sums run in another order
        assert torch.allclose(out, staged, atol=2e-6, rtol=1e-5)
    else:
        assert torch.equal(out.view(torch.int32), staged.view(torch.int32)), "differs from the per-stage fp32 kernels"
    for shape, why in (((1, 2, 272, 64, 16), "17 blocks"), ((1, 2, 64, 64, 32), "32-row blocks"), ((1, 2, 64, 80, 16), "head dim 80")):
        e, h, n, d, b = shape
        x = torch.zeros(e, h, n, d, device=DEV)
        with pytest.raises(NotImplementedError):
            monarch_attention_hip(x, x, x, None, 1, b, False, variant="resident")


def test_broadcast_over_tokens_is_accepted():
    """expand()-ed inputs (stride 0 along N) are legal for the reference (it pads, i.e. copies); the
    operator takes them too, by making the one copy the library's row-overlap check asks for."""
    E, H, N, D, B, T = 1, 2, 64, 32, 16, 2
    q, k, v = seeded_qkv(E, H, N, D, torch.float16)
    kx = k[:, :, :1].expand(E, H, N, D)
    ref = monarch_attention_oracle(q, kx, v, None, T, B, False, upcast=True)
    qd, kd, vd = to_dev(q, k, v)
    out = run_hip(qd, kd[:, :, :1].expand(E, H, N, D), vd, None, T, B, False, "auto")
    assert_parity(out.cpu(), ref, "f16")


# ---------------------------------------------------------------- stage-level parity (workspace state against the oracle trace)
def _stage_setup(E, H, N, D, Dv, B, T, pre, dt, vdt, variant, with_mask):
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], Dv=Dv)
    v = v.to(DT[vdt])
    mask = block_safe_mask(E, N, B) if with_mask else None
    tr = OracleTrace()
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, trace=tr)
    lib = L.load()
    qd, kd, vd, md = to_dev(q, k, v, mask)
    m8 = None if md is None else (md != 0).to(torch.uint8)
    out = torch.zeros(E, H, N, Dv, dtype=DT[vdt], device=DEV)
    p = make_params(qd, kd, vd, m8, out, T, B, pre, variant)
    lay = L.WsLayout()
    L.check(lib.ma_fwd_workspace_layout(p, lay), "layout")
    ws = torch.zeros(lay.total, dtype=torch.uint8, device=DEV)
    p.workspace, p.workspace_bytes = ws.data_ptr(), lay.total
    keep = (qd, kd, vd, m8, out, ws)
    M = -(-N // B)

    def view(off, shape, dtype):
        n = 1
        for s in shape:
            n *= s
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        return ws[off:off + nbytes].view(dtype).view(*shape)

    state = dict(aR=view(lay.aR, (E, H, M, B, D), DT[dt]), cR=view(lay.cR, (E, H, M, B), torch.float32),
                 aL=view(lay.aL, (E, H, B, M, D), DT[dt]), cL=view(lay.cL, (E, H, B, M), torch.float32),
                 Y=view(lay.Y, (E, H, B, M, Dv), DT[vdt]))
    return lib, p, state, tr, ref, out, keep


def _call(fn, *args):
    st = fn(*args)
    if st == L.MA_ERR_UNSUPPORTED:
        pytest.skip("variant does not expose stage entry points for this problem")
    L.check(st, "stage")
    torch.cuda.synchronize()


STAGE_CASES = [  # E,H,N,D,Dv,B,T,pre,dt,vdt,mask
    (1, 2, 64, 16, 16, 8, 3, False, "f32", "f32", False),
    (2, 2, 50, 16, 24, 8, 3, True, "f32", "f32", True),
    (1, 2, 128, 64, 64, 16, 2, False, "f16", "f16", False),
    (1, 2, 197, 64, 64, 16, 3, True, "f16", "f16", True),
    (1, 2, 256, 64, 64, 32, 2, False, "bf16", "bf16", False),
    (1, 1, 1024, 64, 64, 64, 2, False, "f16", "f16", False),
    (1, 2, 40, 32, 40, 8, 2, False, "f16", "f32", False),
    # heads of 1..8 blocks: the 16-bit L and Z kernels put several in-block positions into one tile
    (1, 2, 200, 64, 64, 64, 2, True, "f16", "f16", True),
    (2, 2, 250, 32, 32, 96, 3, False, "bf16", "bf16", True),
    (1, 2, 100, 64, 64, 100, 2, False, "f16", "f16", False),
    (1, 3, 130, 40, 40, 20, 2, True, "f16", "f16", False),
    (1, 2, 45, 72, 72, 27, 2, False, "bf16", "bf16", False),
    # blocks / block counts of 129 .. 256 rows: the 16-strip tile class (four strips per wave)
    (1, 2, 3000, 64, 64, 200, 2, True, "f16", "f16", True),
    (1, 1, 2600, 32, 32, 20, 2, False, "bf16", "bf16", False),
    (1, 1, 33000, 64, 64, 180, 2, False, "f16", "f16", True),
]


@pytest.mark.parametrize("variant", ["generic", "staged"])
@pytest.mark.parametrize("E,H,N,D,Dv,B,T,pre,dt,vdt,with_mask", STAGE_CASES)
def test_stages_against_oracle_trace(E, H, N, D, Dv, B, T, pre, dt, vdt, with_mask, variant):
    lib, p, st, tr, ref, out, keep = _stage_setup(E, H, N, D, Dv, B, T, pre, dt, vdt, variant, with_mask)
    tol = dict(f32=(2e-6, 1e-5), f16=(2e-3, 4e-3), bf16=(1.6e-2, 3e-2))[dt]

    def close(got, want, what, scale=1.0):
        want = want.to(DEV)
        assert torch.allclose(got.float(), want.float(), atol=tol[0] * scale, rtol=tol[1]), \
            (what, err_metrics(got, want))

    # every stage is fed the ORACLE's inputs so that differences do not compound
    for t, step in enumerate(tr.steps):
        last = t == len(tr.steps) - 1
        if t > 0:
            st["aR"].copy_(step["aR"].to(DEV))
            st["cR"].copy_(step["cR"].to(DEV))
        _call(lib.ma_r_step, p, int(t == 0), int(last), None)
        close(st["aL"], step["aL"], f"aL[{t}]")
        close(st["cL"], step["cL"], f"cL[{t}]", scale=10.0)
        if last:
            vt = dict(f32=1.0, f16=1.0, bf16=1.0)[vdt]
            close(st["Y"], step["Y"], "Y", scale=vt if vdt == dt else 1000.0)
            break
        st["aL"].copy_(step["aL"].to(DEV))
        st["cL"].copy_(step["cL"].to(DEV))
        _call(lib.ma_l_step, p, None)
        nxt = tr.steps[t + 1]
        close(st["cR"], nxt["cR"], f"cR[{t}]", scale=10.0)
        # aR rows scale with cR; compare on that scale
        close(st["aR"], nxt["aR"], f"aR[{t}]", scale=4.0)
    st["aL"].copy_(tr.steps[-1]["aL"].to(DEV))
    st["cL"].copy_(tr.steps[-1]["cL"].to(DEV))
    st["Y"].copy_(tr.steps[-1]["Y"].to(DEV))
    _call(lib.ma_z_step, p, None)
    assert_parity(out.cpu(), ref, dt if dt == vdt else dt, "Z")


def test_empty_and_invalid_inputs_raise():
    q = torch.empty(1, 2, 0, 64, dtype=torch.float16, device=DEV)
    with pytest.raises(ValueError):
        monarch_attention_hip(q, q, q, None, 1, 16, False)
    q, k, v = to_dev(*seeded_qkv(1, 2, 32, 64, torch.float16))
    with pytest.raises(ValueError):
        monarch_attention_hip(q, k, v, None, 1, 16, False, variant="nope")
    with pytest.raises(NotImplementedError):                 # fp32 has stage kernels only: no silent fallback
        monarch_attention_hip(q.float(), k.float(), v.float(), None, 1, 16, False, variant="chained")
    with pytest.raises(NotImplementedError):                 # an fp32 V with fp16 q / k is for the generic kernels
        monarch_attention_hip(q, k, v.float(), None, 1, 16, False, variant="staged")


def test_workspace_is_shared_across_shapes_and_calls():
    """One cached workspace serves calls of different shapes back to back (the
    fused kernels' barrier epochs continue across launches)."""
    outs = []
    shapes = [(1, 16, 1024, 64, 64, 2), (2, 40, 128, 64, 16, 3), (1, 2, 2048, 64, 32, 1), (1, 16, 1024, 64, 64, 2)]
    for rep in range(3):
        for (E, H, N, D, B, T) in shapes:
            q, k, v = seeded_qkv(E, H, N, D, torch.float16)
            ref = monarch_attention_oracle(q, k, v, None, T, B, False, upcast=True)
            for variant in ("fused", "chained", "staged"):
                out = run_hip(*to_dev(q, k, v), None, T, B, False, variant)
                assert_parity(out.cpu(), ref, "f16", f"rep{rep}/{variant}/{(E, H, N, B, T)}")
    assert sync_status() == 0   # no wait between workgroups ever ran out


@pytest.mark.parametrize("E,H,N,D,B,T", [(1, 16, 1024, 64, 64, 2), (3, 7, 197, 64, 16, 3), (2, 40, 128, 32, 16, 1)])
def test_chained_kernel_leaves_its_flags_cleared(E, H, N, D, B, T):
    """Through the C ABI on a caller-owned workspace: after a chained forward
    every flag word and per-head counter of the kernel is zero again (what
    MA_FLAG_SYNC_READY promises for the next call), the error word is zero (no
    wait timed out, every producer ran on its consumers' XCD), and a second call
    on the same workspace gives the same bits."""
    lib = L.load()
    q, k, v = to_dev(*seeded_qkv(E, H, N, D, torch.float16))
    out = torch.zeros(E, H, N, D, dtype=torch.float16, device=DEV)
    p = make_params(q, k, v, None, out, T, B, False, "chained")
    lay = L.WsLayout()
    L.check(lib.ma_fwd_workspace_layout(p, lay), "layout")
    ws = torch.zeros(lay.total, dtype=torch.uint8, device=DEV)
    p.workspace, p.workspace_bytes, p.flags = ws.data_ptr(), lay.total, L.MA_FLAG_SYNC_READY
    sync_bytes = lay.aR - lay.sync                      # the sync area ends where the first state array starts
    chain_bytes = 4 * 256 * 1024                        # the chained kernel's flag words are its last megabyte
    outs = []
    for _ in range(2):
        L.check(lib.ma_fwd(p, None), "ma_fwd")
        torch.cuda.synchronize()
        words = ws[lay.sync:lay.sync + sync_bytes].view(torch.int32)
        assert int(words[1]) == 0, "sync error word raised"
        assert not words[-chain_bytes // 4 - 64:].any(), "chained kernel left flags behind"
        outs.append(out.clone())
    assert torch.equal(outs[0], outs[1])
    ref = monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False, upcast=True)
    assert_parity(outs[0].cpu(), ref, "f16")


# ---------------------------------------------------------------- caller-side layouts and masks
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_permuted_views_as_models_pass_them(dt, variant):
    """(E,H,N,D) views of an (E,N,H,D) buffer, as every model in the reference
    passes them (experiments/vit/model.py:73-79)."""
    E, H, N, D, B, T = 2, 3, 197, 64, 16, 2
    g = torch.Generator().manual_seed(0)
    buf = [(0.2 * torch.randn(E, N, H, D, generator=g)).to(DT[dt]) for _ in range(3)]
    q, k, v = (b.permute(0, 2, 1, 3) for b in buf)
    assert not q.is_contiguous()
    ref = monarch_attention_oracle(q, k, v, None, T, B, True, upcast=True)
    qd, kd, vd = (b.to(DEV).permute(0, 2, 1, 3) for b in buf)
    out = run_hip(qd, kd, vd, None, T, B, True, variant)
    assert_parity(out.cpu(), ref, dt)
    assert torch.equal(qd.cpu(), q)       # inputs are not modified
    # the output follows v's layout, so the model's permute(0, 2, 1, 3).contiguous() copies nothing
    back = out.permute(0, 2, 1, 3)
    assert back.is_contiguous() and back.contiguous().data_ptr() == out.data_ptr()


@pytest.mark.parametrize("variant", VARIANTS)
def test_broadcast_keys_and_values(variant):
    """k and v shared by all heads and batch entries (expanded views, stride 0):
    read in place, same result as with materialised copies."""
    E, H, N, D, B, T = 2, 6, 160, 64, 32, 2
    q, k, v = seeded_qkv(E, H, N, D, torch.float16)
    k1, v1 = k[:1, :1], v[:1, :1]
    ref = monarch_attention_oracle(q, k1.expand(E, H, N, D).contiguous(), v1.expand(E, H, N, D).contiguous(), None, T, B, False,
                                   upcast=True)
    qd, kd, vd = to_dev(q, k1, v1)
    out = run_hip(qd, kd.expand(E, H, N, D), vd.expand(E, H, N, D), None, T, B, False, variant)
    assert_parity(out.cpu(), ref, "f16")


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("kind", ["bool", "uint8", "int16", "int32", "int64", "float16", "bfloat16", "float32", "float64"])
def test_mask_dtypes(kind, variant):
    """The mask is read in place by the kernels, whatever its element type: truthy = keep, the way
    torch.logical_and sees it (ma/ma_torch.py:98) - for floats -0.0 is false and NaN is true, for
    wide integers a value with only high bits set is true.  Callers pass int64 tokenizer masks
    (experiments/roberta/model.py:104-106) and float masks (experiments/bart/model.py:145-147)."""
    E, H, N, D, B, T = 2, 2, 384, 64, 32, 2
    q, k, v = seeded_qkv(E, H, N, D, torch.float16)
    keep = torch.arange(N)[None] < torch.tensor([N, N - 131])[:, None]
    dt = getattr(torch, kind)
    mask = keep.to(dt)
    if dt.is_floating_point:
        mask[0, 5], mask[1, 7] = float("nan"), 0.25           # kept
        mask[1, N - 100] = -0.0                                 # dropped, although its bits are not zero
    elif kind == "int64":
        mask[0, 5], mask[1, 7] = 1 << 40, -(1 << 35)           # kept: only high bits set
    elif kind in ("int16", "int32"):
        mask[0, 5], mask[1, 7] = -2, 1 << 9
    ref = monarch_attention_oracle(q, k, v, mask != 0, T, B, False, upcast=True)
    out = run_hip(*to_dev(q, k, v, mask), T, B, False, variant)
    assert_parity(out.cpu(), ref, "f16")
    # the same mask as a strided view (every other element of a wider buffer), still without a copy
    wide = torch.zeros(E, 2 * N, dtype=dt)
    wide[:, ::2] = mask
    qd, kd, vd, wd = to_dev(q, k, v, wide)
    out2 = run_hip(qd, kd, vd, wd[:, ::2], T, B, False, variant)
    assert torch.equal(out2.view(torch.uint8), out.view(torch.uint8))


@pytest.mark.parametrize("variant", VARIANTS)
def test_dead_key_block_gives_no_nan(variant):
    E, H, N, D, B, T = 1, 2, 256, 64, 32, 2
    q, k, v = seeded_qkv(E, H, N, D, torch.float16)
    mask = torch.ones(E, N, dtype=torch.bool)
    mask[:, 64:96] = False
    ref = monarch_attention_oracle(q, k, v, mask, T, B, False, upcast=True)
    out = run_hip(*to_dev(q, k, v, mask), T, B, False, variant)
    assert torch.isfinite(out.float()).all()
    assert_parity(out.cpu(), ref, "f16")


@pytest.mark.parametrize("D", [40, 72, 80])
def test_state_in_lds_ignores_what_earlier_kernels_left_there(D):
    """Head dims that do not fill their 32-column MFMA tiles (D = 40, 72, 80):
    the columns between the written width of a state row and the tile width must
    read as zero whatever used the LDS before - fp32 kernels leave bit patterns
    there that are NaN as fp16.  Alternates the fp32 kernels with the
    state-in-LDS kernel on many heads so that every CU has run both."""
    E, H, N, B, T = 8, 64, 128, 32, 3
    q, k, v = seeded_qkv(E, H, N, D, torch.float16)
    ref = monarch_attention_oracle(q[:1, :4], k[:1, :4], v[:1, :4], None, T, B, False, upcast=True)
    dq, dk, dv = to_dev(q, k, v)
    big = [t.float() * 3e4 for t in (dq, dk, dv)]   # fp32 run whose LDS contents are large / non-fp16 patterns
    for _ in range(3):
        monarch_attention_hip(*big, None, 1, B, False, variant="generic")
        out = run_hip(dq, dk, dv, None, T, B, False, "resident")
        assert torch.isfinite(out.float()).all()
        assert_parity(out[:1, :4].cpu(), ref, "f16")


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_get_matrix_through_the_module(dt):
    E, H, N, D, B, T = 1, 2, 96, 32, 16, 2
    q, k, _ = seeded_qkv(E, H, N, D, DT[dt])
    mod = MonarchAttention(B, T, PadType.post)
    A = mod.get_matrix(q.to(DEV), k.to(DEV))
    ref = monarch_matrix_oracle(q, k, None, T, B, False)
    assert A.dtype == torch.float32 and A.shape == (E, H, N, N)
    assert_parity(A.cpu(), ref, dt)
    assert torch.allclose(A.sum(-1).cpu(), torch.ones(E, H, N), atol=5e-3)


# ---------------------------------------------------------------- dense matrix, written directly
MATRIX_CASES = [  # E, H, N, D, B, T, pre, dt, masked
    (1, 2, 96, 32, 16, 1, False, "f32", False), (2, 3, 96, 32, 16, 2, False, "f16", True),
    (1, 2, 197, 64, 14, 2, True, "f16", False), (2, 1, 61, 24, 7, 3, True, "f32", True),
    (1, 2, 300, 40, 32, 3, False, "bf16", True), (1, 1, 5, 4, 8, 2, False, "f32", False),
    (1, 1, 1000, 64, 4, 2, True, "f16", False),
]


@pytest.mark.parametrize("case", MATRIX_CASES, ids=lambda c: "-".join(map(str, c)))
def test_matrix_kernel_equals_forward_on_identity(case):
    """ma_matrix against what it replaces, the forward pass on an fp32 identity
    (reference get_matrix): with the FMA kernels for the T steps every entry is
    the same single product, so the two agree bit for bit; with the MFMA
    kernels for the steps they agree within the dtype's gate.  Both are checked
    against the oracle as well."""
    E, H, N, D, B, T, pre, dt, masked = case
    q, k, _ = seeded_qkv(E, H, N, D, DT[dt])
    mask = block_safe_mask(E, N, B, seed=N) if masked else None
    dq, dk, dm = to_dev(q, k, mask)
    eye = torch.eye(N, device=DEV).expand(E, H, N, N)
    via_identity = monarch_attention_hip(dq, dk, eye, dm, T, B, pre, variant="generic")
    A = monarch_matrix_hip(dq, dk, dm, T, B, pre, variant="generic")
    assert A.shape == (E, H, N, N) and A.dtype == torch.float32 and A.is_contiguous()
    assert torch.equal(A, via_identity)
    ref = monarch_matrix_oracle(q, k, mask, T, B, pre)
    assert_parity(A.cpu(), ref, dt)
    A2 = monarch_matrix_hip(dq, dk, dm, T, B, pre)      # AUTO: MFMA kernels for the steps where they apply
    assert_parity(A2.cpu(), ref, dt)
    assert sync_status() == 0


@pytest.mark.parametrize("name", ["matrix_f16_eye32", "matrix_f32_eye_ragged"])
def test_matrix_kernel_golden_vectors(name):
    g = load_golden(name)
    q, k, mask = to_dev(g["q"], g["k"], g["mask"])
    for variant in ("generic", "auto"):
        A = monarch_matrix_hip(q, k, mask, g["T"], g["B"], g["pre"], variant=variant)
        assert_parity(A.cpu(), g["out"], g["dt"])


def test_matrix_kernel_limits():
    q, k, _ = seeded_qkv(1, 1, 64, 16, torch.float16)
    dq, dk = to_dev(q, k)
    for variant in ("fused", "resident", "chained"):
        with pytest.raises(NotImplementedError):
            monarch_matrix_hip(dq, dk, None, 1, 8, False, variant=variant)
    with pytest.raises(ValueError):
        monarch_matrix_hip(dq, dk[:, :, :32], None, 1, 8, False)
    # a padded sequence beyond the kernel's LDS: the entry point refuses before launching anything
    # (MonarchAttention.get_matrix then takes the identity route)
    ql, kl, _ = seeded_qkv(1, 1, 45000, 8, torch.float32)
    with pytest.raises(NotImplementedError):
        monarch_matrix_hip(ql.to(DEV), kl.to(DEV), None, 1, 4096, False)
    assert sync_status() == 0


def test_module_forward_pre_and_post_pad():
    q, k, v = seeded_qkv(2, 12, 197, 64, torch.float16, scale=0.125)
    for pad in (PadType.pre, "post"):
        mod = MonarchAttention(14, 2, pad)
        out = mod(*to_dev(q, k, v))
        ref = monarch_attention_oracle(q, k, v, None, 2, 14, pad == "pre", upcast=True)
        assert_parity(out.cpu(), ref, "f16")


# ---------------------------------------------------------------- size-independent properties at full benchmark sizes
FULL = [  # E, H, N, D, B, T, dt
    (64, 12, 197, 64, 16, 2, "f16"), (16, 12, 512, 64, 32, 2, "bf16"), (8, 16, 1024, 72, 32, 3, "f16"),
    (1, 16, 4096, 64, 64, 2, "f16"), (1, 16, 16384, 64, 128, 3, "f16"),
]


@pytest.mark.parametrize("variant", ["staged", "fused", "resident", "chained", "auto"])
@pytest.mark.parametrize("E,H,N,D,B,T,dt", FULL)
def test_full_size_properties(E, H, N, D, B, T, dt, variant):
    """At the full benchmark sizes: finite output, bit-reproducible, a single
    (e, h) slice equals the full call (batch/head independence), the output is
    within the convex hull of V per coordinate (rows of A are distributions),
    and the MFMA variants agree with the generic FMA kernels."""
    g = torch.Generator(device="cpu").manual_seed(11)
    scale = 0.125 if N == 197 else 1.0
    q, k, v = ((scale * torch.randn(E, H, N, D, generator=g)).to(DT[dt]).to(DEV) for _ in range(3))
    out = run_hip(q, k, v, None, T, B, False, variant)
    assert torch.isfinite(out.float()).all()
    again = run_hip(q, k, v, None, T, B, False, variant)
    assert torch.equal(out, again)
    e, h = E - 1, H // 2
    one = run_hip(q[e:e + 1, h:h + 1], k[e:e + 1, h:h + 1], v[e:e + 1, h:h + 1], None, T, B, False, variant)
    assert torch.equal(one[0, 0], out[e, h])
    slack = 2e-2 * v.float().abs().max()
    assert (out.float() <= v.float().amax(dim=2, keepdim=True) + slack).all()
    assert (out.float() >= v.float().amin(dim=2, keepdim=True) - slack).all()
    sub = slice(0, min(E, 2))
    gen = run_hip(q[sub], k[sub], v[sub], None, T, B, False, "generic")
    assert_parity(out[sub].cpu(), gen.cpu(), dt, "vs generic")
    assert sync_status() == 0


# ---------------------------------------------------------------- seeded random shapes, every variant
def _random_cases(n, seed):
    import random
    rng = random.Random(seed)
    cases = []
    for i in range(n):
        dt = rng.choice(["f16", "f16", "bf16", "f32"])
        D = rng.choice([8, 16, 24, 32, 40, 48, 56, 64, 72, 80, 96, 128] if dt != "f32" else [4, 8, 12, 16, 32, 36, 48, 64, 100, 128])
        B = rng.choice([1, 2, 3, 5, 8, 14, 16, 17, 24, 31, 32, 33, 48, 64, 65, 96, 128])
        M = rng.choice([1, 2, 3, 4, 7, 8, 15, 16, 17, 31, 32, 33, 64] if B <= 32 else [1, 2, 3, 5, 8, 9])
        N = max(1, M * B - rng.randrange(0, B))           # ragged last block most of the time
        E, H = rng.choice([1, 1, 2, 3]), rng.choice([1, 2, 3, 5])
        T = rng.choice([1, 1, 2, 2, 3, 4])
        pre = rng.random() < 0.5
        masked = rng.random() < 0.4
        cases.append((i, E, H, N, D, B, T, pre, dt, masked))
    return cases


@pytest.mark.parametrize("idx,E,H,N,D,B,T,pre,dt,masked", _random_cases(200, seed=2024))
def test_random_shapes_every_variant(idx, E, H, N, D, B, T, pre, dt, masked):
    """Seeded random problems over the whole argument space (ragged N, odd block
    sizes and counts, every head-dim class, both pad sides, key masks, 1..4
    steps): every variant that accepts the problem must meet the parity gate,
    and AUTO / GENERIC must accept all of them."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], scale=0.7, seed=100 + idx)
    mask = block_safe_mask(E, N, B, seed=idx) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=dt != "f32")
    ran = []
    for variant in VARIANTS:
        try:
            out = monarch_attention_hip(*to_dev(q, k, v, mask), T, B, pre, variant=variant)
        except NotImplementedError:
            assert variant not in ("auto", "generic")
            continue
        torch.cuda.synchronize()
        assert_parity(out.cpu(), ref, dt, f"case {idx} {(E, H, N, D, B, T, pre, dt, masked)} / {variant}")
        ran.append(variant)
    assert "auto" in ran and "generic" in ran
    assert sync_status() == 0


def _random_large_cases(n, seed):
    import random
    rng = random.Random(seed)
    cases = []
    for i in range(n):
        side = rng.choice(["blocks", "rows", "both"])
        B = rng.randint(129, 256) if side != "blocks" else rng.choice([1, 7, 16, 24, 33, 64])
        M = rng.randint(129, 256) if side != "rows" else rng.choice([1, 2, 5, 16, 40])
        N = max(1, M * B - rng.randrange(0, B))
        dt = rng.choice(["f16", "bf16"])
        D = rng.choice([8, 16, 32, 40, 64, 72, 96, 128])
        H = 1 if side == "both" else rng.choice([1, 2, 3])
        cases.append((i, 1, H, N, D, B, rng.choice([1, 2, 3]), rng.random() < 0.5, dt, rng.random() < 0.4))
    return cases


@pytest.mark.parametrize("idx,E,H,N,D,B,T,pre,dt,masked", _random_large_cases(24, seed=65536))
def test_random_shapes_in_the_192_and_256_row_classes(idx, E, H, N, D, B, T, pre, dt, masked):
    """Seeded random problems whose blocks and / or block counts lie in 129 .. 256 (heads of up to 65536
    tokens): AUTO must run them on the MFMA stage kernels and meet the parity gate."""
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], scale=0.7, seed=300 + idx)
    mask = block_safe_mask(E, N, B, seed=idx) if masked else None
    ref = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    dev = to_dev(q, k, v, mask)
    out = torch.empty_like(dev[2])
    assert L.VARIANT_NAMES[L.load().ma_fwd_select_variant(make_params(*dev[:3], None, out, T, B, pre, "auto"))] == "staged"
    got = monarch_attention_hip(*dev, T, B, pre, variant="auto")
    torch.cuda.synchronize()
    assert_parity(got.cpu(), ref, dt, f"large case {idx} {(E, H, N, D, B, T, pre, dt, masked)}")


# ---------------------------------------------------------------- a wait between workgroups that runs out is loud
@pytest.mark.parametrize("shape", [(1, 2, 1024, 64, 32, 2), (3, 8, 512, 64, 32, 3), (1, 16, 2048, 64, 64, 1)])
@pytest.mark.parametrize("variant", ["fused", "chained"])
def test_wait_that_runs_out_is_loud_and_leaves_the_workspace_usable(variant, shape):
    """MA_FLAG_TEST_NO_SPIN makes every wait of the one-launch kernels give up at once (forced from the
    host; every kernel still runs to its end).  The call must then raise the sticky error word and
    write NaN rows instead of results computed from a state that may be incomplete, and the next
    call on the same workspace must be an ordinary, correct one.  Tasks that do not wait run in no
    particular order, so the failed call is repeated: whatever order they finish in, the sync area
    must come out consistent."""
    lib = L.load()
    E, H, N, D, B, T = shape
    q, k, v = to_dev(*seeded_qkv(E, H, N, D, torch.float16, seed=3))
    want = monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False)
    out = torch.zeros_like(v)
    p = make_params(q, k, v, None, out, T, B, False, variant)
    nbytes = lib.ma_fwd_workspace_bytes(p)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    word = ws[4:8].view(torch.int32)
    p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
    host_word = torch.zeros(1, dtype=torch.int32, pin_memory=True)   # ma_fwd_params.error_word: the same code, in host memory
    p.error_word = host_word.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream

    p.flags = L.MA_FLAG_SYNC_READY
    L.check(lib.ma_fwd(p, stream), "ma_fwd")
    torch.cuda.synchronize()
    assert int(word.item()) == 0 and int(host_word[0]) == 0
    assert_parity(out.cpu(), want, "f16", f"{variant} before")

    for rep in range(4):
        out.zero_()
        p.flags = L.MA_FLAG_SYNC_READY | L.MA_FLAG_TEST_NO_SPIN
        for _ in range(1 + rep % 2):   # also two failed calls back to back
            L.check(lib.ma_fwd(p, stream), "ma_fwd")
        torch.cuda.synchronize()
        assert int(word.item()) == 1, "the wait that ran out was not reported"
        assert int(host_word[0]) == 1, "the wait that ran out was not reported in the caller's host word"
        assert torch.isnan(out.float()).any(dim=-1).all(), "every output row depends on a wait that gave up: all must be NaN"

        word.zero_()
        host_word.zero_()
        out.zero_()
        p.flags = L.MA_FLAG_SYNC_READY   # no clearing of the sync area: the failed call must have left it consistent
        for _ in range(2):
            L.check(lib.ma_fwd(p, stream), "ma_fwd")
        torch.cuda.synchronize()
        assert int(word.item()) == 0 and int(host_word[0]) == 0
        assert_parity(out.cpu(), want, "f16", f"{variant} after failed call {rep}")


def test_module_reports_a_failed_call_at_a_later_call(monkeypatch):
    """The Python operator never synchronises to look at the error word: the kernel stores it into
    pinned host memory as well, every call looks there first, and so a failed call is reported by a
    RuntimeError from the next call made after its work is complete; calls are normal again after that."""
    from ma import ma_hip
    E, H, N, D, B, T = 1, 2, 1024, 64, 32, 2
    q, k, v = to_dev(*seeded_qkv(E, H, N, D, torch.float16, seed=4))
    want = monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False)
    ma_hip.clear_workspace_cache()
    good = monarch_attention_hip(q, k, v, None, T, B, False, variant="fused")
    torch.cuda.synchronize()
    monkeypatch.setattr(ma_hip, "_TEST_FLAGS", L.MA_FLAG_TEST_NO_SPIN)
    bad = monarch_attention_hip(q, k, v, None, T, B, False, variant="fused")   # returns: nothing is known yet
    monkeypatch.setattr(ma_hip, "_TEST_FLAGS", 0)
    torch.cuda.synchronize()
    assert torch.isnan(bad.float()).any()
    with pytest.raises(RuntimeError, match="earlier forward call"):
        monarch_attention_hip(q, k, v, None, T, B, False, variant="fused")   # the very next call
    again = monarch_attention_hip(q, k, v, None, T, B, False, variant="fused")
    torch.cuda.synchronize()
    assert_parity(good.cpu(), want, "f16", "before the failure")
    assert_parity(again.cpu(), want, "f16", "after the failure")
    assert sync_status() == 0
    ma_hip.clear_workspace_cache()
