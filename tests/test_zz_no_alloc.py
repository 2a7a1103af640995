"""``ma_fwd_static``: the forward entry point that allocates nothing (its state
lives in an array the library holds on the GPU) against ``ma_fwd`` with a
caller-provided workspace, through the C ABI.

Both run the same kernels on the same inputs, so the gate is the strictest one:
bit-identical outputs (and, as a cross-check of the test itself, parity with the
CPU oracle at the usual tolerance).  Two calls in a row share the array, the
second on a smaller problem; problems beyond the array's size are refused; the
calls change neither the device's free memory nor PyTorch's allocator
statistics; and a call that would overlap with one on another stream is turned
away (MA_ERR_BUSY).
"""
import gc

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


def test_static_allocates_and_frees_nothing():
    """After a warm-up call (code objects, the array's address, the guard's event) a ma_fwd_static
    call leaves the device's free memory (hipMemGetInfo) and PyTorch's allocator statistics as they
    were - for a one-launch variant, whose sync area is cleared by a fill kernel, and for the
    per-stage launches."""
    lib = L.load()
    stream = torch.cuda.current_stream().cuda_stream
    for (E, H, N, D, B, T, dt, variant) in [(1, 16, 4096, 64, 64, 2, "f16", "chained"), (1, 16, 4096, 64, 64, 1, "f16", "fused"),
                                            (2, 3, 512, 64, 32, 3, "bf16", "staged"), (1, 2, 300, 48, 16, 2, "f32", "auto")]:
        q, k, v = (t.to(DEV) for t in seeded_qkv(E, H, N, D, DT[dt], seed=1))
        out = torch.empty_like(v)
        p = make_params(q, k, v, None, out, T, B, False, variant)
        L.check(lib.ma_fwd_static(p, stream), "warm-up")
        torch.cuda.synchronize()
        # nothing of this process may allocate or free in the measured region but the calls themselves: tensors
        # that earlier tests left to the garbage collector are collected now, and the collector is held off
        gc.collect()
        gc.disable()
        try:
            free0, total0 = torch.cuda.mem_get_info()
            stats0 = {k_: v_ for k_, v_ in torch.cuda.memory_stats().items() if k_.startswith(("allocation.all.", "segment.all."))}
            for _ in range(3):
                L.check(lib.ma_fwd_static(p, stream), "ma_fwd_static")
            torch.cuda.synchronize()
            free1, total1 = torch.cuda.mem_get_info()
            stats1 = {k_: v_ for k_, v_ in torch.cuda.memory_stats().items() if k_ in stats0}
        finally:
            gc.enable()
        assert (free1, total1) == (free0, total0), f"{variant}: free device memory changed by {free0 - free1} bytes"
        assert stats1 == stats0, f"{variant}: PyTorch allocator statistics changed"


def test_static_turns_away_a_call_that_would_overlap():
    """All calls on a GPU share one array.  A call on another stream than the previous call's, made
    while that call's work is still queued or running, returns MA_ERR_BUSY and launches nothing;
    calls on one stream are ordered and always accepted; once the earlier work is complete the
    other stream's call is accepted too."""
    lib = L.load()
    E, H, N, D, B, T = 1, 4, 1000, 64, 32, 2
    q, k, v = (t.to(DEV) for t in seeded_qkv(E, H, N, D, torch.float16, seed=11))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    out1, out1b, out2 = (torch.full(v.shape, float("nan"), dtype=v.dtype, device=DEV) for _ in range(3))
    p1, p1b, p2 = (make_params(q, k, v, None, o, T, B, False, "auto") for o in (out1, out1b, out2))
    L.check(lib.ma_fwd_static(p1, s1.cuda_stream), "warm-up")
    torch.cuda.synchronize()
    out1.fill_(float("nan"))
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        torch.cuda._sleep(400_000_000)    # keeps s1 busy for a good tenth of a second: what follows on s1 stays queued
    assert lib.ma_fwd_static(p1, s1.cuda_stream) == L.MA_OK
    assert lib.ma_fwd_static(p2, s2.cuda_stream) == L.MA_ERR_BUSY      # would run while s1's call is pending
    assert lib.ma_fwd_static(p1b, s1.cuda_stream) == L.MA_OK           # ordered behind it: fine
    assert "another stream" in L.strerror(L.MA_ERR_BUSY)
    torch.cuda.synchronize()
    assert torch.isnan(out2).all()                                      # the refused call launched nothing
    assert lib.ma_fwd_static(p2, s2.cuda_stream) == L.MA_OK            # s1's work is complete now
    torch.cuda.synchronize()
    want = monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False)
    assert_parity(out1.cpu(), want, "f16", "static call on the first stream")
    for o in (out1b, out2):
        assert torch.equal(o.view(torch.uint8), out1.view(torch.uint8))
