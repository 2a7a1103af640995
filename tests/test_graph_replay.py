"""The forward entry points under HIP graph capture: ``ma_fwd`` (caller workspace) and
``ma_fwd_static`` (no allocation at all) are captured once and replayed several times, with eager
forward calls and synchronisations between the replays; every replay must reproduce the eager
result bit for bit.  The one-launch variants keep their barrier epochs and counters in the
workspace, so a replay continues from what the previous launch left there - this is what the test
pins - and the sync area is cleared by a fill kernel, never by a memset node.
"""
import pytest
import torch

from helpers import DT, assert_parity, seeded_qkv
from ma import _hip_lib as L
from ma.ma_hip import make_params, monarch_attention_hip
from oracle.ma_oracle import monarch_attention_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = [  # E, H, N, D, B, T, dtype, variant
    (1, 16, 1024, 64, 32, 1, "f16", "auto"),      # few heads of small blocks: the chained kernel
    (1, 16, 1024, 64, 32, 2, "f16", "fused"),
    (1, 16, 4096, 64, 64, 1, "f16", "fused"),     # teams that fill the device
    (2, 4, 512, 64, 32, 2, "f16", "resident"),    # one state tile in LDS, Y through the workspace
    (2, 6, 384, 64, 128, 2, "bf16", "chained"),   # heads of three blocks: several positions per tile
    (4, 12, 512, 64, 32, 2, "bf16", "chained"),
    (8, 16, 197, 64, 16, 2, "f16", "resident"),
    (1, 4, 2048, 64, 128, 2, "f16", "staged"),
    (1, 2, 300, 48, 16, 2, "f32", "auto"),
]


@pytest.mark.parametrize("static", [False, True], ids=["workspace", "static"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_captured_forward_replays_like_eager(case, static):
    lib = L.load()
    E, H, N, D, B, T, dt, variant = CASES[case]
    q, k, v = (t.to(DEV) for t in seeded_qkv(E, H, N, D, DT[dt], seed=case))
    entry = lib.ma_fwd_static if static else lib.ma_fwd

    def params(out):
        p = make_params(q, k, v, None, out, T, B, False, variant)
        if not static:
            p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
        return p

    probe = make_params(q, k, v, None, torch.empty_like(v), T, B, False, variant)
    ws = torch.zeros(max(int(lib.ma_fwd_workspace_bytes(probe)), 1), dtype=torch.uint8, device=DEV)

    def eager():
        out = torch.full(v.shape, float("nan"), dtype=v.dtype, device=DEV)
        L.check(entry(params(out), torch.cuda.current_stream().cuda_stream), "eager forward")
        torch.cuda.synchronize()
        return out

    try:
        want = eager()   # also the warm-up: one-time set-up (kernel attributes, the static array's address) happens here
    except NotImplementedError as ex:
        pytest.skip(f"variant {variant}: {ex}")
    assert_parity(want.cpu(), monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False), dt, f"eager case {case}")

    out_g = torch.full(v.shape, float("nan"), dtype=v.dtype, device=DEV)
    p_g = params(out_g)   # kept alive: the graph holds the device pointers it names
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = entry(p_g, torch.cuda.current_stream().cuda_stream)
    L.check(status, "captured forward")
    for rep in range(4):
        out_g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.uint8), want.view(torch.uint8)), f"case {case} replay {rep} differs from eager"
        again = eager()   # the program's own eager work on the same workspace between replays
        assert torch.equal(again.view(torch.uint8), want.view(torch.uint8)), f"case {case} eager call after replay {rep} differs"


@pytest.mark.parametrize("case", [0, 1, 2, 3, 7, 8])
def test_captured_module_call_replays_like_eager(case):
    """The Python operator itself under capture: it allocates its output from the graph's pool, looks
    at the host-visible error word (a host read) and queues nothing but the library's kernels, so a
    captured call replays like the eager one - with eager calls on the same stream, which share the
    workspace with the captured call, between the replays."""
    E, H, N, D, B, T, dt, variant = CASES[case]
    q, k, v = (t.to(DEV) for t in seeded_qkv(E, H, N, D, DT[dt], seed=case))
    side = torch.cuda.Stream()

    def eager():
        with torch.cuda.stream(side):
            out = monarch_attention_hip(q, k, v, None, T, B, False, variant=variant)
        side.synchronize()
        return out

    side.wait_stream(torch.cuda.current_stream())
    want = eager()   # warm-up: the call plan and the workspace of this stream exist before the capture
    assert_parity(want.cpu(), monarch_attention_oracle(q.cpu(), k.cpu(), v.cpu(), None, T, B, False), dt, f"eager case {case}")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_g = monarch_attention_hip(q, k, v, None, T, B, False, variant=variant)
    for rep in range(3):
        out_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.uint8), want.view(torch.uint8)), f"case {case} replay {rep} differs from eager"
        again = eager()
        assert torch.equal(again.view(torch.uint8), want.view(torch.uint8)), f"case {case} eager call after replay {rep} differs"
