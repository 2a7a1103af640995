"""Parity of the HIP backward pass (ma_bwd, through the C ABI) with the
gradients autograd yields through the reference / the CPU oracle.  Runs on a
MI355X only (``-m gpu``).

Gate: fp32 relative Frobenius error <= 1e-4 per gradient (and max-abs <= 1e-4
of the gradient's largest entry); fp16 <= 4e-3 (max-abs 8e-3), bf16 <= 1.5e-2
(max-abs 3e-2) - a few units of the operand type's rounding step (2^-10, 2^-7):
the reference's autograd rounds every intermediate gradient to the operand
dtype, the HIP backward keeps fp32 between its kernels and rounds once at the end.
"""
import pytest
import torch

from helpers import DT, block_safe_mask, grad_golden_names, load_grad_golden, seeded_qkv
from ma.ma_hip import monarch_attention_hip, monarch_attention_hip_backward
from ma.monarch_attention import MonarchAttention
from oracle.ma_oracle import monarch_attention_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def to_dev(*ts):
    return tuple(None if t is None else t.to(DEV) for t in ts)


def oracle_grads(q, k, v, mask, w, T, B, pre):
    q, k, v = (t.detach().clone().requires_grad_() for t in (q, k, v))
    out = monarch_attention_oracle(q, k, v, mask, T, B, pre, upcast=True)
    (out * w).sum().backward()
    return q.grad, k.grad, v.grad


def assert_grads(got, ref, dt, what=""):
    tol, tol_max = {"f32": (1e-4, 1e-4), "f16": (4e-3, 8e-3), "bf16": (1.5e-2, 3e-2)}[dt]
    for x, r, name in zip(got, ref, ("dq", "dk", "dv")):
        x, r = x.detach().double().cpu(), r.detach().double().cpu()
        assert x.shape == r.shape
        assert torch.isfinite(x).all(), (what, name)
        rel = ((x - r).norm() / r.norm().clamp(min=1e-30)).item()
        mx = ((x - r).abs().max() / r.abs().max().clamp(min=1e-30)).item()
        assert rel <= tol and mx <= tol_max, (what, name, rel, mx)


@pytest.mark.parametrize("variant", ["generic", "auto"])
@pytest.mark.parametrize("name", grad_golden_names())
def test_gradient_fixtures(name, variant):
    g = load_grad_golden(name)
    q, k, v, mask, w = to_dev(g["q"], g["k"], g["v"], g["mask"], g["w"])
    got = monarch_attention_hip_backward(q, k, v, mask, w, g["T"], g["B"], g["pre"], variant=variant)
    for x, r in zip(got, (g["dq"], g["dk"], g["dv"])):
        assert x.dtype == r.dtype and x.is_contiguous()
    assert_grads(got, (g["dq"], g["dk"], g["dv"]), g["dt"], name)


CASES = [  # E, H, N, D, Dv, B, T, pre, dt, masked
    (2, 3, 64, 32, 32, 16, 1, False, "f32", False), (2, 3, 64, 32, 32, 16, 2, False, "f16", True),
    (1, 2, 197, 64, 64, 14, 2, True, "f16", False), (2, 1, 61, 24, 40, 7, 3, True, "f32", True),
    (1, 2, 300, 40, 40, 32, 3, False, "bf16", True), (1, 1, 5, 4, 4, 8, 2, False, "f32", False),
    (1, 4, 256, 64, 64, 16, 2, False, "f32", False), (1, 2, 130, 16, 16, 1, 1, False, "f32", False),
    (1, 2, 48, 16, 16, 64, 2, True, "f32", True), (1, 1, 700, 8, 8, 2, 2, False, "f32", False),
    # problems walked in several row tiles: 128 key blocks (L / Z stages), 128-row blocks with d = 128 (R stage;
    # in fp32 that one is beyond the matrix-core kernels' LDS and takes the FMA kernels)
    (1, 2, 1024, 64, 64, 8, 2, False, "bf16", True), (1, 2, 1024, 64, 64, 8, 2, False, "f32", False),
    (1, 2, 256, 128, 128, 128, 2, False, "f16", False), (1, 1, 256, 128, 128, 128, 2, True, "f32", True),
    # few large blocks: the R stage gives a block's tiles of query rows to different workgroups (partial dk / dv)
    (1, 2, 300, 48, 48, 128, 2, False, "f32", True), (1, 3, 260, 64, 64, 128, 3, True, "bf16", False),
    # 16-bit R stage with the probabilities in registers: head dims of 72 and 128, 64-row blocks with a mask,
    # 128-row blocks in enough blocks (512) that they are not split over workgroups
    (1, 2, 224, 72, 72, 32, 3, True, "f16", True), (1, 2, 512, 128, 128, 64, 2, False, "bf16", False),
    (2, 2, 512, 64, 64, 64, 2, False, "f16", True), (1, 8, 8192, 32, 32, 128, 2, False, "bf16", False),
    # 129 .. 256 blocks / rows per block: the forward steps run in the stage kernels' 16-strip class, the
    # derivative stages in the LDS kernels (row tiles)
    (1, 2, 1600, 64, 64, 10, 2, False, "f16", True), (1, 1, 1500, 32, 32, 150, 2, True, "bf16", False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(map(str, c)))
def test_backward_against_oracle_autograd(case):
    E, H, N, D, Dv, B, T, pre, dt, masked = case
    q, k, v = seeded_qkv(E, H, N, D, DT[dt], Dv=Dv)
    mask = block_safe_mask(E, N, B, seed=N) if masked else None
    w = torch.randn(E, H, N, Dv, generator=torch.Generator().manual_seed(7)).to(DT[dt])
    ref = oracle_grads(q, k, v, mask, w, T, B, pre)
    dq, dk, dv, dm, dw = to_dev(q, k, v, mask, w)
    for variant in ("generic", "auto"):
        got = monarch_attention_hip_backward(dq, dk, dv, dm, dw, T, B, pre, variant=variant)
        assert_grads(got, ref, dt, variant)
    again = monarch_attention_hip_backward(dq, dk, dv, dm, dw, T, B, pre, variant="auto")
    for a, b in zip(got, again):   # fixed summation order: bit-reproducible
        assert torch.equal(a, b)


def test_autograd_through_the_module_and_strided_views():
    """loss.backward() through MonarchAttention on the permuted (E,N,H,D) views
    that models pass, with an integer mask; the gradients land in the leaf
    tensors' layout."""
    E, H, N, D, B, T = 2, 4, 100, 32, 16, 2
    gen = torch.Generator().manual_seed(2)
    x = [torch.randn(E, N, H, D, generator=gen) for _ in range(3)]
    mask = (torch.arange(N)[None, :] < torch.tensor([N, N - 17])[:, None]).to(torch.int64)
    w = torch.randn(E, H, N, D, generator=gen)
    ref = oracle_grads(*(t.permute(0, 2, 1, 3) for t in x), mask, w, T, B, False)
    leaves = [t.to(DEV).requires_grad_() for t in x]
    mod = MonarchAttention(B, T, "post")
    out = mod(*(t.permute(0, 2, 1, 3) for t in leaves), mask.to(DEV))
    assert out.requires_grad
    (out * w.to(DEV)).sum().backward()
    got = [t.grad.permute(0, 2, 1, 3) for t in leaves]
    assert_grads(got, ref, "f32")
    # no graph is recorded when nothing requires grad or grad mode is off
    with torch.no_grad():
        assert not mod(*(t.permute(0, 2, 1, 3) for t in leaves)).requires_grad
    assert not mod(*(t.detach().permute(0, 2, 1, 3) for t in leaves)).requires_grad


def test_only_some_inputs_require_grad_and_half_precision_training_step():
    E, H, N, D, B, T = 1, 8, 128, 64, 16, 2
    q, k, v = to_dev(*seeded_qkv(E, H, N, D, torch.bfloat16))
    v.requires_grad_()
    out = monarch_attention_hip(q, k, v, None, T, B, False)
    out.float().square().sum().backward()
    assert v.grad is not None and v.grad.dtype == torch.bfloat16 and q.grad is None
    assert torch.isfinite(v.grad.float()).all()


def test_backward_against_finite_differences_of_the_hip_forward():
    """Directional derivatives of the fp32 HIP forward at a model-like shape."""
    E, H, N, D, B, T = 1, 2, 197, 32, 14, 2
    q, k, v = to_dev(*seeded_qkv(E, H, N, D, torch.float32, scale=0.5))
    gen = torch.Generator().manual_seed(5)
    w = torch.randn(E, H, N, D, generator=gen).to(DEV)
    grads = monarch_attention_hip_backward(q, k, v, None, w, T, B, True, variant="generic")

    def loss(q_, k_, v_):
        return (monarch_attention_hip(q_, k_, v_, None, T, B, True, variant="generic").double() * w.double()).sum().item()

    h = 1e-2
    for which, gx in enumerate(grads):
        d = torch.randn(gx.shape, generator=gen).to(DEV)
        d = d / d.norm()
        args_p, args_m = [q, k, v], [q, k, v]
        args_p[which], args_m[which] = args_p[which] + h * d, args_m[which] - h * d
        fd = (loss(*args_p) - loss(*args_m)) / (2 * h)
        an = (gx.double() * d.double()).sum().item()
        assert abs(fd - an) <= 2e-2 * max(abs(an), 1e-2), (which, fd, an)


def test_backward_rejects_what_it_cannot_run():
    q, k, v = to_dev(*seeded_qkv(1, 2, 64, 16, torch.float16))
    w = torch.ones_like(v)
    for variant in ("fused", "chained", "resident"):
        with pytest.raises(NotImplementedError):
            monarch_attention_hip_backward(q, k, v, None, w, 2, 16, False, variant=variant)
    with pytest.raises(ValueError):
        monarch_attention_hip_backward(q, k, v, None, w[:, :, :32], 2, 16, False)


def test_backward_through_broadcast_keys_and_values():
    """k and v shared by all heads (expanded views, stride 0): the forward reads them in place, the
    gradient of the shared tensor is the sum over the heads."""
    E, H, N, D, B, T = 2, 3, 64, 32, 16, 2
    q, k1, v1 = seeded_qkv(E, H, N, D, torch.float32)
    k1, v1 = k1[:1, :1].contiguous(), v1[:1, :1].contiguous()
    w = torch.randn(E, H, N, D, generator=torch.Generator().manual_seed(3))
    cpu = [t.clone().requires_grad_() for t in (q, k1, v1)]
    out = monarch_attention_oracle(cpu[0], cpu[1].expand(E, H, N, D), cpu[2].expand(E, H, N, D), None, T, B, False)
    (out * w).sum().backward()
    dev = [t.to(DEV).requires_grad_() for t in (q, k1, v1)]
    out = monarch_attention_hip(dev[0], dev[1].expand(E, H, N, D), dev[2].expand(E, H, N, D), None, T, B, False)
    (out * w.to(DEV)).sum().backward()
    assert_grads([t.grad for t in dev], [t.grad for t in cpu], "f32")


def test_backward_with_an_fp32_value_tensor_and_16_bit_queries():
    """fp16 q / k with an fp32 v of another width (the dtype mix of get_matrix): the FMA backward kernels."""
    E, H, N, D, Dv, B, T = 1, 2, 45, 16, 24, 8, 2
    q, k, v = seeded_qkv(E, H, N, D, torch.float16, Dv=Dv)
    v = v.float()
    mask = block_safe_mask(E, N, B, seed=9)
    w = torch.randn(E, H, N, Dv, generator=torch.Generator().manual_seed(4))
    ref = oracle_grads(q, k, v, mask, w, T, B, True)
    got = monarch_attention_hip_backward(*to_dev(q, k, v, mask, w), T, B, True)
    assert got[0].dtype == torch.float16 and got[2].dtype == torch.float32
    assert_grads(got, ref, "f16")
