"""The oracle's gradients (autograd through the CPU restatement) against the
gradient fixtures written from the reference, and against finite differences.

The reference has no backward code: training differentiates its forward with
autograd, and the fixtures under tests/golden/grads hold what that yields.
The oracle is plain PyTorch as well, so autograd through it is the gradient
oracle for the HIP backward pass; these tests pin it.
"""
import pytest
import torch

from helpers import DT, block_safe_mask, grad_golden_names, load_grad_golden, seeded_qkv
from oracle.ma_oracle import monarch_attention_oracle


def oracle_grads(q, k, v, mask, w, T, B, pre, **kw):
    q, k, v = (t.detach().clone().requires_grad_() for t in (q, k, v))
    out = monarch_attention_oracle(q, k, v, mask, T, B, pre, **kw)
    (out * w).sum().backward()
    return q.grad, k.grad, v.grad


def rel_err(a, b):
    a, b = a.double(), b.double()
    return ((a - b).norm() / b.norm().clamp(min=1e-30)).item()


@pytest.mark.parametrize("name", grad_golden_names())
def test_oracle_autograd_matches_the_reference_gradients(name):
    g = load_grad_golden(name)
    got = oracle_grads(g["q"], g["k"], g["v"], g["mask"], g["w"], g["T"], g["B"], g["pre"])
    tol = 1e-5 if g["dt"] == "f32" else 2e-2
    for x, ref, what in zip(got, (g["dq"], g["dk"], g["dv"]), "qkv"):
        assert x.dtype == ref.dtype and x.shape == ref.shape
        assert torch.isfinite(x.float()).all()
        assert rel_err(x, ref) <= tol, (name, what, rel_err(x, ref))


@pytest.mark.parametrize("T,pre,masked", [(1, False, False), (2, True, True), (3, False, True)])
def test_oracle_autograd_against_finite_differences(T, pre, masked):
    """Directional derivatives of loss = sum(out * w) by central differences of
    the fp32 forward: (loss(x + h d) - loss(x - h d)) / 2h = <grad, d>."""
    E, H, N, D, B = 1, 2, 13, 8, 4
    q, k, v = seeded_qkv(E, H, N, D, torch.float32, Dv=6, seed=3)
    mask = block_safe_mask(E, N, B, seed=5) if masked else None
    gen = torch.Generator().manual_seed(11)
    w = torch.randn(E, H, N, 6, generator=gen)
    grads = oracle_grads(q, k, v, mask, w, T, B, pre)

    def loss(q_, k_, v_):
        return (monarch_attention_oracle(q_.double().float(), k_.double().float(), v_.double().float(),
                                         mask, T, B, pre).double() * w.double()).sum().item()

    h = 2e-3
    for which, (x, gx) in enumerate(zip((q, k, v), grads)):
        for _ in range(3):
            d = torch.randn(x.shape, generator=gen)
            args_p, args_m = [q, k, v], [q, k, v]
            args_p[which], args_m[which] = x + h * d, x - h * d
            fd = (loss(*args_p) - loss(*args_m)) / (2 * h)
            an = (gx.double() * d.double()).sum().item()
            assert abs(fd - an) <= 2e-2 * max(1.0, abs(an)), (which, fd, an)
