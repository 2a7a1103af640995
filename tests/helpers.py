"""Shared helpers for the test-suite: golden-vector loading, seeded inputs,
error metrics and the tolerances of the parity gate."""
import glob
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def _unpack(a: np.ndarray, dt: str) -> torch.Tensor:
    if dt == "bf16":
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


def golden_names():
    return sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN_DIR, "*.npz")))


def load_golden(name: str) -> dict:
    """One committed golden vector: inputs, parameters and the output the
    reference produced for them on the CPU."""
    z = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
    E, H, N, D, Dv, B, T, pre = (int(x) for x in z["meta"])
    dt, vdt = str(z["dt"]), str(z["vdt"])
    q, k = _unpack(z["q"], dt), _unpack(z["k"], dt)
    if bool(z["v_eye"]):
        v = torch.eye(N, dtype=DT[vdt]).expand(E, H, N, N)
    else:
        v = _unpack(z["v"], vdt)
    mask = torch.from_numpy(z["mask"].copy()) if "mask" in z.files else None
    return dict(name=name, q=q, k=k, v=v, mask=mask, T=T, B=B, pre=bool(pre), dt=dt, vdt=vdt,
                out=_unpack(z["out"], vdt), E=E, H=H, N=N, D=D, Dv=Dv)


GRAD_DIR = os.path.join(GOLDEN_DIR, "grads")


def grad_golden_names():
    return sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GRAD_DIR, "*.npz")))


def load_grad_golden(name: str) -> dict:
    """One committed gradient fixture: inputs, the weights w of the loss
    sum(out * w) (= the output gradient) and the gradients autograd through
    the reference produced on the CPU."""
    z = np.load(os.path.join(GRAD_DIR, name + ".npz"), allow_pickle=False)
    E, H, N, D, Dv, B, T, pre = (int(x) for x in z["meta"])
    dt = str(z["dt"])
    t = {n: _unpack(z[n], dt) for n in ("q", "k", "v", "w", "dq", "dk", "dv")}
    mask = torch.from_numpy(z["mask"].copy()) if "mask" in z.files else None
    return dict(name=name, mask=mask, T=T, B=B, pre=bool(pre), dt=dt, **t)


def seeded_qkv(E, H, N, D, dtype, Dv=None, scale=1.0, seed=0):
    """fp32 CPU randn in the order q, k, v (as ma/tests/test_ma.py:11-15),
    then scaled and cast."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(E, H, N, D, generator=g)
    k = torch.randn(E, H, N, D, generator=g)
    v = torch.randn(E, H, N, Dv or D, generator=g)
    return tuple((scale * t).to(dtype) for t in (q, k, v))


def block_safe_mask(E, N, B, seed=1):
    """Random key mask, at least one kept token per block (the construction of
    ma/tests/test_ma.py:18-29)."""
    g = torch.Generator().manual_seed(seed)
    M = -(-N // B)
    mask = torch.rand(E, N, generator=g) > 0.3
    for e in range(E):
        for m in range(M):
            lo, hi = m * B, min(m * B + B, N)
            if not mask[e, lo:hi].any():
                mask[e, lo] = True
    return mask


def err_metrics(out: torch.Tensor, ref: torch.Tensor) -> dict:
    o, r = out.detach().double().cpu(), ref.detach().double().cpu()
    d = (o - r).abs()
    return dict(max_abs=d.max().item(),
                rel_max=(d.max() / r.abs().max().clamp(min=1e-30)).item(),
                rel_fro=((o - r).norm() / r.norm().clamp(min=1e-30)).item())


# Parity gate: fp32 max-abs <= 1e-5; fp16/bf16 <= 2e-2 relative (evaluated both
# as max|d|/max|ref| and as the Frobenius ratio) plus the reference's own
# allclose criterion (ma/tests/test_ma.py:64-65): atol = rtol = 1e-2 (fp16),
# 5e-2 (bf16).
FP32_MAX_ABS = 1e-5
LOWP_REL = 2e-2
REF_ALLCLOSE = {"f16": 1e-2, "bf16": 5e-2}


def assert_parity(out, ref, dt: str, what: str = ""):
    assert out.shape == ref.shape, (what, out.shape, ref.shape)
    assert out.dtype == ref.dtype, (what, out.dtype, ref.dtype)
    assert torch.isfinite(out.float()).all(), f"{what}: non-finite output"
    m = err_metrics(out, ref)
    if dt == "f32":
        assert m["max_abs"] <= FP32_MAX_ABS, (what, m)
    else:
        assert m["rel_max"] <= LOWP_REL and m["rel_fro"] <= LOWP_REL, (what, m)
        tol = REF_ALLCLOSE[dt]
        assert torch.allclose(out.float().cpu(), ref.float().cpu(), atol=tol, rtol=tol), (what, m)
    return m
