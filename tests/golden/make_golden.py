"""Write the golden vectors under tests/golden/ from the reference implementation.

Run ONCE, in the build container only (the reference tree does not travel):

    python tests/golden/make_golden.py [/root/reference]

It imports the reference's pure-PyTorch forward (``ma/ma_torch.py``,
``monarch_attention_torch``) on the CPU, feeds it seeded inputs and stores
inputs + outputs as data (``.npz``; fp16 tensors as float16 arrays, bfloat16
tensors as their uint16 bit patterns, fp32 as float32).  The shapes are the
reference's own test tables (``ma/tests/test_ma.py:34-48,70-80,105-109,
125-133``) plus the first benchmark configuration and a few cases for the
behaviours only an execution of the reference can pin: low-precision rounding
points at T >= 2, an fp32 identity ``V`` with fp16 ``q/k`` (``get_matrix``),
an all-masked key block, ragged N with both pad types, and d = 72.
Nothing in the test-suite, the library or the benchmark imports this script.
"""

import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))

DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def block_safe_mask(E, N, B, gen):
    """Random key mask with at least one kept token per block
    (same construction as ma/tests/test_ma.py:18-29, on the CPU)."""
    M = -(-N // B)
    mask = torch.rand(E, N, generator=gen) > 0.3
    for e in range(E):
        for m in range(M):
            lo, hi = m * B, min(m * B + B, N)
            if not mask[e, lo:hi].any():
                mask[e, lo] = True
    return mask


def pack(t):
    """Tensor -> numpy array without loss (bf16 as raw uint16 bits)."""
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    return t.contiguous().numpy()


def cases():
    c = []

    def add(name, E, H, N, D, B, T, pre, dt, Dv=None, mask=None, vdt=None, scale=1.0, v_eye=False):
        c.append(dict(name=name, E=E, H=H, N=N, D=D, B=B, T=T, pre=pre, dt=dt, Dv=Dv or D,
                      mask=mask, vdt=vdt or dt, scale=scale, v_eye=v_eye))

    # first benchmark configuration, in full
    add("c1_f32_N256_B16_T1", 1, 1, 256, 64, 16, 1, False, "f32")
    # the reference's agreement table (test_ma.py:34-48), in its dtype and in fp32
    match = [(1, 1, 16, 16, 4, 2, False, "f16"), (1, 1, 16, 16, 4, 2, True, "f16"),
             (1, 4, 16, 16, 8, 3, False, "f16"), (1, 1, 19, 16, 4, 2, False, "f16"),
             (1, 1, 19, 16, 4, 2, True, "f16"), (2, 4, 32, 32, 8, 2, False, "f16"),
             (2, 1, 24, 16, 8, 3, False, "f16"), (2, 4, 16, 32, 4, 2, False, "bf16"),
             (1, 1, 16, 32, 4, 2, True, "bf16"), (1, 1, 24, 16, 8, 2, False, "bf16")]
    for i, (E, H, N, D, B, T, pre, dt) in enumerate(match):
        add(f"match{i}_{dt}", E, H, N, D, B, T, pre, dt)
        add(f"match{i}_f32", E, H, N, D, B, T, pre, "f32")
    # masked table (test_ma.py:70-80)
    masked = [(1, 1, 16, 16, 4, 2, False, "f16"), (1, 1, 16, 16, 4, 2, True, "f16"),
              (1, 1, 19, 16, 4, 2, False, "f16"), (1, 4, 19, 16, 4, 3, True, "f16"),
              (1, 1, 32, 16, 8, 2, False, "f16"), (2, 4, 32, 32, 8, 2, False, "f16"),
              (1, 1, 16, 16, 4, 2, True, "bf16"), (2, 4, 16, 32, 4, 2, False, "bf16")]
    for i, (E, H, N, D, B, T, pre, dt) in enumerate(masked):
        add(f"mask{i}_{dt}", E, H, N, D, B, T, pre, dt, mask="safe")
        add(f"mask{i}_f32", E, H, N, D, B, T, pre, "f32", mask="safe")
    # T = 1 tables (test_ma.py:105-109,125-133)
    t1 = [(1, 1, 16, 16, 4, False, "f16"), (2, 4, 19, 32, 8, True, "bf16"),
          (1, 1, 16, 16, 4, True, "f16"), (2, 4, 32, 32, 8, False, "f16"),
          (1, 1, 19, 16, 4, False, "f16"), (1, 1, 19, 16, 4, True, "f16"),
          (2, 4, 16, 32, 4, False, "bf16")]
    for i, (E, H, N, D, B, pre, dt) in enumerate(t1):
        add(f"t1_{i}_{dt}", E, H, N, D, B, 1, pre, dt)
    # behaviours only an execution pins
    for dt in ("f16", "bf16", "f32"):
        add(f"mid_T3_{dt}", 1, 2, 128, 64, 16, 3, False, dt)            # MFMA-sized tiles, T=3
        add(f"ragged_pre_T2_{dt}", 1, 1, 197, 64, 16, 2, True, dt, scale=0.125)   # ViT shape
        add(f"ragged_post_T2_{dt}", 1, 1, 197, 64, 16, 2, False, dt, scale=0.125)
        add(f"d72_T3_{dt}", 1, 1, 128, 72, 32, 3, False, dt)             # DiT head dim
    for dt in ("f16", "bf16"):
        add(f"b32_T2_{dt}", 1, 1, 512, 64, 32, 2, False, dt)             # RoBERTa shape
        add(f"b64_T2_{dt}", 1, 1, 1024, 64, 64, 2, False, dt, mask="tail")  # masked tail, 64x16
    add("matrix_f16_eye32", 1, 2, 48, 32, 8, 2, False, "f16", Dv=48, vdt="f32", v_eye=True)
    add("matrix_f32_eye_ragged", 1, 1, 21, 16, 4, 2, True, "f32", Dv=21, vdt="f32", v_eye=True)
    add("dv_ne_d_f16", 1, 2, 64, 32, 8, 2, False, "f16", Dv=40)
    add("deadblock_f16", 1, 2, 32, 16, 8, 2, False, "f16", mask="dead")
    add("deadblock_f32", 1, 2, 32, 16, 8, 3, False, "f32", mask="dead")
    add("intmask_bf16", 2, 2, 40, 32, 8, 2, False, "bf16", mask="int")
    return c


def main():
    sys.path.insert(0, REF)
    from ma.ma_torch import monarch_attention_torch  # the reference (namespace package)

    n_written = 0
    for c in cases():
        gen = torch.Generator().manual_seed(0)
        E, H, N, D, Dv = c["E"], c["H"], c["N"], c["D"], c["Dv"]
        q = torch.randn(E, H, N, D, generator=gen)
        k = torch.randn(E, H, N, D, generator=gen)
        v = torch.randn(E, H, N, Dv, generator=gen)
        q, k, v = (c["scale"] * t for t in (q, k, v))
        if c["v_eye"]:
            v = torch.eye(N).expand(E, H, N, N).contiguous()
        q, k = q.to(DT[c["dt"]]), k.to(DT[c["dt"]])
        v = v.to(DT[c["vdt"]])
        mask = None
        if c["mask"] == "safe":
            mask = block_safe_mask(E, N, c["B"], gen)
        elif c["mask"] == "tail":                      # keep a prefix per batch entry
            keep = torch.tensor([N - 37 - 11 * e for e in range(E)])
            mask = torch.arange(N)[None, :] < keep[:, None]
        elif c["mask"] == "dead":                      # second key block entirely masked
            mask = torch.ones(E, N, dtype=torch.bool)
            mask[:, c["B"]:2 * c["B"]] = False
        elif c["mask"] == "int":                       # tokenizer-style int64 mask
            mask = (torch.arange(N)[None, :] < torch.tensor([N, N - 13])[:, None]).to(torch.int64)
        with torch.no_grad():
            out = monarch_attention_torch(q, k, v, mask, c["T"], c["B"], c["pre"])
        assert out.shape == (E, H, N, Dv) and out.dtype == v.dtype
        arrays = dict(q=pack(q), k=pack(k), out=pack(out),
                      meta=np.array([E, H, N, D, Dv, c["B"], c["T"], int(c["pre"])], dtype=np.int64),
                      dt=np.array(c["dt"]), vdt=np.array(c["vdt"]), v_eye=np.array(c["v_eye"]))
        if not c["v_eye"]:
            arrays["v"] = pack(v)
        if mask is not None:
            arrays["mask"] = mask.numpy()
        np.savez_compressed(os.path.join(OUT, c["name"] + ".npz"), **arrays)
        n_written += 1
    print(f"wrote {n_written} fixtures to {OUT}")


if __name__ == "__main__":
    main()
