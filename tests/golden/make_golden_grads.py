"""Write gradient fixtures (tests/golden/grads/grad_*.npz) from the reference.

Run ONCE, in the build container only (the reference tree does not travel):

    python tests/golden/make_golden_grads.py [/root/reference [case-name ...]]

The reference has no backward code of its own; training differentiates its
pure-PyTorch forward (``ma/ma_torch.py``, ``monarch_attention_torch``) with
autograd.  This script does exactly that on the CPU for a few seeded cases -
loss ``sum(out * w)`` with a seeded ``w`` - and stores inputs, ``w`` and the
gradients of q, k, v as data.  What only an execution can pin is the
low-precision case: autograd runs the backward matmuls in fp16 / bf16 and
rounds every intermediate gradient.  Nothing in the test-suite, the library
or the benchmark imports this script.
"""

import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from make_golden import DT, block_safe_mask, pack  # noqa: E402

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "grads")

CASES = [  # name, E, H, N, D, Dv, B, T, pre, dtype, mask
    ("grad_f32_T1", 1, 2, 24, 16, 16, 4, 1, False, "f32", None),
    ("grad_f32_T2_mask", 2, 2, 24, 16, 16, 4, 2, False, "f32", "safe"),
    ("grad_f32_T3_ragged_pre", 1, 1, 21, 16, 16, 4, 3, True, "f32", None),
    ("grad_f32_T2_dv", 1, 2, 30, 8, 20, 6, 2, False, "f32", "safe"),
    ("grad_f32_T2_dead", 1, 2, 32, 16, 16, 8, 2, False, "f32", "dead"),
    ("grad_f16_T2", 1, 2, 32, 32, 32, 8, 2, False, "f16", None),
    ("grad_f16_T3_mask_pre", 2, 1, 27, 16, 16, 4, 3, True, "f16", "safe"),
    ("grad_bf16_T2", 1, 2, 32, 32, 32, 8, 2, False, "bf16", "safe"),
    # a long-document training shape (the BART recipe's block size): 64-row blocks on the matrix-core backward kernels
    ("grad_bf16_T2_N512_b64", 1, 1, 512, 64, 64, 64, 2, False, "bf16", None),
]


def main():
    sys.path.insert(0, REF)
    from ma.ma_torch import monarch_attention_torch  # the reference (namespace package)

    os.makedirs(OUT, exist_ok=True)
    only = sys.argv[2:]
    for name, E, H, N, D, Dv, B, T, pre, dt, mk in CASES:
        if only and name not in only:
            continue
        gen = torch.Generator().manual_seed(0)
        q = torch.randn(E, H, N, D, generator=gen).to(DT[dt]).requires_grad_()
        k = torch.randn(E, H, N, D, generator=gen).to(DT[dt]).requires_grad_()
        v = torch.randn(E, H, N, Dv, generator=gen).to(DT[dt]).requires_grad_()
        w = torch.randn(E, H, N, Dv, generator=gen).to(DT[dt])
        mask = None
        if mk == "safe":
            mask = block_safe_mask(E, N, B, gen)
        elif mk == "dead":
            mask = torch.ones(E, N, dtype=torch.bool)
            mask[:, B:2 * B] = False
        out = monarch_attention_torch(q, k, v, mask, T, B, pre)
        (out * w).sum().backward()
        arrays = dict(q=pack(q.detach()), k=pack(k.detach()), v=pack(v.detach()), w=pack(w),
                      dq=pack(q.grad), dk=pack(k.grad), dv=pack(v.grad),
                      meta=np.array([E, H, N, D, Dv, B, T, int(pre)], dtype=np.int64), dt=np.array(dt))
        if mask is not None:
            arrays["mask"] = mask.numpy()
        np.savez_compressed(os.path.join(OUT, name + ".npz"), **arrays)
    print(f"wrote {len(only) or len(CASES)} gradient fixtures to {OUT}")


if __name__ == "__main__":
    main()
