"""CPU oracle for the MonarchAttention forward pass.

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the ``ma`` package, the C-ABI
library, the HIP kernels) may import, call or link this file; only the test
suite, the smoke check and the ``cpu_baseline`` leg of the benchmark use it,
and only as the checker / the timed CPU baseline.

It restates, in plain PyTorch CPU ops, the algorithm of the reference's
``ma/ma_torch.py`` (``monarch_attention_torch`` ``:65-108`` and its four
stage functions ``al_cl_ref :10-23``, ``ar_cr_ref :26-35``, ``al_y_cl_ref
:38-52``, ``z_ref :55-62``).  The restatement keeps the reference's rounding
points and numerical quirks (they are listed next to the code that
reproduces them) but is organised by *stage problem* rather than by tensor
expression, and exposes every intermediate so the HIP stages can be checked
one at a time.

Notation: ``E`` batch, ``H`` heads, ``N`` tokens, ``D`` q/k head dim, ``Dv``
value head dim, ``B`` block size, ``M = ceil(N/B)`` blocks, ``Np = M*B``.
Token ``n = m*B + j`` lives in block ``m`` at in-block position ``j``.

How each function here is pinned (see ``tests/test_oracle_*.py``):

* ``monarch_attention_oracle`` (whole path): golden vectors written from the
  reference in the build container (``tests/golden``), the dense-softmax
  special cases ``M == 1`` (any T) and ``B == 1`` (T = 1), the T = 1 closed
  form, an independent dense L/R alternating-maximisation formulation (after
  ``ma/ma_history.py:15-44``), scalar brute force on tiny inputs, and the
  structural invariants (row-stochastic matrix, masked-key independence,
  batch/head independence, pre-pad == post-pad for divisible N).
* ``r_step`` / ``l_step`` / ``z_step``: through the same checks (they are the
  only code the whole path runs) plus the hand-computable quirk cases (an
  all-masked key block, an all-negative logit row).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

Tensor = torch.Tensor

EPS = 1e-12  # ma/ma_torch.py:10,38 (default ``eps`` of both R-step functions)


# --------------------------------------------------------------------------
# small helpers
# --------------------------------------------------------------------------

def _mm_nt(a: Tensor, b: Tensor, upcast: bool) -> Tensor:
    """``a @ b^T`` over the last two dims, result in ``a.dtype``.

    The reference multiplies in the tensor dtype (``ma_torch.py:11,27,39,56``);
    PyTorch's CPU half/bfloat16 GEMM accumulates in fp32 and rounds once, which
    is what ``upcast=True`` spells out (and is much faster on CPU).
    """
    if upcast and a.dtype != torch.float32:
        return (a.float() @ b.float().transpose(-1, -2)).to(a.dtype)
    return a @ b.transpose(-1, -2)


def _mm_nn(p: Tensor, w: Tensor, upcast: bool) -> Tensor:
    """``round_w(p) @ w``: probabilities are cast to the operand dtype first
    (``ma_torch.py:21,33,49,50,60``)."""
    p = p.to(w.dtype)
    if upcast and w.dtype != torch.float32:
        return (p.float() @ w.float()).to(w.dtype)
    return p @ w


def _pad_tokens(x: Tensor, pad: int, front: bool) -> Tensor:
    """Zero-pad dim -2 by ``pad`` rows at the front or the back (``:81-86``)."""
    if pad == 0:
        return x
    z = x.new_zeros(*x.shape[:-2], pad, x.shape[-1])
    return torch.cat((z, x), dim=-2) if front else torch.cat((x, z), dim=-2)


# --------------------------------------------------------------------------
# the three stage problems
# --------------------------------------------------------------------------

def r_step(aR: Tensor, K: Tensor, cR: Tensor, key_ok: Tensor, sm_scale: float,
           V: Tensor | None = None, *, upcast: bool = False, eps: float = EPS):
    """R update: one ``B x B`` softmax problem per ``(e, h, m)``.

    ``aR, K : (E,H,M,B,D)``, ``cR : (E,H,M,B) f32``, ``key_ok : (.., M, B) bool``
    broadcastable over ``(E,H)``, ``V : (E,H,M,B,Dv)`` or ``None``.

    Returns ``aL (E,H,B,M,D)``, ``cL (E,H,B,M) f32`` and, if ``V`` is given,
    ``Y (E,H,B,M,Dv)`` (``al_cl_ref`` ``ma_torch.py:10-23`` / ``al_y_cl_ref``
    ``:38-52``).  Quirks kept:

    * logits are rounded to the q/k dtype by the matmul *before* the fp32 math;
    * the row maximum is clamped from below by ``eps`` before it is
      subtracted, so an all-negative row is not shifted (``:15,:43``);
    * ``+eps`` in the ``cR`` divisor and in the normaliser (``:12,:17``);
    * probabilities are clamped to ``finfo(float32).tiny`` before ``x log x``
      (``:18,:46``) - an all-masked key block gives ``R = tiny``, no NaN;
    * ``sm_scale *`` is applied to ``aL`` in the low-precision dtype after the
      matmul (``:21,:49``).
    """
    S = _mm_nt(aR, K, upcast).to(torch.float32)          # (E,H,M,Bj,Bi)
    S = sm_scale * S
    S = S / (cR.unsqueeze(-1) + eps)
    S = S.masked_fill(~key_ok.unsqueeze(-2), -math.inf)   # key mask on the i axis
    shift = S.amax(dim=-1, keepdim=True).clamp(min=eps)
    P = torch.exp(S - shift)
    R = P / (P.sum(dim=-1, keepdim=True) + eps)
    R = R.clamp(min=torch.finfo(torch.float32).tiny)

    cL = torch.special.xlogy(R, R).sum(dim=-1).transpose(-1, -2)        # (E,H,B,M)
    aL = (sm_scale * _mm_nn(R, K, upcast)).transpose(-2, -3)            # (E,H,B,M,D)
    if V is None:
        return aL, cL
    Y = _mm_nn(R, V, upcast).transpose(-2, -3)                           # (E,H,B,M,Dv)
    return aL, cL, Y


def l_step(aL: Tensor, Qt: Tensor, cL: Tensor, query_ok_t: Tensor, *, upcast: bool = False):
    """L update: one ``M x M`` softmax problem per ``(e, h, j)``.

    ``aL, Qt : (E,H,B,M,D)``, ``cL : (E,H,B,M) f32``, ``query_ok_t : (.., B, M)``
    (the token mask transposed).  Returns ``aR (E,H,M,B,D)``, ``cR (E,H,M,B) f32``
    (``ar_cr_ref`` ``ma_torch.py:26-35``): the softmax runs over the *key block*
    index ``k`` for every query block ``l``; masked / padded query tokens are
    zeroed after the softmax so they add nothing to ``aR`` / ``cR``.
    """
    G = _mm_nt(aL, Qt, upcast).to(torch.float32)          # (E,H,B,Mk,Ml)
    G = G - cL.unsqueeze(-1)
    L = torch.softmax(G, dim=-2)
    L = query_ok_t.unsqueeze(-2) * L                      # bool * float, as :30

    cR = L.sum(dim=-1).transpose(-1, -2)                  # (E,H,M,B)
    aR = _mm_nn(L, Qt, upcast).transpose(-2, -3)          # (E,H,M,B,D)
    return aR, cR


def z_step(aL: Tensor, Qt: Tensor, cL: Tensor, Y: Tensor, *, upcast: bool = False) -> Tensor:
    """Output stage, per ``(e, h, j)``: ``Z[j,l,:] = softmax_k(Qt.aL^T - cL) @ Y``
    returned block-major ``(E,H,M,B,Dv)`` (``z_ref`` ``ma_torch.py:55-62``)."""
    U = _mm_nt(Qt, aL, upcast).to(torch.float32)          # (E,H,B,Ml,Mk)
    U = U - cL.unsqueeze(-2)
    Lz = torch.softmax(U, dim=-1)
    return _mm_nn(Lz, Y, upcast).transpose(-2, -3).contiguous()


# --------------------------------------------------------------------------
# driver
# --------------------------------------------------------------------------

@dataclass
class OracleTrace:
    """Every intermediate of one forward call (stage-level parity tests)."""
    Qb: Tensor | None = None          # (E,H,M,B,D) padded, block-major
    Kb: Tensor | None = None
    Vb: Tensor | None = None
    token_ok: Tensor | None = None    # (E|1,1,M,B) bool (or (M,B) without attn_mask)
    steps: list = field(default_factory=list)   # dicts: aR,cR (inputs), aL,cL, [Y]
    Zb: Tensor | None = None          # (E,H,M,B,Dv)


def monarch_attention_oracle(q: Tensor, k: Tensor, v: Tensor, attn_mask: Tensor | None,
                             T: int, B: int, pre_pad: bool, *, upcast: bool = False,
                             trace: OracleTrace | None = None) -> Tensor:
    """Forward pass, same contract as ``monarch_attention_torch``
    (``ma/ma_torch.py:65-108``): ``q,k (E,H,N,D)``, ``v (E,H,N,Dv)``,
    ``attn_mask (E,N)`` truthy = keep or ``None``; returns ``(E,H,N,Dv)`` in
    ``v.dtype``.  ``T-1`` (R,L) rounds starting from ``aR = Q, cR = 1`` (i.e.
    ``L = I``), then the R-step that also forms ``Y = R V`` and the Z-step.
    """
    E, H, N, D = q.shape
    Dv = v.shape[-1]
    M = -(-N // B)
    Np = M * B
    pad = Np - N
    sm_scale = 1.0 / math.sqrt(D)

    Qb = _pad_tokens(q, pad, pre_pad).reshape(E, H, M, B, D)
    Kb = _pad_tokens(k, pad, pre_pad).reshape(E, H, M, B, D)
    Vb = _pad_tokens(v, pad, pre_pad).reshape(E, H, M, B, Dv)
    Qt = Qb.transpose(-2, -3)                              # (E,H,B,M,D), a view as in :90

    n = torch.arange(Np, device=q.device).reshape(M, B)
    token_ok = (n >= pad) if pre_pad else (n < N)          # :92-94
    if attn_mask is not None:                              # :96-98
        am = attn_mask.reshape(E, 1, N)
        zeros = am.new_zeros(E, 1, pad)
        am = torch.cat((zeros, am), -1) if pre_pad else torch.cat((am, zeros), -1)
        token_ok = torch.logical_and(token_ok, am.reshape(E, 1, M, B))

    aR = Qb
    cR = torch.ones(E, H, M, B, dtype=torch.float32, device=q.device)
    if trace is not None:
        trace.Qb, trace.Kb, trace.Vb, trace.token_ok = Qb, Kb, Vb, token_ok

    for _ in range(T - 1):
        aL, cL = r_step(aR, Kb, cR, token_ok, sm_scale, upcast=upcast)
        if trace is not None:
            trace.steps.append(dict(aR=aR, cR=cR, aL=aL, cL=cL))
        aR, cR = l_step(aL, Qt, cL, token_ok.transpose(-1, -2), upcast=upcast)

    aL, cL, Y = r_step(aR, Kb, cR, token_ok, sm_scale, Vb, upcast=upcast)
    Zb = z_step(aL, Qt, cL, Y, upcast=upcast)
    if trace is not None:
        trace.steps.append(dict(aR=aR, cR=cR, aL=aL, cL=cL, Y=Y))
        trace.Zb = Zb

    Z = Zb.reshape(E, H, Np, Dv)
    return Z[..., pad:, :] if pre_pad else Z[..., :N, :]


def monarch_matrix_oracle(q: Tensor, k: Tensor, attn_mask: Tensor | None, T: int, B: int,
                          pre_pad: bool, *, upcast: bool = False) -> Tensor:
    """Dense ``(E,H,N,N)`` Monarch attention matrix: the forward pass applied to
    an fp32 identity ``V`` (``MonarchAttention.get_matrix``,
    ``ma/monarch_attention.py:61-66``)."""
    E, H, N, _ = q.shape
    eye = torch.eye(N, device=q.device).expand(E, H, N, N)
    return monarch_attention_oracle(q, k, eye, attn_mask, T, B, pre_pad, upcast=upcast)


# --------------------------------------------------------------------------
# work counts used by the benchmark (matmul FLOPs on padded sizes, the
# reference's ``bmm.default`` convention, experiments/vit/evaluation.py:50-59)
# --------------------------------------------------------------------------

def forward_flops(E: int, H: int, N: int, D: int, Dv: int, B: int, T: int) -> int:
    M = -(-N // B)
    Np = M * B
    per_head = ((T - 1) * (4 * Np * B * D + 4 * Np * M * D)
                + (4 * Np * B * D + 2 * Np * B * Dv)
                + (2 * Np * M * D + 2 * Np * M * Dv))
    return E * H * per_head


def forward_bytes(E: int, H: int, N: int, D: int, Dv: int, elt: int) -> int:
    """Compulsory traffic: read Q, K, V once, write Z once."""
    return E * H * (2 * N * D + 2 * N * Dv) * elt
