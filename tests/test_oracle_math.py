"""Checks that pin the CPU oracle by mathematics alone (no reference output):
special cases that reduce to dense softmax attention, the T = 1 closed form, an
independent dense alternating-maximisation formulation, scalar brute force on
tiny inputs, structural invariants and the hand-computable quirk cases.
Each is chosen so that a plausible slip (a transposed operand, a dropped
``cL``/``cR`` term, softmax over the wrong axis, a wrong pad side) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import seeded_qkv
from oracle.ma_oracle import (forward_bytes, forward_flops, monarch_attention_oracle,
                              monarch_matrix_oracle)

TINY = float(np.finfo(np.float32).tiny)


# ---------------------------------------------------------------- special cases
@pytest.mark.parametrize("T", [1, 2, 3])
@pytest.mark.parametrize("N,B", [(24, 24), (19, 32)])
def test_single_block_is_dense_softmax(N, B, T):
    """B >= N: one block, the L / Z softmaxes run over one element, so any T
    gives softmax(QK^T/sqrt(D)) V."""
    q, k, v = seeded_qkv(2, 3, N, 16, torch.float32)
    out = monarch_attention_oracle(q, k, v, None, T, B, False)
    ref = F.scaled_dot_product_attention(q, k, v)
    assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)


def test_unit_blocks_T1_is_dense_softmax():
    """B = 1, T = 1: R = 1 per block, aL = K/sqrt(D), Y = V and the Z-step is
    dense softmax attention."""
    q, k, v = seeded_qkv(1, 2, 20, 8, torch.float32)
    out = monarch_attention_oracle(q, k, v, None, 1, 1, False)
    ref = F.scaled_dot_product_attention(q, k, v)
    assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)


# ---------------------------------------------------------------- T = 1 closed form
def _closed_form_T1(q, k, v, B):
    """Z[(l,j)] = sum_k softmax_k(q_lj . abar_jk + Hent_jk) (R_k V_k)[j] with
    R_k = rowsoftmax(Q_k K_k^T / sqrt(D)), abar_jk = (R_k K_k)[j] / sqrt(D),
    Hent_jk = -sum_i R_k[j,i] log R_k[j,i]   (fp64, divisible N, no mask)."""
    N, D = q.shape
    M = N // B
    s = 1.0 / math.sqrt(D)
    Q, K, V = (t.double().reshape(M, B, -1) for t in (q, k, v))
    R = torch.softmax(s * torch.einsum("mjd,mid->mji", Q, K), dim=-1)
    abar = s * torch.einsum("mji,mid->mjd", R, K)                   # [k, j, d]
    hent = -(R * R.log()).sum(-1)                                   # [k, j]
    y = torch.einsum("mji,mid->mjd", R, V)                          # [k, j, dv]
    logit = torch.einsum("ljd,kjd->ljk", Q, abar) + hent.t()[None]  # [l, j, k]
    w = torch.softmax(logit, dim=-1)
    return torch.einsum("ljk,kjd->ljd", w, y).reshape(N, -1)


@pytest.mark.parametrize("N,B,D", [(32, 8, 16), (48, 4, 8), (36, 12, 24)])
def test_T1_closed_form(N, B, D):
    q, k, v = seeded_qkv(1, 1, N, D, torch.float32, Dv=D + 3)
    out = monarch_attention_oracle(q, k, v, None, 1, B, False)[0, 0]
    ref = _closed_form_T1(q[0, 0], k[0, 0], v[0, 0], B)
    assert torch.allclose(out.double(), ref, atol=3e-6, rtol=1e-5)


# ---------------------------------------------------------------- dense alternating formulation
def _dense_monarch(q, k, T, B):
    """Dense L (B,M,M), R (M,B,B) iterated T times from L = I, returned as the
    N x N matrix A[(l,j),(k,i)] = L[j,k,l] R[k,j,i] (independent statement of
    the method, after ma/ma_history.py:15-44; fp64, divisible N, no mask)."""
    N, D = q.shape
    M = N // B
    qb = (q.double() / math.sqrt(D)).reshape(M, B, D)      # [l, j, d]
    kb = k.double().reshape(M, B, D)                        # [k, i, d]
    L = torch.eye(M, dtype=torch.float64).repeat(B, 1, 1)   # [j, k, l]
    for _ in range(T):
        a = torch.einsum("jkl,ljd->kjd", L, qb)
        c = L.sum(-1).t()                                   # [k, j]
        R = torch.softmax(torch.einsum("kjd,kid->kji", a, kb) / c[:, :, None], dim=-1)
        a = torch.einsum("kji,kid->jkd", R, kb)
        ent = (R * R.log()).sum(-1).t()                     # [j, k]
        L = torch.softmax(torch.einsum("jkd,ljd->jkl", a, qb) - ent[:, :, None], dim=1)
    A = torch.einsum("jkl,kji->ljki", L, R)
    return A.reshape(N, N)


@pytest.mark.parametrize("T", [1, 2, 3, 4])
@pytest.mark.parametrize("N,B,D", [(32, 8, 16), (24, 4, 8), (30, 10, 12)])
def test_dense_alternating_formulation(N, B, D, T):
    q, k, v = seeded_qkv(1, 1, N, D, torch.float32, scale=0.7)
    A = _dense_monarch(q[0, 0], k[0, 0], T, B)
    out = monarch_attention_oracle(q, k, v, None, T, B, False)[0, 0]
    assert torch.allclose(out.double(), A @ v[0, 0].double(), atol=1e-5, rtol=1e-4)
    mat = monarch_matrix_oracle(q, k, None, T, B, False)[0, 0]
    assert torch.allclose(mat.double(), A, atol=2e-6, rtol=1e-4)


# ---------------------------------------------------------------- scalar brute force
def _brute(q, k, v, keep, T, B, pre_pad, eps=1e-12):
    """Plain-loop statement of the method with every quirk (clamped row max,
    +eps denominators, tiny clamp, key mask as -inf, query mask after the L
    softmax, zero padding at either end), python floats, tiny inputs only."""
    N, D = q.shape
    Dv = v.shape[1]
    M = -(-N // B)
    Np = M * B
    pad = Np - N
    off = pad if pre_pad else 0
    s = 1.0 / math.sqrt(D)

    def row(x, n, width):
        t = n - off
        return x[t].tolist() if 0 <= t < N else [0.0] * width

    ok = [[(0 <= m * B + j - off < N) and bool(keep[m * B + j - off]) for j in range(B)] for m in range(M)]
    Q = [[row(q, m * B + j, D) for j in range(B)] for m in range(M)]
    K = [[row(k, m * B + j, D) for j in range(B)] for m in range(M)]
    V = [[row(v, m * B + j, Dv) for j in range(B)] for m in range(M)]
    dot = lambda a, b: sum(x * y for x, y in zip(a, b))

    aR = [[list(Q[m][j]) for j in range(B)] for m in range(M)]
    cR = [[1.0] * B for _ in range(M)]
    for step in range(T):
        last = step == T - 1
        aL = [[None] * M for _ in range(B)]
        cL = [[0.0] * M for _ in range(B)]
        Y = [[None] * M for _ in range(B)]
        for m in range(M):
            for j in range(B):
                logit = [s * dot(aR[m][j], K[m][i]) / (cR[m][j] + eps) if ok[m][i] else -math.inf
                         for i in range(B)]
                mx = max(max(logit), eps)
                p = [math.exp(x - mx) for x in logit]
                den = sum(p) + eps
                r = [max(x / den, TINY) for x in p]
                cL[j][m] = sum(x * math.log(x) for x in r)
                aL[j][m] = [s * sum(r[i] * K[m][i][d] for i in range(B)) for d in range(D)]
                Y[j][m] = [sum(r[i] * V[m][i][d] for i in range(B)) for d in range(Dv)]
        if last:
            break
        aR = [[[0.0] * D for _ in range(B)] for _ in range(M)]
        cR = [[0.0] * B for _ in range(M)]
        for j in range(B):
            for l in range(M):
                u = [dot(aL[j][kk], Q[l][j]) - cL[j][kk] for kk in range(M)]
                mx = max(u)
                e = [math.exp(x - mx) for x in u]
                den = sum(e)
                for kk in range(M):
                    w = e[kk] / den if ok[l][j] else 0.0
                    cR[kk][j] += w
                    for d in range(D):
                        aR[kk][j][d] += w * Q[l][j][d]
    Z = np.zeros((Np, Dv))
    for j in range(B):
        for l in range(M):
            u = [dot(Q[l][j], aL[j][kk]) - cL[j][kk] for kk in range(M)]
            mx = max(u)
            e = [math.exp(x - mx) for x in u]
            den = sum(e)
            for kk in range(M):
                Z[l * B + j] += (e[kk] / den) * np.array(Y[j][kk])
    return Z[off:off + N]


BRUTE = [  # N, D, Dv, B, T, pre_pad, mask kind
    (8, 4, 4, 4, 1, False, None), (8, 4, 3, 2, 2, False, None), (12, 4, 5, 4, 3, False, None),
    (11, 4, 4, 4, 2, False, None), (11, 4, 4, 4, 2, True, None), (7, 3, 2, 3, 3, True, None),
    (12, 4, 4, 4, 2, False, "rand"), (13, 4, 4, 4, 3, True, "rand"), (12, 4, 4, 4, 2, False, "dead"),
    (10, 4, 4, 5, 2, False, "tail"), (9, 2, 2, 3, 4, False, "rand"),
]


@pytest.mark.parametrize("N,D,Dv,B,T,pre,mk", BRUTE)
def test_scalar_brute_force(N, D, Dv, B, T, pre, mk):
    q, k, v = seeded_qkv(1, 1, N, D, torch.float32, Dv=Dv, seed=3)
    keep = torch.ones(N, dtype=torch.bool)
    if mk == "rand":
        keep = torch.rand(N, generator=torch.Generator().manual_seed(5)) > 0.35
    elif mk == "dead":
        keep[B:2 * B] = False
    elif mk == "tail":
        keep[N - 3:] = False
    mask = None if mk is None else keep[None]
    out = monarch_attention_oracle(q, k, v, mask, T, B, pre)[0, 0]
    ref = _brute(q[0, 0].double().numpy(), k[0, 0].double().numpy(), v[0, 0].double().numpy(),
                 keep.numpy(), T, B, pre)
    assert np.allclose(out.double().numpy(), ref, atol=2e-5, rtol=1e-4)


# ---------------------------------------------------------------- quirks with hand-computable answers
def test_dead_key_block_competes_with_logit_zero():
    """T = 1, one key block fully masked: its R rows are `tiny`, aL = Y = 0 and
    cL ~ 0, so in the Z softmax it holds logit 0: it takes probability mass and
    contributes nothing (no NaN)."""
    N, B, D = 16, 4, 8
    q, k, v = seeded_qkv(1, 1, N, D, torch.float32, seed=7)
    keep = torch.ones(1, N, dtype=torch.bool)
    keep[:, 4:8] = False
    out = monarch_attention_oracle(q, k, v, keep, 1, B, False)[0, 0].double()
    assert torch.isfinite(out).all()
    M, s = N // B, 1.0 / math.sqrt(D)
    Q, K, V = (t[0, 0].double().reshape(M, B, -1) for t in (q, k, v))
    R = torch.softmax(s * torch.einsum("mjd,mid->mji", Q, K), dim=-1)
    abar = s * torch.einsum("mji,mid->mjd", R, K)
    hent = -(R * R.log()).sum(-1)
    y = torch.einsum("mji,mid->mjd", R, V)
    logit = torch.einsum("ljd,kjd->ljk", Q, abar) + hent.t()[None]
    logit[:, :, 1] = 0.0                                   # the dead block
    y[1] = 0.0
    ref = torch.einsum("ljk,kjd->ljd", torch.softmax(logit, -1), y).reshape(N, -1)
    assert torch.allclose(out, ref, atol=3e-6, rtol=1e-5)


def test_all_negative_row_is_not_max_shifted():
    """Rows whose logits are all below eps subtract eps, not their maximum:
    with logits ~ -40 the un-normalised weights underflow towards the +eps in
    the denominator and the row sums to less than one."""
    N = B = 4
    D = 4
    q = torch.full((1, 1, N, D), 4.0)
    k = torch.full((1, 1, N, D), -5.0)                     # logits = -80/2 = -40
    v = torch.ones(1, 1, N, 1)
    out = monarch_attention_oracle(q, k, v, None, 1, B, False)[0, 0, :, 0].double()
    p = math.exp(-40.0)
    expect = (N * p) / (N * p + 1e-12)                     # row mass of R; Z softmax over one block = 1
    assert expect < 0.9999
    assert torch.allclose(out, torch.full((N,), expect, dtype=torch.float64), rtol=2e-4)


# ---------------------------------------------------------------- invariants
@pytest.mark.parametrize("T", [1, 2, 3])
def test_matrix_rows_are_distributions(T):
    q, k, _ = seeded_qkv(2, 2, 24, 8, torch.float32)
    A = monarch_matrix_oracle(q, k, None, T, 6, False)
    assert A.shape == (2, 2, 24, 24) and A.dtype == torch.float32
    assert (A >= 0).all()
    assert torch.allclose(A.sum(-1), torch.ones(2, 2, 24), atol=1e-5)


def test_mixed_dtype_value_sets_output_dtype():
    q, k, _ = seeded_qkv(1, 2, 16, 8, torch.float16)
    A = monarch_matrix_oracle(q, k, None, 2, 4, True)
    assert A.dtype == torch.float32 and A.shape == (1, 2, 16, 16)
    assert torch.allclose(A.sum(-1), torch.ones(1, 2, 16), atol=2e-3)


@pytest.mark.parametrize("pre", [False, True])
def test_masked_and_padded_keys_do_not_matter(pre):
    q, k, v = seeded_qkv(2, 2, 22, 8, torch.float32)
    keep = torch.rand(2, 22, generator=torch.Generator().manual_seed(2)) > 0.3
    keep[:, ::4] = True
    a = monarch_attention_oracle(q, k, v, keep, 2, 4, pre)
    k2, v2 = k.clone(), v.clone()
    k2[~keep[:, None].expand(2, 2, 22)] = 37.0
    v2[~keep[:, None].expand(2, 2, 22)] = -91.0
    b = monarch_attention_oracle(q, k2, v2, keep, 2, 4, pre)
    assert torch.equal(a, b)


def test_pre_pad_equals_post_pad_when_divisible():
    q, k, v = seeded_qkv(1, 2, 24, 8, torch.float32)
    assert torch.equal(monarch_attention_oracle(q, k, v, None, 3, 6, True),
                       monarch_attention_oracle(q, k, v, None, 3, 6, False))


def test_batch_and_head_independence():
    q, k, v = seeded_qkv(3, 2, 19, 8, torch.float32)
    keep = torch.rand(3, 19, generator=torch.Generator().manual_seed(4)) > 0.2
    full = monarch_attention_oracle(q, k, v, keep, 2, 4, True)
    one = monarch_attention_oracle(q[1:2, 1:2], k[1:2, 1:2], v[1:2, 1:2], keep[1:2], 2, 4, True)
    assert torch.allclose(full[1:2, 1:2], one, atol=1e-6)


def test_block_permutation_equivariance():
    """Permuting whole blocks of q, k, v the same way permutes the output."""
    q, k, v = seeded_qkv(1, 1, 24, 8, torch.float32)
    perm = torch.tensor([2, 0, 3, 1])
    idx = (perm[:, None] * 6 + torch.arange(6)[None]).reshape(-1)
    a = monarch_attention_oracle(q, k, v, None, 2, 6, False)
    b = monarch_attention_oracle(q[:, :, idx], k[:, :, idx], v[:, :, idx], None, 2, 6, False)
    assert torch.allclose(a[:, :, idx], b, atol=2e-6)


def test_mask_truthiness_bool_int_float_agree():
    q, k, v = seeded_qkv(2, 1, 16, 8, torch.float32)
    keep = torch.arange(16)[None] < torch.tensor([16, 9])[:, None]
    a = monarch_attention_oracle(q, k, v, keep, 2, 4, False)
    assert torch.equal(a, monarch_attention_oracle(q, k, v, keep.long(), 2, 4, False))
    assert torch.equal(a, monarch_attention_oracle(q, k, v, keep.float(), 2, 4, False))


def test_sum_of_cR_counts_valid_query_blocks():
    from oracle.ma_oracle import OracleTrace
    q, k, v = seeded_qkv(1, 1, 22, 8, torch.float32)
    tr = OracleTrace()
    monarch_attention_oracle(q, k, v, None, 3, 4, False, trace=tr)
    cR = tr.steps[-1]["cR"][0, 0]                          # (M, B), sum over key blocks k
    valid = tr.token_ok.sum(0).float()                     # valid query blocks per position j
    assert torch.allclose(cR.sum(0), valid, atol=1e-5)


# ---------------------------------------------------------------- work counts
def test_flop_and_byte_formulas():
    # metric configuration: fp16 E1 H16 N4096 D64 B64, T = 1, 2, 3
    assert [round(forward_flops(1, 16, 4096, 64, 64, 64, T) / 1e9, 2) for T in (1, 2, 3)] == [2.68, 4.83, 6.98]
    assert round(forward_bytes(1, 16, 4096, 64, 64, 2) / 1e6, 1) == 33.6
    assert round(forward_flops(1, 16, 16384, 64, 64, 128, 3) / 1e9, 1) == 55.8
    assert round(forward_flops(64, 12, 197, 64, 64, 16, 2) / 1e9, 2) == 2.70
