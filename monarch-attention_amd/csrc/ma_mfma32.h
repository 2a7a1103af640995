// fp32 stage kernels on the matrix cores: v_mfma_f32_16x16x4_f32 (fp32 operands,
// fp32 accumulate) for the R, L and Z steps of monarch_attention_torch
// (ma/ma_torch.py:10-62) when q, k, v are fp32.  Same structure as the 16-bit
// kernels - GEMM1 -> softmax in registers -> GEMM2, one wave per 16-row strip,
// the waves of a problem sharing its operand tiles in LDS - but nothing is
// rounded between the stages (the reference rounds to the operand dtype, which
// is fp32 here), and the operands are single floats per lane:
//
//   16x16x4:  A (16 x 4): lane holds A[r][q]     B (4 x 16): lane holds B[q][r]
//             C / D (16 x 16): lane holds column r, rows 4q .. 4q+3
//   with r = lane % 16, q = lane / 16.
//
// GEMM1  C[w, x] = sum_d W[w, d] X[x, d]: the contraction index is walked as
//        d = 16 t + 4 q + u (t = 16-column group, u = 0..3), so that a lane's A
//        values for one t are ONE 16-byte LDS read of row w and its B values ONE
//        16-byte global load of row x; four MFMAs consume them.
// GEMM2  out^T[d, x] = sum_w Wv[w, d] P[w, x]: k slot q of step (wt, v) is row
//        w = 16 wt + 4 q + v - exactly the C register C[wt][v] the lane already
//        holds as the B value; the A value Wv[w][16 dt + r] is a 4-byte LDS read
//        (the 16 lanes of a group read 16 consecutive floats of one row).
//        The result lands as 4 consecutive d per lane: one 16-byte store.
#pragma once

#include "ma_mfma.h"

namespace ma {
namespace mfma32 {

using mfma::bload16;
using mfma::bloadf;
using mfma::f32x4;
using mfma::kLn2;
using mfma::kLog2e;
using mfma::kNegBig;
using mfma::kOob;
using mfma::make_slices;
using mfma::mask_load;
using mfma::quad_rows_max;
using mfma::quad_rows_sum;
using mfma::rcp;
using mfma::row16_max;
using mfma::row16_sum;
using mfma::rsrc_t;
using mfma::Slices;
using mfma::Split;
using mfma::tok_off;
using mfma::token_kept;
using mfma::u32x4;
using mfma::wave_id;

__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// LDS tile geometry for DTF 16-column groups (D <= 16 DTF): row pitch in floats; the +4 staggers
// consecutive rows by 16 bytes
template <int DTF>
struct Geom32 {
    static constexpr int COLS = 16 * DTF;
    static constexpr int LD = COLS + 4;
};

template <int DTF, int NWT>
struct Lds32 {
    static constexpr int ROWS = 16 * NWT;
    static constexpr int TILE = ROWS * Geom32<DTF>::LD;      // floats
    static constexpr int LDP = ROWS + 4;                     // pitch of the transposed L tile PT[k][l]
    static constexpr size_t R = (2 * TILE + ROWS) * sizeof(float);
    static constexpr size_t Z = (2 * TILE + ROWS) * sizeof(float);
    static constexpr size_t L = (2 * TILE + ROWS * LDP + (1 + Split<NWT>::WPP) * ROWS) * sizeof(float);
};

// Cooperative global -> LDS copy of a ROWS-row tile of 16-byte chunks by NTH threads, in two halves
// so that a problem can put ALL its loads in flight before it waits for any of them: issue() starts
// the loads into registers, commit() writes them to LDS.  rowoff(row) = byte offset of the row in
// src or kOob (rows beyond the problem and columns at or beyond D are zero-filled by the bounds check).
template <int DTF, int ROWS, int NTH>
struct TileCopy32 {
    static constexpr int CH = 4 * DTF;   // chunks per row
    static constexpr int CNT = ROWS * CH / NTH;
    static_assert(ROWS * CH % NTH == 0, "tile chunks must divide evenly among the threads");
    u32x4 val[CNT];
    template <class RowOff>
    __device__ __forceinline__ void issue(rsrc_t src, int D, RowOff rowoff, int tix) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * NTH;
            const int row = c / CH, ch = c % CH;
            const unsigned ro = rowoff(row);
            val[i] = bload16<true>(src, (ch * 4 < D) ? ro + ch * 16 : kOob);
        }
    }
    __device__ __forceinline__ void commit(float* tile, int tix) const {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * NTH;
            *reinterpret_cast<u32x4*>(tile + (c / CH) * Geom32<DTF>::LD + (c % CH) * 4) = val[i];
        }
    }
};

// this lane's 16-byte pieces (columns 16 t + 4 q ..) of the row at byte offset ro (or kOob)
template <int DTF>
__device__ __forceinline__ void load_row(f32x4 (&x)[DTF], rsrc_t src, unsigned ro, int D, int q) {
#pragma unroll
    for (int t = 0; t < DTF; ++t) {
        const int col = 16 * t + 4 * q;
        x[t] = __builtin_bit_cast(f32x4, bload16<true>(src, col < D ? ro + col * 4 : kOob));
    }
}

// GEMM1 tile: acc[v] = sum_d W[16 wt + .., d] X[x, d] with W rows in an LDS tile and X in registers
template <int DTF>
__device__ __forceinline__ f32x4 gemm1_tile(const float* wrow /* tile row 16 wt + r, column 4 q */, const f32x4 (&x)[DTF]) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < DTF; ++t) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(wrow + 16 * t);
#pragma unroll
        for (int u = 0; u < 4; ++u) acc = mma4(a[u], x[t][u], acc);
    }
    return acc;
}

// GEMM2: O[dt][v] = sum_w tile[w][16 dt + 4 q + v'] ... as out^T: rows d = 16 dt + 4 q + v, column x = r
template <int DTF, int NWT>
__device__ __forceinline__ void gemm2(f32x4 (&O)[DTF], const float* tile, const f32x4 (&C)[NWT], int r, int q) {
#pragma unroll
    for (int dt = 0; dt < DTF; ++dt) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc = mma4(tile[(16 * wt + 4 * q + v) * Geom32<DTF>::LD + 16 * dt + r], C[wt][v], acc);
        O[dt] = acc;
    }
}

// lane's 4 consecutive output floats per 16-column group (columns 16 dt + 4 q ..) of the row at ro
template <int DTF>
__device__ __forceinline__ void store_row(rsrc_t dst, unsigned ro, int D, const f32x4 (&O)[DTF], int q) {
#pragma unroll
    for (int dt = 0; dt < DTF; ++dt) {
        const int col = 16 * dt + 4 * q;
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, O[dt]), dst, col < D ? ro + col * 4 : kOob, 0, 0);
    }
}

// (e, h, index) of the block problem a workgroup runs; E * H * Np fits int32 (validated by the host)
struct Which {
    int e, h, idx;
    long long eh;
    bool active;
};
__device__ __forceinline__ Which which_problem(const Problem& P, int count, int parts = 1) {
    Which w;
    const unsigned total = static_cast<unsigned>(P.E) * P.H * count;
    unsigned pid = blockIdx.x / static_cast<unsigned>(parts);
    w.active = pid < total;
    if (!w.active) pid = 0;
    w.idx = pid % static_cast<unsigned>(count);
    const unsigned eh = pid / static_cast<unsigned>(count);
    w.h = eh % static_cast<unsigned>(P.H);
    w.e = eh / static_cast<unsigned>(P.H);
    w.eh = eh;
    return w;
}

// ---------------------------------------------------------------- R step: al_cl_ref / al_y_cl_ref (ma/ma_torch.py:10-23, :38-52)
// HV = 2: a problem whose waves walk two strips each is run as two workgroups of one strip per wave (workgroups
// 2 p and 2 p + 1; both stage the whole key / value tiles).  The fp32 matrix instructions of a strip are one
// dependent chain per accumulator, so a wave's time is its strips' MFMA count: a launch that leaves compute
// units idle asks for the halves (the graph-transformer shape: 120 problems of 128 rows on 256 compute units).
template <int DTF, int NWT, int HV = 1>
__global__ __launch_bounds__(64 * Split<NWT>::WPP) void r_step_f32(Problem P, int first_i, int with_v_i) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, SPW = NWT / WPP / HV, ROWS = 16 * NWT, LD = Geom32<DTF>::LD;
    static_assert(NWT % (WPP * HV) == 0, "a half must be whole strips per wave");
    const int half = HV == 1 ? 0 : static_cast<int>(blockIdx.x % HV);
    float* Kt = reinterpret_cast<float*>(smem);
    float* Vt = Kt + Lds32<DTF, NWT>::TILE;
    float* kbias = Vt + Lds32<DTF, NWT>::TILE;
    const bool first = first_i != 0, with_v = with_v_i != 0;
    const int wig = wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4, tix = threadIdx.x;
    const Which w = which_problem(P, P.M, HV);
    if (!w.active) return;
    const int B = P.B, M = P.M, D = P.D, m = w.idx;
    const Slices S = make_slices<float>(P, w.e, w.h, w.eh);
    const unsigned db = static_cast<unsigned>(D) * 4u;
    const int t0 = m * B - P.pad_off;

    {
        TileCopy32<DTF, ROWS, 64 * WPP> kc, vc;
        kc.issue(S.k, D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.kst) : kOob; }, tix);
        if (with_v) vc.issue(S.v, D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.vst) : kOob; }, tix);
        kc.commit(Kt, tix);
        if (with_v) vc.commit(Vt, tix);
    }
    for (int i = tix; i < ROWS; i += 64 * WPP)
        kbias[i] = (i < B && token_kept(P, t0 + i, mask_load(S, P, t0 + i, i < B))) ? 0.f : kNegBig;
    __syncthreads();

#pragma unroll
    for (int si = 0; si < SPW; ++si) {
        const int j = 16 * (half * (NWT / HV) + wig + si * WPP) + r;
        const bool jv = j < B;
        f32x4 xb[DTF];
        float cr = 1.0f;
        if (first) {
            load_row<DTF>(xb, S.q, jv ? tok_off(t0 + j, P.N, S.qst) : kOob, D, q);
        } else {
            const unsigned rowid = static_cast<unsigned>(m * B + j);
            load_row<DTF>(xb, S.aR, jv ? rowid * db : kOob, D, q);
            cr = bloadf<true>(S.cR, jv ? rowid * 4u : kOob);   // an out-of-range row reads 0: harmless, never stored
        }
        const float cj = (P.sm_scale * kLog2e) * rcp(cr + P.eps);   // logits in log2 units
        f32x4 C[NWT];
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt) {
            const f32x4 acc = gemm1_tile<DTF>(Kt + (16 * wt + r) * LD + 4 * q, xb);
            const f32x4 kb = *reinterpret_cast<const f32x4*>(kbias + 16 * wt + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) C[wt][v] = fmaf(acc[v], cj, kb[v]);
        }
        // clamped row maximum (ma_torch.py:15): max(rowmax, eps), here in log2 units
        float mx = C[0][0];
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) mx = fmaxf(mx, C[wt][v]);
        mx = fmaxf(quad_rows_max(mx), P.eps * kLog2e);
        float sum = 0.f, ent = 0.f;
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float d = C[wt][v] - mx;
                const float p = __builtin_amdgcn_exp2f(d);
                sum += p;
                ent = fmaf(p, d, ent);   // sum p * log2(p)
                C[wt][v] = p;
            }
        sum = quad_rows_sum(sum);
        ent = quad_rows_sum(ent);
        const float den = sum + P.eps, inv = rcp(den);
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) C[wt][v] *= inv;
        const unsigned lrow = static_cast<unsigned>(j * M + m);   // row of aL / cL / Y: (j, m)
        // cL = sum_i r log r with r = p / den (ma_torch.py:20)
        if (q == 0)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, kLn2 * ent * inv - __logf(den) * (sum * inv)), S.cL,
                                                  jv ? lrow * 4u : kOob, 0, 0);
        {
            f32x4 O[DTF];
            gemm2<DTF, NWT>(O, Kt, C, r, q);
#pragma unroll
            for (int dt = 0; dt < DTF; ++dt)
#pragma unroll
                for (int v = 0; v < 4; ++v) O[dt][v] *= P.sm_scale;
            store_row<DTF>(S.aL, jv ? lrow * db : kOob, D, O, q);
        }
        if (with_v) {
            f32x4 O[DTF];
            gemm2<DTF, NWT>(O, Vt, C, r, q);
            store_row<DTF>(S.Y, jv ? lrow * db : kOob, D, O, q);
        }
    }
}

// ---------------------------------------------------------------- Z step: z_ref (ma/ma_torch.py:55-62) and the final slice (:106-108)
template <int DTF, int NWT>
__global__ __launch_bounds__(64 * Split<NWT>::WPP) void z_step_f32(Problem P) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, SPW = NWT / WPP, ROWS = 16 * NWT, LD = Geom32<DTF>::LD;
    float* At = reinterpret_cast<float*>(smem);
    float* Yt = At + Lds32<DTF, NWT>::TILE;
    float* cb = Yt + Lds32<DTF, NWT>::TILE;
    const int wig = wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4, tix = threadIdx.x;
    const Which w = which_problem(P, P.B);
    if (!w.active) return;
    const int B = P.B, M = P.M, D = P.D, j = w.idx;
    const Slices S = make_slices<float>(P, w.e, w.h, w.eh);
    const unsigned db = static_cast<unsigned>(D) * 4u;
    const unsigned row0 = static_cast<unsigned>(j * M);

    {
        TileCopy32<DTF, ROWS, 64 * WPP> ac, yc;
        ac.issue(S.aL, D, [&](int k) { return k < M ? (row0 + k) * db : kOob; }, tix);
        yc.issue(S.Y, D, [&](int k) { return k < M ? (row0 + k) * db : kOob; }, tix);
        ac.commit(At, tix);
        yc.commit(Yt, tix);
    }
    for (int k = tix; k < ROWS; k += 64 * WPP) cb[k] = k < M ? -kLog2e * bloadf<true>(S.cL, (row0 + k) * 4u) : kNegBig;
    __syncthreads();

#pragma unroll
    for (int si = 0; si < SPW; ++si) {
        const int l = 16 * (wig + si * WPP) + r;
        const int t = l * B + j - P.pad_off;
        f32x4 xb[DTF];
        load_row<DTF>(xb, S.q, l < M ? tok_off(t, P.N, S.qst) : kOob, D, q);
        f32x4 C[NWT];
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt) {
            const f32x4 acc = gemm1_tile<DTF>(At + (16 * wt + r) * LD + 4 * q, xb);
            const f32x4 b = *reinterpret_cast<const f32x4*>(cb + 16 * wt + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) C[wt][v] = fmaf(acc[v], kLog2e, b[v]);
        }
        float mx = C[0][0];
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) mx = fmaxf(mx, C[wt][v]);
        mx = quad_rows_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float p = __builtin_amdgcn_exp2f(C[wt][v] - mx);
                sum += p;
                C[wt][v] = p;
            }
        const float inv = rcp(quad_rows_sum(sum));
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) C[wt][v] *= inv;
        f32x4 O[DTF];
        gemm2<DTF, NWT>(O, Yt, C, r, q);
        store_row<DTF>(S.out, l < M ? tok_off(t, P.N, S.ost) : kOob, D, O, q);   // padded query rows are dropped (:108)
    }
}

// ---------------------------------------------------------------- L step: ar_cr_ref (ma/ma_torch.py:26-35)
template <int DTF, int NWT>
__global__ __launch_bounds__(64 * Split<NWT>::WPP) void l_step_f32(Problem P) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, SPW = NWT / WPP, ROWS = 16 * NWT, LD = Geom32<DTF>::LD, LDP = Lds32<DTF, NWT>::LDP;
    float* Qt = reinterpret_cast<float*>(smem);
    float* At = Qt + Lds32<DTF, NWT>::TILE;
    float* PT = At + Lds32<DTF, NWT>::TILE;   // PT[k][l]: the L values, key block major
    float* cb = PT + ROWS * LDP;
    float* crp = cb + ROWS;                    // [WPP][ROWS]
    const int wig = wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4, tix = threadIdx.x;
    const Which w = which_problem(P, P.B);
    if (!w.active) return;
    const int B = P.B, M = P.M, D = P.D, j = w.idx;
    const Slices S = make_slices<float>(P, w.e, w.h, w.eh);
    const unsigned db = static_cast<unsigned>(D) * 4u;
    const unsigned row0 = static_cast<unsigned>(j * M);

    {
        TileCopy32<DTF, ROWS, 64 * WPP> qc, ac;
        qc.issue(S.q, D, [&](int l) { return l < M ? tok_off(l * B + j - P.pad_off, P.N, S.qst) : kOob; }, tix);
        ac.issue(S.aL, D, [&](int k) { return k < M ? (row0 + k) * db : kOob; }, tix);
        qc.commit(Qt, tix);
        ac.commit(At, tix);
    }
    for (int k = tix; k < ROWS; k += 64 * WPP) cb[k] = k < M ? -kLog2e * bloadf<true>(S.cL, (row0 + k) * 4u) : kNegBig;
    __syncthreads();

    // phase 1: L[l, k] for 16-row strips of l; lane holds column k = 16 kt + r, rows l0 + 4 q + v
    float crsum[NWT];
#pragma unroll
    for (int kt = 0; kt < NWT; ++kt) crsum[kt] = 0.f;
#pragma unroll
    for (int si = 0; si < SPW; ++si) {
        const int l0 = 16 * (wig + si * WPP);
        f32x4 xa[DTF];   // this lane's pieces of query row l0 + r
#pragma unroll
        for (int t = 0; t < DTF; ++t) xa[t] = *reinterpret_cast<const f32x4*>(Qt + (l0 + r) * LD + 16 * t + 4 * q);
        f32x4 C[NWT];
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < DTF; ++t) {
                const f32x4 b = *reinterpret_cast<const f32x4*>(At + (16 * kt + r) * LD + 16 * t + 4 * q);
#pragma unroll
                for (int u = 0; u < 4; ++u) acc = mma4(xa[t][u], b[u], acc);
            }
            const float bias = cb[16 * kt + r];
#pragma unroll
            for (int v = 0; v < 4; ++v) C[kt][v] = fmaf(acc[v], kLog2e, bias);
        }
        f32x4 mx = C[0];
#pragma unroll
        for (int kt = 1; kt < NWT; ++kt)
#pragma unroll
            for (int v = 0; v < 4; ++v) mx[v] = fmaxf(mx[v], C[kt][v]);
#pragma unroll
        for (int v = 0; v < 4; ++v) mx[v] = row16_max(mx[v]);
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float p = __builtin_amdgcn_exp2f(C[kt][v] - mx[v]);
                sum[v] += p;
                C[kt][v] = p;
            }
        f32x4 inv;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            // padded / masked query tokens are zeroed after the softmax (ma_torch.py:30)
            const int l = l0 + 4 * q + v;
            const int t = l * B + j - P.pad_off;
            const float sv = row16_sum(sum[v]);
            inv[v] = (l < M && token_kept(P, t, mask_load(S, P, t, l < M))) ? rcp(sv) : 0.f;
        }
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt) {
            f32x4 o;
            float part = 0.f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                o[v] = C[kt][v] * inv[v];
                part += o[v];
            }
            crsum[kt] += part;
            *reinterpret_cast<f32x4*>(PT + (16 * kt + r) * LDP + l0 + 4 * q) = o;
        }
    }
#pragma unroll
    for (int kt = 0; kt < NWT; ++kt) {
        const float sv = quad_rows_sum(crsum[kt]);
        if (q == 0) crp[wig * ROWS + 16 * kt + r] = sv;
    }
    __syncthreads();

    // phase 2: aR[k, :] = sum_l L[l, k] Qt[l, :] for 16-wide tiles of k; out^T rows d, column k = r
    for (int kt = wig; kt < NWT; kt += WPP) {
        const int k = 16 * kt + r;
        const bool kv = k < M;
        f32x4 pl[NWT];   // L[16 lt + 4 q + v][k]
#pragma unroll
        for (int lt = 0; lt < NWT; ++lt) pl[lt] = *reinterpret_cast<const f32x4*>(PT + k * LDP + 16 * lt + 4 * q);
        f32x4 O[DTF];
        gemm2<DTF, NWT>(O, Qt, pl, r, q);
        const unsigned arow = static_cast<unsigned>(k * B + j);   // row of aR / cR: (k, j)
        store_row<DTF>(S.aR, kv ? arow * db : kOob, D, O, q);
        if (q == 0) {
            float sv = 0.f;
#pragma unroll
            for (int wv = 0; wv < WPP; ++wv) sv += crp[wv * ROWS + k];
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, sv), S.cR, kv ? arow * 4u : kOob, 0, 0);
        }
    }
}

}  // namespace mfma32
}  // namespace ma
