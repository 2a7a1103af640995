// fp32 forward pass with a single step (T = 1) for few small heads, in ONE launch and without any
// exchange between workgroups: one workgroup per (head, in-block position j).
//
// With T = 1 the Z problem of position j (z_ref, ma/ma_torch.py:55-62) reads, of every block m, only
// row j of what the R problem of that block produces (al_y_cl_ref, :38-52): aL(j, m), Y(j, m), cL(j, m).
// That row depends on the query row (m, j) and on the keys and values of block m alone, so the
// workgroup computes those M rows itself - one row per block instead of the block's B rows - and
// then its Z problem: nothing is handed from one workgroup to another, there is no second launch and
// no flag.  The price is that every workgroup reads the head's whole K and V (B times the bytes in
// total, from L2), which is why this is for few heads of at most 16 blocks of at most 16 rows (the
// reference's CPU-sized configuration: one fp32 head of 256 tokens, block 16).
//
// 256 threads, thread t = 16 a + b.  Products of one row with a 16-row block are plain fp32 FMAs
// (a 16 x 16 x 4 matrix instruction would compute the block's other 15 rows as well):
//   load     K and V of the head -> LDS tiles (row m*16 + i, pitch LD), the Q rows {l*B + j} -> Qt
//   logits   thread (m, i): s = Qt[m] . K[m, i]; softmax over i within the 16 lanes (DPP), r -> Rt, cL -> cl
//   rows     thread (m, c): aL[m][4c..] = sm_scale sum_i r[m][i] K[m, i][4c..], Y likewise with V -> At, Yt
//   z logits thread (l, k): g = At[k] . Qt[l] - cL[k]; softmax over k within the 16 lanes -> Lt
//   output   thread (l, c): out[l*B + j][4c..] = sum_k Lt[l][k] Yt[k][4c..]
// The arithmetic follows the fp32 stage kernels (log2-domain softmax, clamped row maximum, +eps
// denominators, ma/ma_torch.py:10-23), only the order of the sums differs from theirs.
#pragma once

#include "ma_mfma32.h"

namespace ma {
namespace mfma32 {

template <int DTF>
struct HeadT1 {
    static constexpr int LD = Geom32<DTF>::LD;
    static constexpr int CH = 4 * DTF;             // 16-byte chunks per row
    static constexpr int TILE = 256 * LD;          // floats: 16 blocks x 16 rows
    static constexpr int ROW16 = 16 * LD;          // a 16-row tile (Qt, At, Yt)
    static constexpr size_t lds_bytes = (2 * TILE + 3 * ROW16 + 2 * 256 + 16) * sizeof(float);
};

template <int DTF>
__global__ __launch_bounds__(256) void head_t1_f32(Problem P) {
    using HG = HeadT1<DTF>;
    constexpr int LD = HG::LD, CH = HG::CH;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    float* Kt = reinterpret_cast<float*>(smem);
    float* Vt = Kt + HG::TILE;
    float* Qt = Vt + HG::TILE;       // row l: query (l, j)
    float* At = Qt + HG::ROW16;      // row m: aL(j, m)
    float* Yt = At + HG::ROW16;      // row m: Y(j, m)
    float* Rt = Yt + HG::ROW16;      // [m*16 + i]: probabilities of row (m, j)
    float* Lt = Rt + 256;            // [l*16 + k]
    float* cl = Lt + 256;            // [m]: cL(j, m)
    const int t = threadIdx.x, a = t >> 4, b = t & 15;
    const int B = P.B, M = P.M, D = P.D, N = P.N;
    const unsigned pid = blockIdx.x;
    const int j = pid % static_cast<unsigned>(B);
    const int head = pid / static_cast<unsigned>(B);   // E * H * Np fits int32 (validated by the host)
    const int e = static_cast<unsigned>(head) / static_cast<unsigned>(P.H), h = static_cast<unsigned>(head) % static_cast<unsigned>(P.H);
    const Slices S = make_slices<float>(P, e, h, head);

    // ---- load: tile row m*16 + i <- token m*B + i - pad_off (rows beyond the block, the head or D: zeros)
    {
        u32x4 kv[CH], vv[CH];
#pragma unroll
        for (int n = 0; n < CH; ++n) {
            const int c = t + 256 * n, row = c / CH, ch = c % CH;
            const int m = row >> 4, i = row & 15;
            const bool in = i < B && m < M && ch * 4 < D;
            kv[n] = bload16<false>(S.k, in ? tok_off(m * B + i - P.pad_off, N, S.kst) + ch * 16 : kOob);
        }
        const int ql = t / CH, qch = t % CH;   // Q rows: 16 x CH chunks, one per thread (CH <= 16)
        const u32x4 qv = bload16<false>(S.q, (t < 16 * CH && ql < M && qch * 4 < D) ? tok_off(ql * B + j - P.pad_off, N, S.qst) + qch * 16 : kOob);
#pragma unroll
        for (int n = 0; n < CH; ++n) {
            const int c = t + 256 * n, row = c / CH, ch = c % CH;
            const int m = row >> 4, i = row & 15;
            const bool in = i < B && m < M && ch * 4 < D;
            vv[n] = bload16<false>(S.v, in ? tok_off(m * B + i - P.pad_off, N, S.vst) + ch * 16 : kOob);
        }
#pragma unroll
        for (int n = 0; n < CH; ++n) {
            const int c = t + 256 * n, row = c / CH, ch = c % CH;
            *reinterpret_cast<u32x4*>(Kt + row * LD + ch * 4) = kv[n];
        }
        if (t < 16 * CH) *reinterpret_cast<u32x4*>(Qt + ql * LD + qch * 4) = qv;
#pragma unroll
        for (int n = 0; n < CH; ++n) {
            const int c = t + 256 * n, row = c / CH, ch = c % CH;
            *reinterpret_cast<u32x4*>(Vt + row * LD + ch * 4) = vv[n];
        }
    }
    // key (m = a, i = b) is real and not masked out
    const int tk = a * B + b - P.pad_off;
    const bool key_ok = b < B && a < M && token_kept(P, tk, mask_load(S, P, tk, b < B && a < M));
    __syncthreads();

    // ---- logits of row (m, j) against the keys of block m, softmax over i (al_y_cl_ref, ma/ma_torch.py:38-48)
    {
        const int m = a, i = b;
        const float* qrow = Qt + m * LD;
        const float* krow = Kt + (m * 16 + i) * LD;
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const f32x4 qx = *reinterpret_cast<const f32x4*>(qrow + 4 * c);
            const f32x4 kx = *reinterpret_cast<const f32x4*>(krow + 4 * c);
#pragma unroll
            for (int u = 0; u < 4; ++u) s = fmaf(qx[u], kx[u], s);
        }
        const float cj = (P.sm_scale * kLog2e) * rcp(1.0f + P.eps);   // cR = 1 before the first step (:88-89)
        const float x = fmaf(s, cj, key_ok ? 0.f : kNegBig);
        const float mx = fmaxf(row16_max(x), P.eps * kLog2e);          // clamped row maximum (:43)
        const float d = x - mx;
        const float p = __builtin_amdgcn_exp2f(d);
        const float sum = row16_sum(p), ent = row16_sum(p * d);
        const float den = sum + P.eps, inv = rcp(den);
        Rt[m * 16 + i] = p * inv;
        if (i == 0) cl[m] = kLn2 * ent * inv - __logf(den) * (sum * inv);   // sum_i r log r
    }
    __syncthreads();

    // ---- row j of aL and Y of every block: thread (m, c) forms four columns
    {
        const int m = a, c = b;
        f32x4 ax = {0.f, 0.f, 0.f, 0.f}, yx = {0.f, 0.f, 0.f, 0.f};
        if (c < CH) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 r4 = *reinterpret_cast<const f32x4*>(Rt + m * 16 + 4 * g);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int row = m * 16 + 4 * g + u;
                    const f32x4 kx = *reinterpret_cast<const f32x4*>(Kt + row * LD + 4 * c);
                    const f32x4 vx = *reinterpret_cast<const f32x4*>(Vt + row * LD + 4 * c);
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        ax[w] = fmaf(r4[u], kx[w], ax[w]);
                        yx[w] = fmaf(r4[u], vx[w], yx[w]);
                    }
                }
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) ax[w] *= P.sm_scale;
            *reinterpret_cast<f32x4*>(At + m * LD + 4 * c) = ax;
            *reinterpret_cast<f32x4*>(Yt + m * LD + 4 * c) = yx;
        }
    }
    __syncthreads();

    // ---- Z problem of position j (z_ref, ma/ma_torch.py:55-62): thread (l, k), softmax over k
    {
        const int l = a, k = b;
        const float* arow = At + k * LD;
        const float* qrow = Qt + l * LD;
        float g = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const f32x4 ay = *reinterpret_cast<const f32x4*>(arow + 4 * c);
            const f32x4 qx = *reinterpret_cast<const f32x4*>(qrow + 4 * c);
#pragma unroll
            for (int u = 0; u < 4; ++u) g = fmaf(ay[u], qx[u], g);
        }
        const float x = k < M ? fmaf(g, kLog2e, -kLog2e * cl[k]) : kNegBig;
        const float p = __builtin_amdgcn_exp2f(x - row16_max(x));
        Lt[l * 16 + k] = p * rcp(row16_sum(p));
    }
    // Lt row l is written and read by the 16 lanes of one DPP row of one wave: the LDS executes a wave's
    // accesses in order, the compiler only has to keep them in place
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- output row (l, j): thread (l, c) forms four columns; padded query rows are dropped (:106-108)
    {
        const int l = a, c = b;
        if (c < CH) {
            f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 l4 = *reinterpret_cast<const f32x4*>(Lt + l * 16 + 4 * g);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const f32x4 yx = *reinterpret_cast<const f32x4*>(Yt + (4 * g + u) * LD + 4 * c);
#pragma unroll
                    for (int w = 0; w < 4; ++w) o[w] = fmaf(l4[u], yx[w], o[w]);
                }
            }
            const int tq = l * B + j - P.pad_off;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o), S.out,
                                                   (l < M && 4 * c < D) ? tok_off(tq, N, S.ost) + c * 16 : kOob, 0, 0);
        }
    }
}

}  // namespace mfma32
}  // namespace ma
