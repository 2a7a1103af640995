// fp32 forward pass of small heads in ONE launch: one workgroup per head, all T steps of
// monarch_attention_torch (ma/ma_torch.py:65-108) with the state of the head in LDS and nothing in
// the workspace.  For heads of at most 16 blocks of at most 16 rows (256 tokens: the reference's own
// CPU-sized case, fp32 N = 256, block 16) with head dims up to 64.
//
// Every block problem - R problem of block m, L / Z problem of in-block position j - is a single
// 16 x 16 problem and belongs to one wave (the arithmetic is that of the fp32 stage kernels, see
// ma_mfma32.h: v_mfma_f32_16x16x4_f32, softmax in registers), so a phase needs no barrier inside;
// the 16 waves meet between phases.
//
// LDS: two tiles of 16 blocks x 16 rows, row pitch LD floats, block pitch 16 LD + 4 (the extra 16
// bytes per block spread the rows {block k, row j} of an L / Z problem over the banks; rows of one
// block differ by LD = 4 mod 32 words already).
//   St  state: aR(m, j) before an R step and aL(j, m) after it both live at block m, row j, and an
//       R problem works in place: it takes its aR rows into registers, stages the K rows of its
//       block where they were, and writes aL over them when the products are done.  L problems
//       likewise read the rows {k, j} and write aR(k, j) back to them.
//   Yt  Y(j, m) at block m, row j, written by the last R step over the V rows it staged there;
//       during L steps, when there is no Y yet, it holds the Q rows {l, j} of the L problems.
// Blocks beyond M and rows beyond B stay zero from the fill at the start (an R problem stages zero
// rows there and writes nothing back), so the 16-wide products never meet anything but zeros there.
// cL and cR sit in two 16 x 16 arrays indexed [block][row].
#pragma once

#include "ma_mfma32.h"

namespace ma {
namespace mfma32 {

template <int DTF>
struct Head32 {
    static constexpr int LD = Geom32<DTF>::LD;
    static constexpr int BP = 16 * LD + 4;     // floats per block
    static constexpr int TILE = 16 * BP;       // floats per tile
    static constexpr int W = 16;               // waves per workgroup: one per block problem of a phase
    static constexpr int CH = 4 * DTF;         // 16-byte chunks per row
    static constexpr size_t lds_bytes = (2 * TILE + 2 * 256 + W * 16) * sizeof(float);
    static_assert(TILE % 4 == 0, "tiles are cleared in 16-byte pieces");
};

// out^T = sum_w tile[row w][16 dt + r] P[w][x] for the 16 rows w = 4 q + v at `pitch` floats from each other
template <int DTF>
__device__ __forceinline__ void gemm2_rows(f32x4 (&O)[DTF], const float* row0, int pitch, const f32x4& C, int r, int q) {
#pragma unroll
    for (int dt = 0; dt < DTF; ++dt) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int v = 0; v < 4; ++v) acc = mma4(row0[(4 * q + v) * pitch + 16 * dt + r], C[v], acc);
        O[dt] = acc;
    }
}

template <int DTF>
__device__ __forceinline__ void lds_store_row(float* row, const f32x4 (&O)[DTF], int q) {
#pragma unroll
    for (int dt = 0; dt < DTF; ++dt) *reinterpret_cast<f32x4*>(row + 16 * dt + 4 * q) = O[dt];
}

// keeps the compiler from moving LDS accesses of a wave across this point; the LDS itself executes a
// wave's instructions in order
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int DTF>
__global__ __launch_bounds__(1024) void head_fwd_f32(Problem P) {
    using HG = Head32<DTF>;
    constexpr int LD = HG::LD, BP = HG::BP, TILE = HG::TILE, CH = HG::CH;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    float* St = reinterpret_cast<float*>(smem);
    float* Yt = St + TILE;
    float* cl = Yt + TILE;      // [m * 16 + j]
    float* cr = cl + 256;       // [m * 16 + j]
    float* kb = cr + 256;       // [wave][16]: key bias of the wave's R problem
    const int wave = wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4, tix = threadIdx.x;
    const int B = P.B, M = P.M, D = P.D, N = P.N;
    const int heads = P.E * P.H;   // E * H * Np fits int32 (validated by the host)
    const int nph = 2 * P.T;

    for (int i = tix; i < 2 * TILE / 4; i += 1024) reinterpret_cast<f32x4*>(St)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();

    for (int head = blockIdx.x; head < heads; head += gridDim.x) {
        const int e = static_cast<unsigned>(head) / static_cast<unsigned>(P.H), h = static_cast<unsigned>(head) % static_cast<unsigned>(P.H);
        // the Q rows {l = r, j = wave} of this wave's Z problem: needed last, asked for first
        f32x4 xz[DTF];
        {
            const Slices S = make_slices<float>(P, e, h, head);
            const int t = r * B + wave - P.pad_off;
            load_row<DTF>(xz, S.q, (wave < B && r < M) ? tok_off(t, N, S.qst) : kOob, D, q);
        }
#pragma nounroll
        for (int ph = 0; ph < nph; ++ph) {
            // The problem description is read again from the kernel arguments in every phase, through an
            // offset the compiler cannot see through, and the tensor slices are made inside each branch:
            // a phase then only holds the buffer resources it uses in scalar registers.
            int zero = 0;
            asm volatile("" : "+s"(zero));
            const Problem& Pp = *reinterpret_cast<const Problem*>(reinterpret_cast<const char*>(&P) + zero);
            if (ph == nph - 1) {
                // ---- Z problem of position j: z_ref (ma/ma_torch.py:55-62) and the final slice (:106-108)
                const int j = wave;
                if (j < B) {
                    const Slices S = make_slices<float>(Pp, e, h, head);
                    const f32x4 acc = gemm1_tile<DTF>(St + r * BP + j * LD + 4 * q, xz);
                    f32x4 C;
                    float mx = kNegBig;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int k = 4 * q + v;
                        const float b = k < M ? -kLog2e * cl[k * 16 + j] : kNegBig;
                        C[v] = fmaf(acc[v], kLog2e, b);
                        mx = fmaxf(mx, C[v]);
                    }
                    mx = quad_rows_max(mx);
                    float sum = 0.f;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        C[v] = __builtin_amdgcn_exp2f(C[v] - mx);
                        sum += C[v];
                    }
                    const float inv = rcp(quad_rows_sum(sum));
#pragma unroll
                    for (int v = 0; v < 4; ++v) C[v] *= inv;
                    f32x4 O[DTF];
                    gemm2_rows<DTF>(O, Yt + j * LD, BP, C, r, q);
                    const int t = r * B + j - P.pad_off;
                    store_row<DTF>(S.out, r < M ? tok_off(t, N, S.ost) : kOob, D, O, q);   // padded query rows are dropped (:108)
                }
            } else if (ph & 1) {
                // ---- L problem of position j: ar_cr_ref (ma/ma_torch.py:26-35)
                const int j = wave;
                if (j < B) {
                    const Slices S = make_slices<float>(Pp, e, h, head);
                    u32x4 qv[DTF];
#pragma unroll
                    for (int i = 0; i < DTF; ++i) {
                        const int c = lane + 64 * i, l = c / CH, ch = c % CH;
                        qv[i] = bload16<false>(S.q, (l < M && ch * 4 < D) ? tok_off(l * B + j - P.pad_off, N, S.qst) + ch * 16 : kOob);
                    }
                    unsigned qm[4];
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int l = 4 * q + v;
                        qm[v] = mask_load(S, P, l * B + j - P.pad_off, l < M);
                    }
#pragma unroll
                    for (int i = 0; i < DTF; ++i) {
                        const int c = lane + 64 * i, l = c / CH, ch = c % CH;
                        *reinterpret_cast<u32x4*>(Yt + l * BP + j * LD + ch * 4) = qv[i];
                    }
                    wave_lds_order();
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < DTF; ++t) {
                        const f32x4 a = *reinterpret_cast<const f32x4*>(Yt + r * BP + j * LD + 16 * t + 4 * q);   // query row l = r
                        const f32x4 b = *reinterpret_cast<const f32x4*>(St + r * BP + j * LD + 16 * t + 4 * q);   // aL row k = r
#pragma unroll
                        for (int u = 0; u < 4; ++u) acc = mma4(a[u], b[u], acc);
                    }
                    // lane holds column k = r, rows l = 4 q + v; the softmax runs over k (ma_torch.py:29)
                    const float bias = r < M ? -kLog2e * cl[r * 16 + j] : kNegBig;
                    f32x4 o;
                    float part = 0.f;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float c = fmaf(acc[v], kLog2e, bias);
                        const float p = __builtin_amdgcn_exp2f(c - row16_max(c));
                        const float sv = row16_sum(p);
                        // padded / masked query tokens are zeroed after the softmax (ma_torch.py:30)
                        const int l = 4 * q + v;
                        const float inv = (l < M && token_kept(P, l * B + j - P.pad_off, qm[v])) ? rcp(sv) : 0.f;
                        o[v] = p * inv;
                        part += o[v];
                    }
                    const float crsum = quad_rows_sum(part);   // cR(k, j) = sum_l L[l, k]
                    f32x4 O[DTF];
                    gemm2_rows<DTF>(O, Yt + j * LD, BP, o, r, q);   // aR(k, :) = sum_l L[l, k] Qt[l, :]
                    if (r < M) {
                        lds_store_row<DTF>(St + r * BP + j * LD, O, q);
                        if (q == 0) cr[r * 16 + j] = crsum;
                    }
                }
            } else {
                // ---- R problem of block m: al_cl_ref / al_y_cl_ref (ma/ma_torch.py:10-23, :38-52)
                const int m = wave;
                const bool first = ph == 0, with_v = ph == nph - 2;
                if (m < M) {
                    const Slices S = make_slices<float>(Pp, e, h, head);
                    float* Sb = St + m * BP;
                    float* Yb = Yt + m * BP;
                    const int t0 = m * B - P.pad_off;
                    u32x4 kv[DTF];
#pragma unroll
                    for (int i = 0; i < DTF; ++i) {
                        const int c = lane + 64 * i, row = c / CH, ch = c % CH;
                        kv[i] = bload16<false>(S.k, (row < B && ch * 4 < D) ? tok_off(t0 + row, N, S.kst) + ch * 16 : kOob);
                    }
                    if (with_v) {   // straight into the (free) rows of the Y tile: no registers held for it
#pragma unroll
                        for (int i = 0; i < DTF; ++i) {
                            const int c = lane + 64 * i, row = c / CH, ch = c % CH;
                            const u32x4 vv = bload16<false>(S.v, (row < B && ch * 4 < D) ? tok_off(t0 + row, N, S.vst) + ch * 16 : kOob);
                            *reinterpret_cast<u32x4*>(Yb + row * LD + ch * 4) = vv;
                        }
                    }
                    const unsigned km = mask_load(S, P, t0 + r, r < B);
                    f32x4 xb[DTF];
                    float crv = 1.0f;
                    if (first) {
                        load_row<DTF>(xb, S.q, r < B ? tok_off(t0 + r, N, S.qst) : kOob, D, q);
                    } else {
#pragma unroll
                        for (int t = 0; t < DTF; ++t) xb[t] = *reinterpret_cast<const f32x4*>(Sb + r * LD + 16 * t + 4 * q);
                        if (r < B) crv = cr[m * 16 + r];
                    }
                    wave_lds_order();
#pragma unroll
                    for (int i = 0; i < DTF; ++i) {
                        const int c = lane + 64 * i, row = c / CH, ch = c % CH;
                        *reinterpret_cast<u32x4*>(Sb + row * LD + ch * 4) = kv[i];
                    }
                    if (q == 0) kb[wave * 16 + r] = (r < B && token_kept(P, t0 + r, km)) ? 0.f : kNegBig;
                    wave_lds_order();
                    const float cj = (P.sm_scale * kLog2e) * rcp(crv + P.eps);   // logits in log2 units
                    const f32x4 acc = gemm1_tile<DTF>(Sb + r * LD + 4 * q, xb);
                    const f32x4 kbv = *reinterpret_cast<const f32x4*>(kb + wave * 16 + 4 * q);
                    f32x4 C;
#pragma unroll
                    for (int v = 0; v < 4; ++v) C[v] = fmaf(acc[v], cj, kbv[v]);
                    // clamped row maximum (ma_torch.py:15): max(rowmax, eps), here in log2 units
                    float mx = fmaxf(fmaxf(C[0], C[1]), fmaxf(C[2], C[3]));
                    mx = fmaxf(quad_rows_max(mx), P.eps * kLog2e);
                    float sum = 0.f, ent = 0.f;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float d = C[v] - mx;
                        const float p = __builtin_amdgcn_exp2f(d);
                        sum += p;
                        ent = fmaf(p, d, ent);   // sum p * log2(p)
                        C[v] = p;
                    }
                    sum = quad_rows_sum(sum);
                    ent = quad_rows_sum(ent);
                    const float den = sum + P.eps, inv = rcp(den);
#pragma unroll
                    for (int v = 0; v < 4; ++v) C[v] *= inv;
                    // cL = sum_i r log r with r = p / den (ma_torch.py:20)
                    if (q == 0 && r < B) cl[m * 16 + r] = kLn2 * ent * inv - __logf(den) * (sum * inv);
                    f32x4 O[DTF], OY[DTF];
                    gemm2_rows<DTF>(O, Sb, LD, C, r, q);
                    if (with_v) gemm2_rows<DTF>(OY, Yb, LD, C, r, q);
#pragma unroll
                    for (int dt = 0; dt < DTF; ++dt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) O[dt][v] *= P.sm_scale;
                    wave_lds_order();
                    if (r < B) {
                        lds_store_row<DTF>(Sb + r * LD, O, q);
                        if (with_v) lds_store_row<DTF>(Yb + r * LD, OY, q);
                    }
                }
            }
            __syncthreads();
        }
    }
}

}  // namespace mfma32
}  // namespace ma
