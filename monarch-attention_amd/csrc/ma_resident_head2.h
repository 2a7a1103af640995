// Head-resident forward in TWO tiles, for heads that are too long for the four tiles of ma_resident_head.h
// (257 .. ~540 tokens at D = 64): one workgroup runs a whole head with the state tile S and ONE input tile X in
// LDS, and X holds whatever the running phase reads transposed (monarch_attention_torch, ma/ma_torch.py:65-108):
//
//   phase            X holds                                  read besides
//   R (al_y_cl_ref)  K; in the last R phase block m's rows     S rows aR(m, .) - S starts out as Q, so the first step
//                    become V(m), then Y(., m), in place      reads its query rows there too
//   L (ar_cr_ref)    Q                                        S rows aL(j, .)
//   Z (z_ref)        Y (left there by the last R phase)       S rows aL(j, .); the query rows straight from memory
//                                                             (they are a row operand only)
//
// The tile that the NEXT phase needs is loaded into registers while the current phase computes (the head's Q
// chunks are simply kept from the start for the first L phase) and written to X between two barriers at the
// phase boundary.  Every block problem is what it is in ma_resident_head.h - LDS reads, matrix products, the
// softmax - except the last R problem of a block, which loads the block's V rows itself and swaps them in for
// the K rows when it has formed aL, and the Z problems, which load their query rows a round ahead.
// A head costs one read of Q, V and (T - 1) reads each of Q and K beyond the first (from L2), and one write of
// the output; no state leaves the compute unit.
// Two tiles of a SHORT head are small enough for several workgroups per compute unit: with more heads than compute
// units the launcher runs this kernel in workgroups of 8 or 4 waves, two or four to a compute unit, each walking
// its own heads - they are out of step and fill each other's barrier and load waits (ma_resident_launch.h).
#pragma once

#include "ma_resident_head.h"

namespace ma {
namespace mfma {

template <class T, int DT, int NTB, int NTM, int W, int NI>
struct HeadRes2 {
    using HR = HeadRes<T, DT, NTB, NTM, W, NI>;
    using Layout = typename HR::Layout;
    using Ctx = typename HR::Ctx;
    using Head = typename HR::Head;
    using V8 = typename HR::V8;

    // S, X and the small arrays of the four-tile layout; Q, K and V all name X
    static __host__ __device__ Layout layout(int Np, int B, int M) {
        Layout L;
        unsigned o = 0;
        const unsigned tile = static_cast<unsigned>(Np + HR::pad_rows(B)) * HR::RB + static_cast<unsigned>((Np + HR::pad_rows(B)) / B + 1) * HR::kSkew;
        L.S = o; o += tile;
        L.Q = L.K = L.V = o; o += tile;
        L.ZR = o; o += HR::RB;
        L.TR = o; o += HR::RB;
        L.cb = o; o += static_cast<unsigned>(B) * HR::ROWSM * 4;
        L.cR = o; o += static_cast<unsigned>((Np + 3) / 4 * 4) * 4;
        L.tokb = o; o += static_cast<unsigned>(M) * HR::ROWSB * 4;
        L.stats = o; o += HR::PPM * 2 * HR::ROWSM * 4;
        L.trash = o; o += 16;
        L.total = o;
        return L;
    }
    static __host__ bool fits(int Np, int B, int M, size_t lds_limit) {
        return layout(Np, B, M).total <= lds_limit && (Np + HR::pad_rows(B)) * HR::CH <= NI * HR::NT && M * HR::ROWSB <= HR::NT &&
               (Np + HR::ROWSB) * B < 65536;
    }

    // one input tile of a head into the thread's registers
    static __device__ __forceinline__ void issue_tile(const Problem& P, const Ctx& c, rsrc_t src, unsigned st, u32x4 (&x)[NI], bool live = true) {
        unsigned off[NI];
        HR::chunk_offsets(P, c, st, off, live);
#pragma unroll
        for (int i = 0; i < NI; ++i) x[i] = bload16<false>(src, off[i]);
    }
};

template <class T, int DT, int NTB, int NTM, int W, int NI>
__device__ __forceinline__ void resident_head2_body(const Problem& P) {
    using H2 = HeadRes2<T, DT, NTB, NTM, W, NI>;
    using HR = typename H2::HR;
    using V8 = typename H2::V8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int Np = P.M * P.B;
    typename HR::Ctx c;
    c.smem = smem;
    c.L = H2::layout(Np, P.B, P.M);
    c.tid = threadIdx.x;
    c.wave = wave_id();
    c.lane = threadIdx.x & 63;
    c.r = c.lane & 15;
    c.q = c.lane >> 4;
    c.qst = static_cast<unsigned>(P.qs[2]) * sizeof(T);
    c.kst = static_cast<unsigned>(P.ks[2]) * sizeof(T);
    c.vst = static_cast<unsigned>(P.vs[2]) * sizeof(T);
    c.ost = static_cast<unsigned>(P.os[2]) * sizeof(T);
    c.mst = P.mask ? static_cast<unsigned>(P.ms[1]) << P.mask_shift : 0u;
    c.scale2 = P.sm_scale * kLog2e;
    c.BP = HR::block_pitch(P.B);
    const bool scale_is_f16 = static_cast<float>(static_cast<_Float16>(P.sm_scale)) == P.sm_scale;
    // once per launch: zeros in the tiles (the gaps between the blocks' rows and the rows behind the last block are
    // never written again), in the row of zeros; the softmax bias of key blocks that do not exist
    // (with blocks of exactly 16, 32 or 64 rows no strip reaches across a gap or into the columns behind a row's last, and
    // with a head dim that fills its tile columns every column a product reads is written first: only the row of zeros then)
    const bool fill_tiles = HR::ROWSB != P.B || (DT & 1) != 0;   // uniform
    for (unsigned i = (fill_tiles ? 0u : c.L.ZR) + c.tid * 16u; i < c.L.TR; i += HR::NT * 16u) *reinterpret_cast<u32x4*>(smem + i) = u32x4{0u, 0u, 0u, 0u};
    for (int i = c.tid; i < P.B * HR::ROWSM; i += HR::NT) c.fat(c.L.cb)[i] = kNegBig;

    const int heads = P.E * P.H, stride = static_cast<int>(gridDim.x);
    const int nr = (P.M + HR::PPB - 1) / HR::PPB, nl = (P.B + HR::PPM - 1) / HR::PPM;
    for (int head = static_cast<int>(blockIdx.x); head < heads; head += stride) {
        const typename HR::Head hd = HR::head_of(P, c, head);
        typename HR::Pre pre = {};   // (only its Q chunks and the mask element are used here)
        {
            u32x4 kx[NI];
            HR::issue_q(P, c, hd, pre);
            H2::issue_tile(P, c, hd.k, c.kst, kx);
            __syncthreads();   // the zero fill, or the previous head's last readers
            HR::commit_tile(P, c, c.L.S, pre.q);
            HR::commit_tile(P, c, c.L.K, kx);
            HR::commit_tokb(P, c, pre);
        }
        __syncthreads();
        // pre.q is the one set of registers a tile travels in: Q (kept from the start for the first L phase, fetched
        // again in front of the R phase of a later step), then K while the L phase runs
        for (int t = 0; t < P.T; ++t) {
            const bool last = t == P.T - 1;
            if (t > 0 && !last) H2::issue_tile(P, c, hd.q, c.qst, pre.q);
            for (int rnd = 0; rnd < nr; ++rnd) HR::template round_r<true>(P, c, rnd, t == 0, last, scale_is_f16, &hd);
            if (last) break;
            __syncthreads();   // K has had its last reader of this step
            HR::commit_tile(P, c, c.L.Q, pre.q);
            __syncthreads();
            H2::issue_tile(P, c, hd.k, c.kst, pre.q);
            for (int rnd = 0; rnd < nl; ++rnd) HR::round_l(P, c, rnd);
            __syncthreads();
            HR::commit_tile(P, c, c.L.K, pre.q);
            __syncthreads();
        }
        // The next head of this workgroup: one load per 128-byte line of its Q and K rows, so that they wait in the
        // L2 when the head starts (whole tiles held in registers through the Z problems - and through the loop over
        // heads - spill at 16 waves per workgroup).
        unsigned warm = 0;
        if (head + stride < heads) {   // uniform
            const typename HR::Head hn = HR::head_of(P, c, head + stride);
            const int row = c.tid >> 1;   // even threads: Q's row, odd threads: K's
            for (int r0 = 0; r0 < Np; r0 += HR::NT / 2) {
                const unsigned tk = static_cast<unsigned>(row + r0 - P.pad_off);
                const bool ok = row + r0 < Np && tk < static_cast<unsigned>(P.N);
                warm += __builtin_amdgcn_raw_buffer_load_b32((c.tid & 1) ? hn.k : hn.q, ok ? tk * ((c.tid & 1) ? c.kst : c.qst) : kOob, 0, 0);
            }
        }
        // the query rows of a Z round come from memory a round ahead, the first ones before the barrier
        V8 zq[HR::KS];
        HR::load_zq(P, c, hd, 0, zq);
        __syncthreads();   // the Z problems read the state and Y transposed
        for (int rnd = 0; rnd < nl; ++rnd) {
            V8 cur[HR::KS];
#pragma unroll
            for (int ks = 0; ks < HR::KS; ++ks) cur[ks] = zq[ks];
            if (rnd + 1 < nl) HR::load_zq(P, c, hd, rnd + 1, zq);
            HR::template round_z<true>(P, c, hd, rnd, cur);
        }
        asm volatile("" ::"v"(warm));   // (keeps the loads)
    }
}

// WGS: the number of workgroups a compute unit is meant to hold (W * WGS = 16 waves; the register budget follows from it)
template <class T, int DT, int NTB, int NTM, int W, int NI, int WGS = 1>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(W * WGS / 4))) void resident_head2_mfma(Problem P) {
    resident_head2_body<T, DT, NTB, NTM, W, NI>(P);
}

}  // namespace mfma
}  // namespace ma
