// MFMA building blocks and the three stage bodies (R, L, Z) for fp16 / bf16 on
// gfx950.  One wavefront (64 lanes) works on a 16-row strip of a block problem
// with v_mfma_f32_16x16x32_{f16,bf16}; the four waves of a workgroup share the
// problem's operand tiles in LDS.
//
// Lane naming for the 16x16x32 instruction: r = lane % 16, q = lane / 16.
//   A operand (16 x 32): lane holds row r,    k = 8q .. 8q+7
//   B operand (32 x 16): lane holds column r, k = 8q .. 8q+7
//   C / D     (16 x 16): lane holds column r, rows 4q .. 4q+3
//
// Every stage is "GEMM1 -> softmax in registers -> GEMM2":
//   GEMM1  C[w, x] = sum_d W[w, d] X[x, d]     (both operands row-major in d,
//          so they load as 16-byte vectors: W from its LDS tile, X from HBM)
//   softmax over w for every x.  x is the lane's column, so the reduction is
//          in-lane plus two cross-lane steps.  The L step contracts its second
//          product over x instead of w: it forms the logits a second time with
//          the operand roles swapped (see LProb).
//   GEMM2  out^T[d, x] = sum_w Wv^T[d, w] P[w, x].  P is taken straight from
//          the C registers as the B operand: the k slots of a lane are mapped
//          to w = 32g + 16(s/4) + 4q + s%4, exactly the rows the lane already
//          holds of C tiles 2g and 2g+1.  The transposed A operand comes from
//          the row-major LDS tile with ds_read_b64_tr_b16 (lane 4e+c of a
//          16-lane group supplies row e, columns 4c..4c+3 of a 4x16 block;
//          lane i receives column i of that block).
//
// Numerics follow the reference's rounding points (ma/ma_torch.py:11,21,27,33,
// 39,49,50,56,60): GEMM1 is rounded to the operand dtype before the fp32
// softmax math, probabilities are rounded to the operand dtype for GEMM2,
// sm_scale multiplies the rounded aL.  Masked keys, padded tokens and tile
// tails enter the softmax through a -1e30 bias (exp2 underflows to exactly 0).
#pragma once

#include "ma_common.h"

namespace ma {
namespace mfma {

// Index of the wave inside its workgroup, as a value the compiler knows to be
// uniform: everything derived from it (problem index, tensor slices, buffer
// resources) then lives in scalar registers, and buffer instructions take their
// resource operand directly instead of through a per-lane "waterfall" loop.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x)) >> 6; }


constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

template <class T>
struct Ops;

template <>
struct Ops<f16> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    typedef _Float16 v4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x4 mma(v8 a, v8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Ops<bf16> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    typedef __bf16 v4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x4 mma(v8 a, v8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};

// ---- cross-lane reductions -------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
// all-reduce over the 16 lanes of a DPP row (quad xor 1, xor 2, half mirror, mirror)
__device__ __forceinline__ float row16_max(float x) {
    x = fmaxf(x, dpp<0xB1>(x));
    x = fmaxf(x, dpp<0x4E>(x));
    x = fmaxf(x, dpp<0x141>(x));
    x = fmaxf(x, dpp<0x140>(x));
    return x;
}
__device__ __forceinline__ float row16_sum(float x) {
    x += dpp<0xB1>(x);
    x += dpp<0x4E>(x);
    x += dpp<0x141>(x);
    x += dpp<0x140>(x);
    return x;
}
// all-reduce over the four lanes {r, r+16, r+32, r+48}: two lane-swap steps on the
// VALU (v_permlane16_swap exchanges the odd 16-lane rows of its first operand with
// the even rows of its second, v_permlane32_swap the upper half of the first with
// the lower half of the second; with both operands holding x the two results are
// x of the lane's own row pair / half and x of the other one) - no trip through
// the LDS crossbar as a shuffle would take.  The s_nop covers the wait states the
// swap needs after a VALU write of its operands.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// (the maximum / sum sits inside the asm statement: on a value that comes out of one the compiler would first
// quieten a possible signalling NaN with an extra instruction per operand; the s_nop behind the swap covers the
// wait states a VALU read of its results needs.  The statements are volatile on purpose: they keep their place
// in the instruction stream, and with it the compiler from moving the loads and matrix products of a whole block
// problem in front of its softmax, which costs twice the registers.)
__device__ __forceinline__ float quad_rows_max(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1\n\tv_max_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1\n\tv_max_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    return a;
}
__device__ __forceinline__ float quad_rows_sum(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1\n\tv_add_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1\n\tv_add_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    return a;
}
// 1 / x to 1 ulp (v_rcp_f32) instead of the ten-instruction IEEE division
__device__ __forceinline__ float rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// log2(x) of a normal positive x to 1 ulp (v_log_f32), without the denormal handling of the library call
__device__ __forceinline__ float log2_normal(float x) { return __builtin_amdgcn_logf(x); }

// ---- global memory through buffer resources ---------------------------------
// Every tensor slice a block problem touches is addressed as (uniform base in
// SGPRs) + (32-bit byte offset per lane).  Rows that do not exist (padding,
// masked-out tails, tile tails) get the offset kOob, which the hardware bounds
// check turns into a load of zeros / a dropped store - no branches.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr unsigned kOob = 0xFFFF0000u;  // beyond any slice (extents are validated to stay below it)

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
// The template argument is a cache policy: 0 / false = ordinary, 1 / true = streaming ("nt"), 2 = agent scope
// ("sc1").  State that another workgroup wrote during this launch is read with one of the latter two: both are
// served by the L2 and never by a line this CU's L1 kept from an earlier step.  Which of them is the caller's choice
// per launch (Slices::agent_state): agent-scope loads keep their lines in the L2 like any other, which pays while
// the state arrays fit the caches (2 - 6 % on heads x tokens up to ~256 K) and costs 4 - 6 % where they do not.
constexpr int kPolStream = 1, kPolAgent = 2;
template <int POL>
__device__ __forceinline__ u32x4 bload16(rsrc_t r, unsigned off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, POL == 0 ? 0 : POL == 1 ? 2 : 16);
}
template <int POL>
__device__ __forceinline__ float bloadf(rsrc_t r, unsigned off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, POL == 0 ? 0 : POL == 1 ? 2 : 16));
}

// ---- operand tiles ----------------------------------------------------------
// LDS tile geometry for a head dim that needs DT 16-wide output tiles:
// KS 32-wide k steps, row pitch LD elements (the +8 staggers rows over banks).
template <int DT>
struct Geom {
    static constexpr int KS = (DT + 1) / 2;
    static constexpr int COLS = 32 * KS;
    static constexpr int LD = COLS + 8;
};

// Cooperative global -> LDS copy of ROWS rows of 16-byte chunks by NTH threads, in
// two halves so that a problem can put ALL its loads in flight before it waits
// for any of them: tile_issue starts the loads into registers, tile_commit
// writes them to LDS.  rowoff(row) gives the row's byte offset in the resource
// or kOob; columns at or beyond D are zero-filled.
template <class T, int DT, int ROWS, int NTH>
struct TileCopy {
    static constexpr int CH = Geom<DT>::COLS / 8;
    static constexpr int LD = Geom<DT>::LD;
    static constexpr int CNT = (ROWS * CH + NTH - 1) / NTH;
    static constexpr bool EVEN = ROWS * CH % NTH == 0;   // else the last round of chunks is not for every thread
    u32x4 val[CNT];

    template <int SHARED, class RowOff>
    __device__ __forceinline__ void issue(rsrc_t src, int D, RowOff rowoff, int tix) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * NTH;
            const int row = c / CH, ch = c % CH;
            const unsigned ro = (EVEN || c < ROWS * CH) ? rowoff(row) : kOob;
            val[i] = bload16<SHARED>(src, (ch * 8 < D) ? ro + ch * 16 : kOob);
        }
    }
    __device__ __forceinline__ void commit(T* tile, int tix) const {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * NTH;
            if (EVEN || c < ROWS * CH) *reinterpret_cast<u32x4*>(tile + (c / CH) * LD + (c % CH) * 8) = val[i];
        }
    }
};

// B operand of GEMM1 straight from memory: the row at byte offset ro (or kOob)
template <class T, int DT, int SHARED>
__device__ __forceinline__ void load_x(typename Ops<T>::v8 (&x)[Geom<DT>::KS], rsrc_t src, unsigned ro, int D, int q) {
#pragma unroll
    for (int ks = 0; ks < Geom<DT>::KS; ++ks) {
        const int col = 32 * ks + 8 * q;
        x[ks] = __builtin_bit_cast(typename Ops<T>::v8, bload16<SHARED>(src, col < D ? ro + col * 2 : kOob));
    }
}

template <class T>
__device__ __forceinline__ typename Ops<T>::v8 lds_row8(const T* tile_elem) {
    return __builtin_bit_cast(typename Ops<T>::v8, *reinterpret_cast<const u32x4*>(tile_elem));
}

// Which tile columns a lane ends up with after GEMM2: the first of the four consecutive columns
// that lane group g (r/4 of an MFMA row on the operand side, q of a lane on the result side) has in
// output tile dt.  Tiles 2p and 2p+1 give a lane the 8 columns 8*(g + 4p) .., a 16-byte piece, and
// the four lane groups of a row write 64 contiguous bytes with each store instruction; the last
// tile of an odd DT gives the lane groups the 4-column pieces behind those, 32 contiguous bytes.
// RUN (the kernel that keeps its state in LDS and writes little to memory asks for it: it is at
// its register limit and this form costs it three registers fewer): a lane's 4*DT columns are one
// consecutive run, 4*DT*g ...
template <int DT, bool RUN = false>
__host__ __device__ constexpr int chunk_col(int g, int dt) {
    return RUN ? 4 * DT * g + 4 * dt
               : (DT % 2 == 1 && dt == DT - 1) ? 16 * (DT - 1) + 4 * g : 8 * g + 32 * (dt >> 1) + 4 * (dt & 1);
}

// Transposed A operand of GEMM2 from a row-major LDS tile via ds_read_b64_tr_b16.
// Output tile dt, lane (r, q) = MFMA row r: the row is mapped to the tile column
// d = chunk_col(r/4, dt) + r%4, so that a lane of the C layout (rows 4q..4q+3) owns the columns
// chunk_col(q, dt) .. +3.  row0 is the tile row of k slot 0, hi_rows the distance to the row of
// k slot 4.
template <class T, int DT, bool RUN = false>
__device__ __forceinline__ typename Ops<T>::v8 lds_tr8(const T* tile, int row0, int hi_rows, bool with_hi, int dt, int r) {
    typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
    constexpr int LD = Geom<DT>::LD;
    const int e = r >> 2, c = r & 3;
    const T* p0 = tile + (row0 + e) * LD + chunk_col<DT, RUN>(c, dt);
    i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
    i16x4 hi = {0, 0, 0, 0};
    if (with_hi) hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0 + hi_rows * LD));
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    i16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(typename Ops<T>::v8, v);
}

// P (fp32, C layout, NWT tiles) -> B operands of GEMM2, rounded to T.  k slot s of
// step g is row w = 32g + 16(s/4) + 4q + s%4: slots 0-3 from C tile 2g, 4-7 from 2g+1.
template <class T, int NWT>
__device__ __forceinline__ void pack_p(typename Ops<T>::v8 (&pb)[(NWT + 1) / 2], const f32x4 (&C)[NWT]) {
#pragma unroll
    for (int g = 0; g < (NWT + 1) / 2; ++g) {
        typename Ops<T>::v8 v;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v[s] = from_f<T>(C[2 * g][s]);
            v[4 + s] = (2 * g + 1 < NWT) ? from_f<T>(C[2 * g + 1][s]) : from_f<T>(0.f);
        }
        pb[g] = v;
    }
}

// GEMM2: O[dt][v] = sum_w tile[w][chunk_col(q, dt) + v] * P[w][x = lane column]
template <class T, int DT, int NWT, bool RUN = false>
__device__ __forceinline__ void gemm2(f32x4 (&O)[DT], const T* tile, const typename Ops<T>::v8 (&pb)[(NWT + 1) / 2],
                                      int r, int q) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < (NWT + 1) / 2; ++g)
            acc = Ops<T>::mma(lds_tr8<T, DT, RUN>(tile, 32 * g + 4 * q, 16, 2 * g + 1 < NWT, dt, r), pb[g], acc);
        O[dt] = acc;
    }
}

// Store a lane's 4*DT output elements (columns chunk_col(q, dt) ..) of the row at byte offset ro
// (kOob drops the store) in 16-byte pieces - 8 columns at a multiple of 8, so with D a multiple of
// 8 (a condition of these kernels) a piece lies wholly inside or wholly beyond the row - plus one
// 8-byte piece per lane for the last tile of an odd DT.  (RUN: 16-byte pieces when the head dim
// fills the tiles exactly, else 8-byte pieces.)
// stream: the rows are whole 128-byte lines (see Slices::stream_*): they are written with
// streaming ("nt") stores, which leave for memory while the kernel still runs.  Plain stores
// are acknowledged early and the launch then ends with a long drain of its written lines
// (measured: 5 us after an R step that wrote 17 MB, against 2 us with streaming stores).
// Rows that share lines with other writers keep the plain policy (partial streaming
// writes are several times slower).
template <class T, int DT, bool RUN = false>
__device__ __forceinline__ void store_row(rsrc_t dst, unsigned ro, int D, const f32x4 (&O)[DT], int q, bool stream = false) {
    typedef typename Ops<T>::v4 V4;
    const unsigned base = ro + 2 * chunk_col<DT, RUN>(q, 0);  // bytes; the pieces sit at fixed distances from it
    const bool whole = D == 16 * DT;   // no piece lies beyond the row
    if (!RUN || (DT % 2 == 0 && whole)) {
#pragma unroll
        for (int p = 0; p < DT / 2; ++p) {
            V4 a = {from_f<T>(O[2 * p][0]), from_f<T>(O[2 * p][1]), from_f<T>(O[2 * p][2]), from_f<T>(O[2 * p][3])};
            V4 b = {from_f<T>(O[2 * p + 1][0]), from_f<T>(O[2 * p + 1][1]), from_f<T>(O[2 * p + 1][2]), from_f<T>(O[2 * p + 1][3])};
            const u32x2 lo = __builtin_bit_cast(u32x2, a), hi = __builtin_bit_cast(u32x2, b);
            const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
            unsigned off = base + 2 * (chunk_col<DT, RUN>(0, 2 * p) - chunk_col<DT, RUN>(0, 0));
            if (!whole) off = chunk_col<DT, RUN>(q, 2 * p) < D ? off : kOob;
            if (stream) __builtin_amdgcn_raw_buffer_store_b128(v, dst, off, 0, 2);
            else __builtin_amdgcn_raw_buffer_store_b128(v, dst, off, 0, 0);
        }
        if (DT % 2 == 1) {
            V4 a = {from_f<T>(O[DT - 1][0]), from_f<T>(O[DT - 1][1]), from_f<T>(O[DT - 1][2]), from_f<T>(O[DT - 1][3])};
            const int d0 = chunk_col<DT, RUN>(q, DT - 1);
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, a), dst, d0 < D ? ro + 2 * d0 : kOob, 0, 0);
        }
    } else {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            V4 a = {from_f<T>(O[dt][0]), from_f<T>(O[dt][1]), from_f<T>(O[dt][2]), from_f<T>(O[dt][3])};
            const int d0 = chunk_col<DT, RUN>(q, dt);
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, a), dst, d0 < D ? base + 2 * chunk_col<DT, RUN>(0, dt) : kOob, 0, 0);
        }
    }
}

// How a workgroup's W waves are shared among block problems with NT strips:
// WPP waves per problem (at most four: a wave of a 128-row problem walks two strips, one after
// the other, a wave of a 192- / 256-row problem three / four), PPW problems per workgroup.  Problems of 3 or 6 strips
// (blocks and block counts of 33-48 / 81-96, e.g. the 48- and 96-token blocks of the reference's
// RoBERTa sweep, experiments/roberta/benchmark.py:78) run on three waves: a per-stage launch uses
// workgroups of three waves (WG), a one-launch kernel leaves its fourth wave idle in such a phase.
template <int NT, int W = kWaves>
struct Split {
    static_assert(NT == 1 || NT == 2 || NT == 3 || NT == 4 || NT == 6 || NT == 8 || NT == 12 || NT == 16,
                  "strip counts are 1, 2, 3, 4, 6, 8, 12 or 16");
    static constexpr int WPP = (NT == 3 || NT == 6) ? 3 : (NT < kWaves ? NT : kWaves);
    static constexpr int PPW = W / WPP;
    static constexpr int WG = (NT == 3 || NT == 6) ? 3 : kWaves;   // waves of a per-stage launch's workgroup
};

// LDS bytes of one problem slot of each stage
template <class T, int DT, int NWT>
struct Lds {
    static constexpr int ROWS = 16 * NWT;
    static constexpr int TILE = ROWS * Geom<DT>::LD;                 // elements
    static constexpr size_t R = 2 * TILE * sizeof(T) + ROWS * sizeof(float);
    static constexpr size_t Z = 2 * TILE * sizeof(T) + ROWS * sizeof(float);
    static constexpr size_t L = 2 * TILE * sizeof(T) + 3 * ROWS * sizeof(float);
};

// Uniform (per problem) description of the tensors: resources and row pitches in bytes.
struct Slices {
    rsrc_t q, k, v, out, aR, cR, aL, cL, Y, mask;
    unsigned qst, kst, vst, ost, mst;   // mst: byte pitch of the mask's token dimension, 0 = no mask
    bool stream_state, stream_out;      // rows of the state arrays / of out are whole, aligned 128-byte lines
    bool agent_state;                   // state loads with agent scope instead of the streaming policy (Problem::state_agent)
};

template <class T>
__device__ __forceinline__ Slices make_slices(const Problem& P, int e, int h, long long wh) {
    Slices S;
    const unsigned n1 = static_cast<unsigned>(P.N - 1), db = static_cast<unsigned>(P.D) * sizeof(T);
    S.qst = static_cast<unsigned>(P.qs[2]) * sizeof(T);
    S.kst = static_cast<unsigned>(P.ks[2]) * sizeof(T);
    S.vst = static_cast<unsigned>(P.vs[2]) * sizeof(T);
    S.ost = static_cast<unsigned>(P.os[2]) * sizeof(T);
    S.q = make_rsrc(P.q + (e * P.qs[0] + h * P.qs[1]) * static_cast<long long>(sizeof(T)), n1 * S.qst + db);
    S.k = make_rsrc(P.k + (e * P.ks[0] + h * P.ks[1]) * static_cast<long long>(sizeof(T)), n1 * S.kst + db);
    S.v = make_rsrc(P.v + (e * P.vs[0] + h * P.vs[1]) * static_cast<long long>(sizeof(T)), n1 * S.vst + db);
    S.out = make_rsrc(P.out + (e * P.os[0] + h * P.os[1]) * static_cast<long long>(sizeof(T)), n1 * S.ost + db);
    S.mst = P.mask ? static_cast<unsigned>(P.ms[1]) << P.mask_shift : 0u;
    S.mask = make_rsrc(P.mask ? P.mask + ((e * P.ms[0]) << P.mask_shift) : nullptr, P.mask ? n1 * S.mst + (1u << P.mask_shift) : 0u);
    const long long np = static_cast<long long>(P.M) * P.B;
    const unsigned state = static_cast<unsigned>(np) * db, stat4 = static_cast<unsigned>(np) * 4u;
    S.aR = make_rsrc(P.aR + wh * np * db, state);
    S.aL = make_rsrc(P.aL + wh * np * db, state);
    S.Y = make_rsrc(P.Y + wh * np * db, state);
    S.cR = make_rsrc(P.cR + wh * np, stat4);
    S.cL = make_rsrc(P.cL + wh * np, stat4);
    // the state arrays are 256-byte aligned (workspace layout) with rows of db bytes
    S.stream_state = P.stream_stores != 0 && db % 128u == 0;
    S.agent_state = P.state_agent != 0;
    S.stream_out = P.stream_stores != 0 && db % 128u == 0 && S.ost % 128u == 0 &&
                   (reinterpret_cast<unsigned long long>(P.out) + static_cast<unsigned long long>(e * P.os[0] + h * P.os[1]) * sizeof(T)) % 128u == 0;
    return S;
}

// byte offset of real token t's row (pitch st) or kOob for a padding position
__device__ __forceinline__ unsigned tok_off(int t, int N, unsigned st) {
    return static_cast<unsigned>(t) < static_cast<unsigned>(N) ? static_cast<unsigned>(t) * st : kOob;
}

// Mask element of token t, started as a load and NOT looked at here (a test would wait for it and
// for every load issued before it): padding positions and "no mask" read 0 through the bounds
// check.  The element's words are folded into one (a 64-bit element is non-zero iff the OR of its
// halves is, once the sign bit of a floating-point mask is dropped from the high half; that fold is
// plain ALU work on the loaded registers and waits for nothing until its result is used).
// token_kept() decodes it once the problem runs.
__device__ __forceinline__ unsigned mask_load(const Slices& S, const Problem& P, int t, bool want) {
    if (P.mask == nullptr) return 1u;   // uniform: without a mask nothing is loaded
    const bool in = want && static_cast<unsigned>(t) < static_cast<unsigned>(P.N);
    const unsigned off = in ? (static_cast<unsigned>(t) * S.mst) : kOob;
    switch (P.mask_shift) {   // uniform
        case 0: return __builtin_amdgcn_raw_buffer_load_b8(S.mask, off, 0, 0);
        case 1: return __builtin_amdgcn_raw_buffer_load_b16(S.mask, off, 0, 0) & (P.mask_float ? 0x7fffu : 0xffffu);
        case 2: return __builtin_amdgcn_raw_buffer_load_b32(S.mask, off, 0, 0) & (P.mask_float ? 0x7fffffffu : 0xffffffffu);
        default: {
            const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(S.mask, off, 0, 0);
            return w[0] | (w[1] & (P.mask_float ? 0x7fffffffu : 0xffffffffu));
        }
    }
}
// real (in range) and not masked out
__device__ __forceinline__ bool token_kept(const Problem& P, int t, unsigned mask_word) {
    return static_cast<unsigned>(t) < static_cast<unsigned>(P.N) && (P.mask == nullptr || mask_word != 0u);
}

// Orders the LDS tile writes of a problem's waves before their reads.  A problem that a single
// wave owns (16-row problems) needs no workgroup barrier for that: the LDS executes one wave's
// instructions in order, so only the compiler has to be kept from moving them.  Every barrier
// inside a problem body goes through this, so all waves of a workgroup agree on whether they meet.
template <int WPP>
__device__ __forceinline__ void problem_sync() {
    if constexpr (WPP == 1) __builtin_amdgcn_wave_barrier();
    else __syncthreads();
}

// ============================================================================
// The three block problems.  Each is split in three parts so that a caller can
// overlap memory latency with other work:
//   issue()  starts the loads that depend only on the INPUTS (K / V / Q tiles and
//            rows, mask bytes) into registers (Pre) - they may be issued long
//            before the problem runs, e.g. while the previous problem computes;
//   state()  starts the loads of the STATE another phase produced (aR rows, aL /
//            Y tiles, cL, cR) into registers (St) - only legal once that phase
//            is known to be complete;
//   run()    commits the tiles to LDS and does the arithmetic; it contains no
//            global load of its own for problems of up to 64 rows.
// `active` is uniform per wave; inactive waves only take part in the barriers.
// ============================================================================

// R step for one block problem (e,h,m), run by WPP waves (wig = wave in group).
// smem: K tile, V tile, key bias.   Reference: al_cl_ref / al_y_cl_ref
// (ma/ma_torch.py:10-23, :38-52).
// HV = 2: the problem is run as two halves of NWT / 2 query strips by two workgroups, `half` = 0, 1 (both
// stage the whole key / value tiles); a per-stage launch asks for it when it would not fill the device.
template <class T, int DT, int NWT, int HV = 1>
struct RProb {
    using G = Geom<DT>;
    using V8 = typename Ops<T>::v8;
    static constexpr int WPP = Split<NWT>::WPP;
    static_assert(NWT % (WPP * HV) == 0, "a half must be whole strips per wave");
    static constexpr int SPW = NWT / WPP / HV;   // strips per wave: 2 for blocks of more than 64 rows
    static constexpr int ROWS = Lds<T, DT, NWT>::ROWS;
    static __device__ __forceinline__ int strip_of(int wig, int i, int half) { return half * (NWT / HV) + wig + i * WPP; }
    struct Pre {
        TileCopy<T, DT, ROWS, WPP * 64> kc, vc;
        V8 xq[SPW][G::KS];   // first step: the Q rows of this wave's strips
        unsigned km;         // mask byte of the key token of tile row `tix`
    };
    struct St {
        V8 xa[SPW][G::KS];   // later steps: the aR rows of this wave's strips
        float cr[SPW];
    };

    // NT: the inputs are loaded with the streaming policy (a caller's choice: streaming inputs leave the L2 to
    // the state, which pays where nothing re-reads them from it - few long heads in one launch; ordinary
    // loads keep K and Q in L2 for the later steps of many-head and per-stage launches).  Q is the
    // exception when there are L steps to come (T > 1): they and the Z step read it again, and the
    // caller that streams everything else measured 3 - 5 % faster at T = 2, 3 with Q kept (T = 1: no gain).
    template <bool NT = false>
    static __device__ __forceinline__ void issue(const Problem& P, const Slices& S, Pre& pre, bool active, int e, int m, bool first,
                                                 bool with_v, int wig, int lane, int half = 0) {
        if (!active) return;
        const int B = P.B, D = P.D;
        const int tix = wig * 64 + lane;
        const int t0 = m * B - P.pad_off;
        // order of issue = order of arrival: what the logits need first, the V tile (needed last) last
        pre.kc.template issue<NT>(S.k, D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.kst) : kOob; }, tix);
        if (first) {
#pragma unroll
            for (int i = 0; i < SPW; ++i) {
                const int j = 16 * strip_of(wig, i, half) + (lane & 15);
                const unsigned ro = j < B ? tok_off(t0 + j, P.N, S.qst) : kOob;
                if (NT && P.T == 1) load_x<T, DT, true>(pre.xq[i], S.q, ro, D, lane >> 4);
                else load_x<T, DT, false>(pre.xq[i], S.q, ro, D, lane >> 4);
            }
        }
        pre.km = mask_load(S, P, t0 + tix, tix < B);
        if (with_v) issue_v<NT>(P, S, pre, active, m, wig, lane);
    }
    // the V tile alone (a caller that starts the state loads right away issues it after them)
    template <bool NT = false>
    static __device__ __forceinline__ void issue_v(const Problem& P, const Slices& S, Pre& pre, bool active, int m, int wig, int lane) {
        if (!active) return;
        const int B = P.B;
        const int t0 = m * B - P.pad_off;
        pre.vc.template issue<NT>(S.v, P.D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.vst) : kOob; }, wig * 64 + lane);
    }

    template <int POL>
    static __device__ __forceinline__ void load_state_strip(const Problem& P, const Slices& S, V8 (&xa)[G::KS], float& cr, int m,
                                                            int strip, int lane) {
        const int j = 16 * strip + (lane & 15);
        const unsigned rowid = static_cast<unsigned>(m * P.B + j);   // row inside the head's state
        const unsigned db = static_cast<unsigned>(P.D) * sizeof(T);
        load_x<T, DT, POL>(xa, S.aR, j < P.B ? rowid * db : kOob, P.D, lane >> 4);
        cr = bloadf<POL>(S.cR, j < P.B ? rowid * 4u : kOob);   // an out-of-range row reads 0: harmless, never stored
    }

    static __device__ __forceinline__ void state(const Problem& P, const Slices& S, St& st, bool active, int m, bool first, int wig,
                                                 int lane, int half = 0) {
#pragma unroll
        for (int i = 0; i < SPW; ++i) {
            st.cr[i] = 1.0f;
            if (active && !first) {
                if (S.agent_state) load_state_strip<kPolAgent>(P, S, st.xa[i], st.cr[i], m, strip_of(wig, i, half), lane);   // uniform
                else load_state_strip<kPolStream>(P, S, st.xa[i], st.cr[i], m, strip_of(wig, i, half), lane);
            }
        }
    }

    static __device__ __forceinline__ void run(const Problem& P, const Slices& S, char* smem, const Pre& pre, const St& st, bool active,
                                               int m, bool first, bool with_v, int wig, int lane, int half = 0) {
        T* Kt = reinterpret_cast<T*>(smem);
        T* Vt = Kt + Lds<T, DT, NWT>::TILE;
        float* kbias = reinterpret_cast<float*>(Vt + Lds<T, DT, NWT>::TILE);
        const int B = P.B, M = P.M, D = P.D;
        const int r = lane & 15, q = lane >> 4;
        const int tix = wig * 64 + lane;
        const unsigned db = static_cast<unsigned>(D) * sizeof(T);
        if (active) {
            pre.kc.commit(Kt, tix);
            if (with_v) pre.vc.commit(Vt, tix);
            if (tix < ROWS) kbias[tix] = (tix < P.B && token_kept(P, m * P.B - P.pad_off + tix, pre.km)) ? 0.f : kNegBig;
        }
        problem_sync<WPP>();
#pragma unroll
        for (int si = 0; si < SPW; ++si) {
          f32x4 OY[DT];
          V8 pb[(NWT + 1) / 2];
          bool jv = false;
          unsigned lrow = 0;
          if (active) {
            const int strip = strip_of(wig, si, half);
            const int j = 16 * strip + r;
            jv = j < B;
            V8 xb[G::KS];
#pragma unroll
            for (int ks = 0; ks < G::KS; ++ks) xb[ks] = first ? pre.xq[si][ks] : st.xa[si][ks];
            const float cr = st.cr[si];
            const float cj = (P.sm_scale * kLog2e) * rcp(cr + P.eps);  // logits in log2 units

            f32x4 C[NWT];
#pragma unroll
            for (int wt = 0; wt < NWT; ++wt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < G::KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(Kt + (16 * wt + r) * G::LD + 32 * ks + 8 * q), xb[ks], acc);
                const f32x4 kb = *reinterpret_cast<const f32x4*>(kbias + 16 * wt + 4 * q);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[v] = fmaf(round_to<T>(acc[v]), cj, kb[v]);
                C[wt] = acc;
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
                    ent = fmaf(p, d, ent);  // sum p * log2(p)
                    C[wt][v] = p;
                }
            sum = quad_rows_sum(sum);
            ent = quad_rows_sum(ent);
            const float den = sum + P.eps;
            const float inv = rcp(den);
#pragma unroll
            for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
                for (int v = 0; v < 4; ++v) C[wt][v] *= inv;
            // cL = sum_i r log r with r = p / den (ma_torch.py:20); rows of tiny r add ~1e-36
            lrow = static_cast<unsigned>(j * M + m);   // row of aL / cL / Y: (j, m)
            if (q == 0)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, kLn2 * (ent * inv - log2_normal(den) * (sum * inv))),
                                                      S.cL, jv ? lrow * 4u : kOob, 0, 0);

            pack_p<T, NWT>(pb, C);
            {
                f32x4 O[DT];
                gemm2<T, DT, NWT>(O, Kt, pb, r, q);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) O[dt][v] = P.sm_scale * round_to<T>(O[dt][v]);
                store_row<T, DT>(S.aL, jv ? lrow * db : kOob, D, O, q, S.stream_state);
            }
          }
          if (with_v) {
            if (active) {
                gemm2<T, DT, NWT>(OY, Vt, pb, r, q);
                store_row<T, DT>(S.Y, jv ? lrow * db : kOob, D, OY, q, S.stream_state);
            }
          }
        }
    }
};

// Index x of a 16-row tile of an L / Z problem -> (in-block position, block).  A problem of a head with
// more than 16 blocks, and every problem of the one-launch kernels, belongs to ONE position j: x is the
// block.  Per-stage launches of heads with at most 8 blocks pack several positions into the tile
// (Problem::pack_shift): x stands for block x % pack_m of position j + x / pack_m, the logits between
// different positions are masked out (a block-diagonal problem), everything else is unchanged.
template <int NWT>
struct TileIndex {
    int j, sh;
    __device__ __forceinline__ TileIndex(const Problem& P, int j_) : j(j_), sh(NWT == 1 ? P.pack_shift : 4) {}
    __device__ __forceinline__ int pos(int x) const { return NWT == 1 ? j + (x >> sh) : j; }
    __device__ __forceinline__ int blk(int x) const { return NWT == 1 ? (x & ((1 << sh) - 1)) : x; }
    __device__ __forceinline__ bool ok(const Problem& P, int x) const { return blk(x) < P.M && pos(x) < P.B; }
    __device__ __forceinline__ bool same(int x, int y) const { return NWT != 1 || (x >> sh) == (y >> sh); }
    // token of query block blk(x) at position pos(x)
    __device__ __forceinline__ int token(const Problem& P, int x) const { return blk(x) * P.B + pos(x) - P.pad_off; }
    // row of the (.., B, M, .) state arrays
    __device__ __forceinline__ unsigned state_row(const Problem& P, int x) const { return static_cast<unsigned>(pos(x) * P.M + blk(x)); }
};

// Z step for one column problem (e,h,j).  smem: aL tile, Y tile, cL bias.
// Reference: z_ref (ma/ma_torch.py:55-62) and the final slice (:106-108).
template <class T, int DT, int NWT, int HV = 1>   // HV: as in RProb
struct ZProb {
    using G = Geom<DT>;
    using V8 = typename Ops<T>::v8;
    static constexpr int WPP = Split<NWT>::WPP;
    static constexpr int ROWS = Lds<T, DT, NWT>::ROWS;
    static_assert(NWT % (WPP * HV) == 0, "a half must be whole strips per wave");
    static constexpr int SPW = NWT / WPP / HV;   // strips per wave
    static __device__ __forceinline__ int strip_of(int wig, int i, int half) { return half * (NWT / HV) + wig + i * WPP; }
    struct Pre {
        V8 xq[SPW][G::KS];   // the Q rows of this wave's strips
    };
    struct St {
        TileCopy<T, DT, ROWS, WPP * 64> ac, yc;
        float cbv;      // softmax bias of tile row `tix`
    };

    template <bool NT>
    static __device__ __forceinline__ void load_strip(const Problem& P, const Slices& S, V8 (&xb)[G::KS], int j, int strip, int lane) {
        const TileIndex<NWT> ti(P, j);
        const int l = 16 * strip + (lane & 15);
        load_x<T, DT, NT>(xb, S.q, ti.ok(P, l) ? tok_off(ti.token(P, l), P.N, S.qst) : kOob, P.D, lane >> 4);
    }
    template <bool NT = false>
    static __device__ __forceinline__ void issue(const Problem& P, const Slices& S, Pre& pre, bool active, int j, int wig, int lane,
                                                 int half = 0) {
        if (!active) return;
#pragma unroll
        for (int i = 0; i < SPW; ++i) load_strip<NT>(P, S, pre.xq[i], j, strip_of(wig, i, half), lane);
    }
    static __device__ __forceinline__ void state(const Problem& P, const Slices& S, St& st, bool active, int j, int wig, int lane) {
        if (!active) return;
        const int D = P.D;
        const int tix = wig * 64 + lane;
        const unsigned db = static_cast<unsigned>(D) * sizeof(T);
        const TileIndex<NWT> ti(P, j);
        // the Y tile (needed last) last
        const auto rowoff = [&](int k) { return ti.ok(P, k) ? ti.state_row(P, k) * db : kOob; };
        const unsigned cloff = (tix < ROWS && ti.ok(P, tix)) ? ti.state_row(P, tix) * 4u : kOob;
        float clv;
        if (S.agent_state) {   // uniform
            st.ac.template issue<kPolAgent>(S.aL, D, rowoff, tix);
            clv = bloadf<kPolAgent>(S.cL, cloff);
            st.yc.template issue<kPolAgent>(S.Y, D, rowoff, tix);
        } else {
            st.ac.template issue<kPolStream>(S.aL, D, rowoff, tix);
            clv = bloadf<kPolStream>(S.cL, cloff);
            st.yc.template issue<kPolStream>(S.Y, D, rowoff, tix);
        }
        st.cbv = (tix < ROWS && ti.ok(P, tix)) ? -kLog2e * clv : kNegBig;
    }
    static __device__ __forceinline__ void run(const Problem& P, const Slices& S, char* smem, const Pre& pre, const St& st, bool active,
                                               int j, int wig, int lane, int half = 0) {
        T* At = reinterpret_cast<T*>(smem);
        T* Yt = At + Lds<T, DT, NWT>::TILE;
        float* cb = reinterpret_cast<float*>(Yt + Lds<T, DT, NWT>::TILE);
        const int D = P.D;
        const int r = lane & 15, q = lane >> 4;
        const int tix = wig * 64 + lane;
        const TileIndex<NWT> ti(P, j);
        if (active) {
            st.ac.commit(At, tix);
            st.yc.commit(Yt, tix);
            if (tix < ROWS) cb[tix] = st.cbv;
        }
        problem_sync<WPP>();
#pragma unroll
        for (int si = 0; si < SPW; ++si) {
          V8 pb[(NWT + 1) / 2];
          if (active) {
            const int strip = strip_of(wig, si, half);
            V8 xb[G::KS];
#pragma unroll
            for (int ks = 0; ks < G::KS; ++ks) xb[ks] = pre.xq[si][ks];
            f32x4 C[NWT];
#pragma unroll
            for (int wt = 0; wt < NWT; ++wt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < G::KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(At + (16 * wt + r) * G::LD + 32 * ks + 8 * q), xb[ks], acc);
                const f32x4 b = *reinterpret_cast<const f32x4*>(cb + 16 * wt + 4 * q);
#pragma unroll
                for (int v = 0; v < 4; ++v)   // (packed tiles: only the key blocks of the query's own position count)
                    acc[v] = ti.same(16 * wt + 4 * q + v, 16 * strip + r) ? fmaf(round_to<T>(acc[v]), kLog2e, b[v]) : kNegBig;
                C[wt] = acc;
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
            pack_p<T, NWT>(pb, C);
          }
          if (active) {
            const int l = 16 * strip_of(wig, si, half) + r;
            f32x4 O[DT];
            gemm2<T, DT, NWT>(O, Yt, pb, r, q);
            store_row<T, DT>(S.out, ti.ok(P, l) ? tok_off(ti.token(P, l), P.N, S.ost) : kOob, D, O, q, S.stream_out);   // padded query rows are dropped (:108)
          }
        }
    }
};

// NaN into the output rows of column problem (e,h,j): what a one-launch kernel writes instead of
// results when the workgroup that owns the rows gave up waiting for the state they depend on.
template <class T, int DT, int NWT>
__device__ __forceinline__ void z_poison(const Problem& P, const Slices& S, int j, int wig, int lane) {
    constexpr int WPP = Split<NWT>::WPP, SPW = NWT / WPP;
    const int r = lane & 15, q = lane >> 4;
    f32x4 O[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) O[dt] = f32x4{__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""), __builtin_nanf("")};
    const TileIndex<NWT> ti(P, j);
#pragma unroll
    for (int si = 0; si < SPW; ++si) {
        const int l = 16 * (wig + si * WPP) + r;
        store_row<T, DT>(S.out, ti.ok(P, l) ? tok_off(ti.token(P, l), P.N, S.ost) : kOob, P.D, O, q);
    }
}

// L step for one column problem (e,h,j).  smem: Q^T tile, aL tile, softmax bias of the key blocks,
// row maximum and 1 / row sum of the query blocks.  Reference: ar_cr_ref (ma/ma_torch.py:26-35).
//
// The softmax runs over the key blocks k of every query block l, the product that follows
// contracts over l - and a lane can only feed the second product from accumulators whose ROWS are
// the contraction index, while a softmax is cheapest along the rows of the accumulators (in-lane
// plus two lane swaps).  So the logits are formed twice:
//   pass 1, wave = strip of query blocks l (accumulator rows = key blocks k): maximum and sum of
//           every row l, kept in LDS;
//   pass 2, wave = strip of key blocks k (accumulator rows = query blocks l): the logits again with
//           the operand roles swapped, the probabilities from pass 1's statistics, straight into
//           the B operand of aR[k] = sum_l L[l,k] Q[l]; cR[k] = sum_l L[l,k] in-lane.
// The second evaluation costs a few instructions on idle matrix pipes and a second exp2 per entry;
// it saves the transposed copy of the probabilities in LDS (which was as large as both operand
// tiles together and halved the workgroups per compute unit), its write, its read and the 16-lane
// reductions of the column-wise softmax.
template <class T, int DT, int NWT>
struct LProb {
    using G = Geom<DT>;
    using V8 = typename Ops<T>::v8;
    using LS = Lds<T, DT, NWT>;
    static constexpr int WPP = Split<NWT>::WPP;
    static constexpr int ROWS = LS::ROWS;
    static constexpr int nth = WPP * 64;
    static constexpr int SPW = NWT / WPP;   // strips per wave (2 for blocks counts above 64)
    struct Pre {
        TileCopy<T, DT, ROWS, nth> qc;   // Q^T tile
        unsigned qm[SPW];                // mask word of the query token of block 16*(wig + i*WPP) + lane % 16
    };
    struct St {
        TileCopy<T, DT, ROWS, nth> ac;    // aL tile
        float cbv;
    };

    template <bool NT = false>
    static __device__ __forceinline__ void issue(const Problem& P, const Slices& S, Pre& pre, bool active, int e, int j, int wig,
                                                 int lane) {
        if (!active) return;
        const int tix = wig * 64 + lane;
        const TileIndex<NWT> ti(P, j);
        // (never streamed: an L step is followed by at least the Z step, which reads Q again)
        pre.qc.template issue<false>(S.q, P.D, [&](int l) { return ti.ok(P, l) ? tok_off(ti.token(P, l), P.N, S.qst) : kOob; }, tix);
#pragma unroll
        for (int i = 0; i < SPW; ++i) {
            const int l = 16 * (wig + i * WPP) + (lane & 15);
            pre.qm[i] = mask_load(S, P, ti.token(P, l), ti.ok(P, l));
        }
    }
    static __device__ __forceinline__ void state(const Problem& P, const Slices& S, St& st, bool active, int j, int wig, int lane) {
        if (!active) return;
        const int D = P.D;
        const int tix = wig * 64 + lane;
        const unsigned db = static_cast<unsigned>(D) * sizeof(T);
        const TileIndex<NWT> ti(P, j);
        const auto rowoff = [&](int k) { return ti.ok(P, k) ? ti.state_row(P, k) * db : kOob; };
        const unsigned cloff = (tix < ROWS && ti.ok(P, tix)) ? ti.state_row(P, tix) * 4u : kOob;
        float clv;
        if (S.agent_state) {   // uniform
            st.ac.template issue<kPolAgent>(S.aL, D, rowoff, tix);
            clv = bloadf<kPolAgent>(S.cL, cloff);
        } else {
            st.ac.template issue<kPolStream>(S.aL, D, rowoff, tix);
            clv = bloadf<kPolStream>(S.cL, cloff);
        }
        st.cbv = (tix < ROWS && ti.ok(P, tix)) ? -kLog2e * clv : kNegBig;
    }
    static __device__ __forceinline__ void run(const Problem& P, const Slices& S, char* smem, const Pre& pre, const St& st, bool active,
                                               int j, int wig, int lane) {
        T* Qt = reinterpret_cast<T*>(smem);
        T* At = Qt + LS::TILE;
        float* cb = reinterpret_cast<float*>(At + LS::TILE);
        float* mxs = cb + ROWS;
        float* invs = mxs + ROWS;
        const int B = P.B, D = P.D;
        const int r = lane & 15, q = lane >> 4;
        const int tix = wig * 64 + lane;
        const unsigned db = static_cast<unsigned>(D) * sizeof(T);
        const TileIndex<NWT> ti(P, j);
        if (active) {
            pre.qc.commit(Qt, tix);
            st.ac.commit(At, tix);
            if (tix < ROWS) cb[tix] = st.cbv;
        }
        problem_sync<WPP>();
        if (active) {
            // pass 1: lane holds query block l = l0 + r, rows = key blocks 16kt + 4q + v
#pragma unroll
            for (int si = 0; si < SPW; ++si) {
                const int l = 16 * (wig + si * WPP) + r;
                V8 xq[G::KS];
#pragma unroll
                for (int ks = 0; ks < G::KS; ++ks) xq[ks] = lds_row8<T>(Qt + l * G::LD + 32 * ks + 8 * q);
                f32x4 C[NWT];
                float mx = kNegBig;
#pragma unroll
                for (int kt = 0; kt < NWT; ++kt) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < G::KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(At + (16 * kt + r) * G::LD + 32 * ks + 8 * q), xq[ks], acc);
                    const f32x4 b = *reinterpret_cast<const f32x4*>(cb + 16 * kt + 4 * q);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {   // (packed tiles: only the key blocks of the query's own position count)
                        acc[v] = ti.same(16 * kt + 4 * q + v, l) ? fmaf(round_to<T>(acc[v]), kLog2e, b[v]) : kNegBig;
                        mx = fmaxf(mx, acc[v]);
                    }
                    C[kt] = acc;
                }
                mx = quad_rows_max(mx);
                float sum = 0.f;
#pragma unroll
                for (int kt = 0; kt < NWT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) sum += __builtin_amdgcn_exp2f(C[kt][v] - mx);
                sum = quad_rows_sum(sum);
                if (q == 0) {
                    mxs[l] = mx;
                    // padded / masked query tokens are zeroed after the softmax (ma_torch.py:30)
                    invs[l] = (ti.ok(P, l) && token_kept(P, ti.token(P, l), pre.qm[si])) ? rcp(sum) : 0.f;
                }
            }
        }
        problem_sync<WPP>();
        if (active) {
            // pass 2: lane holds key block k = 16 strip + r, rows = query blocks 16lt + 4q + v
#pragma unroll
            for (int si = 0; si < SPW; ++si) {
                const int k = 16 * (wig + si * WPP) + r;
                const bool kv = ti.ok(P, k);
                V8 xk[G::KS];
#pragma unroll
                for (int ks = 0; ks < G::KS; ++ks) xk[ks] = lds_row8<T>(At + k * G::LD + 32 * ks + 8 * q);
                const float cbk = cb[k];
                f32x4 C[NWT];
                float crs = 0.f;
#pragma unroll
                for (int lt = 0; lt < NWT; ++lt) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < G::KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(Qt + (16 * lt + r) * G::LD + 32 * ks + 8 * q), xk[ks], acc);
                    const f32x4 mx4 = *reinterpret_cast<const f32x4*>(mxs + 16 * lt + 4 * q);
                    const f32x4 inv4 = *reinterpret_cast<const f32x4*>(invs + 16 * lt + 4 * q);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float u = ti.same(16 * lt + 4 * q + v, k) ? fmaf(round_to<T>(acc[v]), kLog2e, cbk) : kNegBig;
                        const float lv = __builtin_amdgcn_exp2f(u - mx4[v]) * inv4[v];
                        crs += lv;
                        acc[v] = lv;
                    }
                    C[lt] = acc;
                }
                crs = quad_rows_sum(crs);
                // aR[k, :] = sum_l round(L[l,k]) Qt[l, :]
                V8 pb[(NWT + 1) / 2];
                pack_p<T, NWT>(pb, C);
                f32x4 O[DT];
                gemm2<T, DT, NWT>(O, Qt, pb, r, q);
                const unsigned arow = static_cast<unsigned>(ti.blk(k) * B + ti.pos(k));   // row of aR / cR: (block, position)
                store_row<T, DT>(S.aR, kv ? arow * db : kOob, D, O, q, S.stream_state);
                if (q == 0) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, crs), S.cR, kv ? arow * 4u : kOob, 0, 0);
            }
        }
    }
};

// the three parts back to back (one launch per half step has nothing to overlap them with)
template <class T, int DT, int NWT, int HV = 1>
__device__ __forceinline__ void r_problem(const Problem& P, char* smem, bool active, int e, int h, long long wh, int m,
                                          bool first, bool with_v, int wig, int lane, int half = 0) {
    using RP = RProb<T, DT, NWT, HV>;
    const Slices S = make_slices<T>(P, e, h, wh);
    typename RP::Pre pre;
    typename RP::St st;
    RP::issue(P, S, pre, active, e, m, first, false, wig, lane, half);
    RP::state(P, S, st, active, m, first, wig, lane, half);
    if (with_v) RP::issue_v(P, S, pre, active, m, wig, lane);
    RP::run(P, S, smem, pre, st, active, m, first, with_v, wig, lane, half);
}
template <class T, int DT, int NWT, int HV = 1>
__device__ __forceinline__ void z_problem(const Problem& P, char* smem, bool active, int e, int h, long long wh, int j,
                                          int wig, int lane, int half = 0) {
    using ZP = ZProb<T, DT, NWT, HV>;
    const Slices S = make_slices<T>(P, e, h, wh);
    typename ZP::Pre pre;
    typename ZP::St st;
    ZP::issue(P, S, pre, active, j, wig, lane, half);
    ZP::state(P, S, st, active, j, wig, lane);
    ZP::run(P, S, smem, pre, st, active, j, wig, lane, half);
}
template <class T, int DT, int NWT>
__device__ __forceinline__ void l_problem(const Problem& P, char* smem, bool active, int e, int h, long long wh, int j,
                                          int wig, int lane) {
    using LP = LProb<T, DT, NWT>;
    const Slices S = make_slices<T>(P, e, h, wh);
    typename LP::Pre pre;
    typename LP::St st;
    LP::state(P, S, st, active, j, wig, lane);
    LP::issue(P, S, pre, active, e, j, wig, lane);
    LP::run(P, S, smem, pre, st, active, j, wig, lane);
}

// ---- staged kernels: one launch per half step ---------------------------------
// Workgroup -> (problem, half) when a launch runs its problems as two halves (HV = 2, one problem per
// workgroup): workgroups b and b + 8 are the halves of one problem - same XCD, dispatched close together,
// so the second finds the operand tiles the first staged in that XCD's L2.
__device__ __forceinline__ unsigned half_problem(unsigned b, int& half) {
    half = static_cast<int>((b >> 3) & 1u);
    return ((b >> 4) << 3) | (b & 7u);
}

template <class T, int DT, int NWT, int HV = 1>
__global__ __launch_bounds__(64 * Split<NWT>::WG) void r_step_mfma(Problem P, int first, int with_v) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, PPW = Split<NWT, Split<NWT>::WG>::PPW;
    static_assert(HV == 1 || PPW == 1, "halves: one problem per workgroup");
    const int wave = wave_id(), lane = threadIdx.x & 63;
    const int slot = wave / WPP, wig = wave % WPP;
    // E * H * Np fits int32 (validated by the host), so all problem indices are 32-bit
    const unsigned total = static_cast<unsigned>(P.E) * P.H * P.M;
    int half = 0;
    unsigned pid = HV == 1 ? blockIdx.x * PPW + slot : half_problem(blockIdx.x, half);
    const bool active = pid < total;
    if (!active) pid = 0;
    const int m = pid % static_cast<unsigned>(P.M);
    const unsigned eh = pid / static_cast<unsigned>(P.M);
    const int h = eh % static_cast<unsigned>(P.H);
    const int e = eh / static_cast<unsigned>(P.H);
    r_problem<T, DT, NWT, HV>(P, smem + slot * Lds<T, DT, NWT>::R, active, e, h, static_cast<long long>(eh), m, first != 0,
                              with_v != 0, wig, lane, half);
}

template <class T, int DT, int NWT>
__global__ __launch_bounds__(64 * Split<NWT>::WG) void l_step_mfma(Problem P) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, PPW = Split<NWT, Split<NWT>::WG>::PPW;
    const int wave = wave_id(), lane = threadIdx.x & 63;
    const int slot = wave / WPP, wig = wave % WPP;
    // problems per head: one per in-block position, or per group of positions that share a tile (TileIndex)
    const unsigned per = NWT == 1 ? static_cast<unsigned>(16 >> P.pack_shift) : 1u;
    const unsigned groups = (static_cast<unsigned>(P.B) + per - 1) / per;
    const unsigned total = static_cast<unsigned>(P.E) * P.H * groups;
    unsigned pid = blockIdx.x * PPW + slot;
    const bool active = pid < total;
    if (!active) pid = 0;
    const int j = static_cast<int>((pid % groups) * per);
    const unsigned eh = pid / groups;
    const int h = eh % static_cast<unsigned>(P.H);
    const int e = eh / static_cast<unsigned>(P.H);
    l_problem<T, DT, NWT>(P, smem + slot * Lds<T, DT, NWT>::L, active, e, h, static_cast<long long>(eh), j, wig, lane);
}

template <class T, int DT, int NWT, int HV = 1>
__global__ __launch_bounds__(64 * Split<NWT>::WG) void z_step_mfma(Problem P) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int WPP = Split<NWT>::WPP, PPW = Split<NWT, Split<NWT>::WG>::PPW;
    static_assert(HV == 1 || PPW == 1, "halves: one problem per workgroup");
    const int wave = wave_id(), lane = threadIdx.x & 63;
    const int slot = wave / WPP, wig = wave % WPP;
    // problems per head: one per in-block position, or per group of positions that share a tile (TileIndex)
    const unsigned per = NWT == 1 ? static_cast<unsigned>(16 >> P.pack_shift) : 1u;
    const unsigned groups = (static_cast<unsigned>(P.B) + per - 1) / per;
    const unsigned total = static_cast<unsigned>(P.E) * P.H * groups;
    int half = 0;
    unsigned pid = HV == 1 ? blockIdx.x * PPW + slot : half_problem(blockIdx.x, half);
    const bool active = pid < total;
    if (!active) pid = 0;
    const int j = static_cast<int>((pid % groups) * per);
    const unsigned eh = pid / groups;
    const int h = eh % static_cast<unsigned>(P.H);
    const int e = eh / static_cast<unsigned>(P.H);
    z_problem<T, DT, NWT, HV>(P, smem + slot * Lds<T, DT, NWT>::Z, active, e, h, static_cast<long long>(eh), j, wig, lane, half);
}

}  // namespace mfma
}  // namespace ma
