// Head-resident forward: one workgroup runs a whole head with EVERYTHING in LDS - the head's Q, K and V
// rows as well as the state (aL, aR, Y, cL, cR of monarch_attention_torch, ma/ma_torch.py:88-104) - from
// the first step to the last.  Q, K, V are read from memory once per head, the output is written once,
// and a block problem is nothing but LDS reads, matrix products and the softmax: no loads, no staging, no
// address arithmetic beyond "row of the head + lane's constant".
//
// Why it exists: the small block problems of short heads (16 x 16 ... 32 x 32) are bound by the number of
// instructions a compute unit issues - a wave's instruction takes a four-cycle turn of its SIMD whatever its
// type, and the waves of a workgroup move through a round in step, so a round costs (instructions per wave)
// x (waves per SIMD) x 4 cycles.  The tile-pipelined resident kernel (ma_resident.h) spends half of a
// round's instructions on starting, committing and addressing that round's input tiles; here the inputs of
// the NEXT head are loaded once, by all threads, into registers while the current head computes, and are
// written to LDS at the head boundary.
//
// It applies when four tiles of Np rows fit the 160 KB of LDS (heads of up to ~270 padded tokens at
// D = 64): S (aL and aR share it in place: the R problem of block m reads the rows aR(m, .) and writes
// aL(., m) over them, the L problem of position j reads aL(j, .) and writes aR(., j) over those), Q, K
// and V.  Y takes the place of V: the last R problem of block m is the only reader of V's rows of block m
// and writes its Y rows over them when it has read them.  All four tiles, cR and Y index a token by its
// row p = m*B + j of the padded sequence, so every row a problem touches is (block row) + (lane's row).
// A block's rows start 16 bytes later than B rows behind the block before it: the rows at one position of
// 16 consecutive blocks - what the lanes of an L or Z problem read with one instruction - would otherwise
// all start in the same LDS bank whenever the block size is a multiple of 16.
//
//   S     aR(m, j), then aL(j, m), ...            row m*B + j
//   Q, K  the padded inputs (zero rows for padding, ma/ma_torch.py:81-86), with zero rows behind the last block
//         up to the 16 * NTB rows an R problem reads
//   V     likewise; the last R phase leaves Y(j, m) in row m*B + j
//   ZR    a row of zeros (stands in for rows beyond the tile tails), TR a row nobody reads
//   cb    [j][k] (pitch 16*NTM): -log2(e) * cL(j, k), the bias of key block k in the softmax over k of the
//         L and Z problems of position j; -1e30 for k >= M
//   cR    [m*B + j]
//   tokb  [m][i] (pitch 16*NTB): 0 for a real, unmasked token i of block m, else -1e30 (the key bias of the
//         R problems; a query token with a non-zero entry is zeroed after the softmax of the L problems)
//   mxs, invs  per L problem in flight: row maximum and 1 / row sum of its query blocks
#pragma once

#include "ma_mfma.h"

namespace ma {
namespace mfma {

template <class T, int DT, int NTB, int NTM, int W, int NI>   // NI: 16-byte chunks per thread and input tile
struct HeadRes {
    using G = Geom<DT>;
    using V8 = typename Ops<T>::v8;
    using V4 = typename Ops<T>::v4;
    static_assert(NTB <= 4 && NTM <= 4, "one strip per wave: blocks and block counts of at most 64");
    static constexpr int LD = G::LD, KS = G::KS, CH = G::COLS / 8;
    static constexpr int WPB = NTB, PPB = W / WPB;   // waves per R problem, R problems per round
    static constexpr int WPM = NTM, PPM = W / WPM;   // same for the L / Z problems
    static constexpr int ROWSB = 16 * NTB, ROWSM = 16 * NTM;
    static constexpr int NT = 64 * W;
    // zero rows behind the input tiles: an R problem reads 16 * NTB rows from the first row of its block on, also in the last block
    static __host__ __device__ int pad_rows(int B) { return ROWSB > B ? ROWSB - B : 0; }
    static constexpr unsigned RB = LD * sizeof(T);   // bytes of a tile row
    static constexpr unsigned kSkew = 16;            // bytes a block's rows are shifted against the block before
    static __host__ __device__ unsigned block_pitch(int B) { return static_cast<unsigned>(B) * RB + kSkew; }

    struct Layout {
        unsigned S, Q, K, V, ZR, TR, cb, cR, tokb, stats, trash, total;
    };
    static __host__ __device__ Layout layout(int Np, int B, int M) {
        Layout L;
        unsigned o = 0;
        // (the rows behind the last block count as further blocks of B rows)
        const unsigned tile = static_cast<unsigned>(Np + pad_rows(B)) * RB + static_cast<unsigned>((Np + pad_rows(B)) / B + 1) * kSkew;
        L.S = o; o += tile;
        L.Q = o; o += tile;
        L.K = o; o += tile;
        L.V = o; o += tile;
        L.ZR = o; o += RB;
        L.TR = o; o += RB;
        L.cb = o; o += static_cast<unsigned>(B) * ROWSM * 4;
        L.cR = o; o += static_cast<unsigned>((Np + 3) / 4 * 4) * 4;
        L.tokb = o; o += static_cast<unsigned>(M) * ROWSB * 4;
        L.stats = o; o += PPM * 2 * ROWSM * 4;
        L.trash = o; o += 16;
        L.total = o;
        return L;
    }
    static __host__ bool fits(int Np, int B, int M, size_t lds_limit) {
        return layout(Np, B, M).total <= lds_limit && (Np + pad_rows(B)) * CH <= NI * NT && M * ROWSB <= NT && (Np + ROWSB) * B < 65536;
    }

    // What a thread loads of the next head while the current one computes: chunk c = tid + i * NT of each
    // input tile (row c / CH, 16-byte piece c % CH), and the mask element of one token.
    struct Pre {
        u32x4 q[NI], k[NI], v[NI];
        // mask element of the thread's token, as loaded; one register per element width: a single one written by
        // loads of different widths is merged with copies, and a copy waits for the load
        unsigned mk8, mk16, mk32;
        u32x2 mk64;
    };
    struct Ctx {
        char* smem;
        Layout L;
        int tid, wave, lane, r, q;
        unsigned qst, kst, vst, ost, mst;
        float scale2;   // sm_scale * log2(e)
        unsigned BP;    // bytes from a block's first row to the next block's
        // row j of block m of the tile at byte offset `tile`
        __device__ __forceinline__ T* row(unsigned tile, int m, int j) const { return reinterpret_cast<T*>(smem + tile + static_cast<unsigned>(m) * BP + static_cast<unsigned>(j) * RB); }
        __device__ __forceinline__ T* at(unsigned off) const { return reinterpret_cast<T*>(smem + off); }
        __device__ __forceinline__ float* fat(unsigned off) const { return reinterpret_cast<float*>(smem + off); }
    };
    struct Head {
        rsrc_t q, k, v, mask, out;
    };
    // (re-read from the kernel arguments through an offset the compiler cannot see through: the
    // descriptions are only needed at a head boundary and would otherwise be kept - and spilled - in
    // scalar registers across all rounds)
    static __device__ __forceinline__ const Problem& reread(const Problem& P) {
        int zero = 0;
        asm volatile("" : "+s"(zero));
        return *reinterpret_cast<const Problem*>(reinterpret_cast<const char*>(&P) + zero);
    }
    static __device__ __forceinline__ Head head_of(const Problem& P0, const Ctx& c, int head) {
        const Problem& P = reread(P0);
        Head hd;
        const int e = static_cast<unsigned>(head) / static_cast<unsigned>(P.H), h = static_cast<unsigned>(head) % static_cast<unsigned>(P.H);
        const unsigned n1 = static_cast<unsigned>(P.N - 1), db = static_cast<unsigned>(P.D) * sizeof(T);
        hd.q = make_rsrc(P.q + (e * P.qs[0] + h * P.qs[1]) * static_cast<long long>(sizeof(T)), n1 * c.qst + db);
        hd.k = make_rsrc(P.k + (e * P.ks[0] + h * P.ks[1]) * static_cast<long long>(sizeof(T)), n1 * c.kst + db);
        hd.v = make_rsrc(P.v + (e * P.vs[0] + h * P.vs[1]) * static_cast<long long>(sizeof(T)), n1 * c.vst + db);
        hd.out = make_rsrc(P.out + (e * P.os[0] + h * P.os[1]) * static_cast<long long>(sizeof(T)), n1 * c.ost + db);
        hd.mask = make_rsrc(P.mask ? P.mask + ((e * P.ms[0]) << P.mask_shift) : nullptr, P.mask ? n1 * c.mst + (1u << P.mask_shift) : 0u);
        return hd;
    }

    // The loads of the next head: Q and the mask, K, V.  Their offsets are recomputed every time: a few dozen
    // instructions per head, against registers that would be held through every round.
    // (live = false: nothing is fetched - every chunk reads as zeros - but the registers are written all the same)
    static __device__ __forceinline__ void chunk_offsets(const Problem& P, const Ctx& c, unsigned st, unsigned (&off)[NI], bool live = true) {
        const int Np = live ? P.M * P.B : 0;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int cc = c.tid + i * NT, p = cc / CH, ch = cc % CH;
            const int t = p - P.pad_off;
            const bool ok = p < Np && static_cast<unsigned>(t) < static_cast<unsigned>(P.N) && ch * 8 < P.D;
            off[i] = ok ? static_cast<unsigned>(t) * st + ch * 16 : kOob;
        }
    }
    // POL: the cache policy of the row loads (compile time: a run-time choice between two runs of loads into the same
    // registers measured 1.02 - 1.18 of the time - the merged registers cost the prefetch its head start).  The four-tile
    // kernel reads every input exactly once and streams them (kPolStream), which leaves the L2 to the rows other compute
    // units are waiting for: 0.91 - 0.98 for 192 heads and more of 224 .. 256 tokens (the ViT shape at N = 256: 34.7 -> 33.3 us),
    // 1.02 - 1.04 for 64 .. 128 such heads with more than one step, +-1 % elsewhere.  The two-tile kernel reads Q and K
    // again later and keeps the ordinary policy (streamed: the ViT shape 28.2 -> 29.8 us).
    template <int POL = 0>
    static __device__ __forceinline__ void issue_q(const Problem& P, const Ctx& c, const Head& hd, Pre& pre, bool live = true) {
        if (P.mask != nullptr) {   // uniform; first: whoever looks at it waits for nothing issued behind it
            // the thread's entry of tokb: block tid / ROWSB, row tid % ROWSB
            const int m = c.tid / ROWSB, i = c.tid % ROWSB, t = m * P.B + i - P.pad_off;
            const unsigned moff = (m < P.M && i < P.B && static_cast<unsigned>(t) < static_cast<unsigned>(P.N)) ? static_cast<unsigned>(t) * c.mst : kOob;
            if (P.mask_shift == 0) pre.mk8 = __builtin_amdgcn_raw_buffer_load_b8(hd.mask, moff, 0, 0);   // uniform, all four
            if (P.mask_shift == 1) pre.mk16 = __builtin_amdgcn_raw_buffer_load_b16(hd.mask, moff, 0, 0);
            if (P.mask_shift == 2) pre.mk32 = __builtin_amdgcn_raw_buffer_load_b32(hd.mask, moff, 0, 0);
            if (P.mask_shift == 3) pre.mk64 = __builtin_amdgcn_raw_buffer_load_b64(hd.mask, moff, 0, 0);
        }
        unsigned off[NI];
        chunk_offsets(P, c, c.qst, off, live);
#pragma unroll
        for (int i = 0; i < NI; ++i) pre.q[i] = bload16<POL>(hd.q, off[i]);
    }
    template <int POL = 0>
    static __device__ __forceinline__ void issue_k(const Problem& P, const Ctx& c, const Head& hd, Pre& pre) {
        unsigned off[NI];
        chunk_offsets(P, c, c.kst, off);
#pragma unroll
        for (int i = 0; i < NI; ++i) pre.k[i] = bload16<POL>(hd.k, off[i]);
    }
    template <int POL = 0>
    static __device__ __forceinline__ void issue_v(const Problem& P, const Ctx& c, const Head& hd, Pre& pre) {
        unsigned off[NI];
        chunk_offsets(P, c, c.vst, off);
#pragma unroll
        for (int i = 0; i < NI; ++i) pre.v[i] = bload16<POL>(hd.v, off[i]);
    }
    // write a thread's chunks to the tile at byte offset `tile` (chunks beyond the tile go to the row nobody reads)
    static __device__ __forceinline__ void commit_tile(const Problem& P, const Ctx& c, unsigned tile, const u32x4 (&val)[NI]) {
        const int rows = P.M * P.B + pad_rows(P.B);
        const unsigned recip = (65536u + static_cast<unsigned>(P.B) - 1u) / static_cast<unsigned>(P.B);   // p / B == p * recip >> 16 for the few hundred rows of a tile
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int cc = c.tid + i * NT, p = cc / CH, ch = cc % CH;
            const unsigned pm = (static_cast<unsigned>(p) * recip) >> 16;   // block of row p
            const unsigned at = p < rows ? tile + static_cast<unsigned>(p) * RB + pm * kSkew + ch * 16 : c.L.TR + ch * 16;
            *reinterpret_cast<u32x4*>(c.smem + at) = val[i];
        }
    }
    static __device__ __forceinline__ void commit_tokb(const Problem& P, const Ctx& c, const Pre& pre) {
        const int m = c.tid / ROWSB, i = c.tid % ROWSB, t = m * P.B + i - P.pad_off;
        bool keep = m < P.M && i < P.B && static_cast<unsigned>(t) < static_cast<unsigned>(P.N);
        if (P.mask != nullptr) {   // uniform
            const unsigned lo = P.mask_shift == 0 ? pre.mk8 : P.mask_shift == 1 ? pre.mk16 : P.mask_shift == 2 ? pre.mk32 : pre.mk64[0];
            keep = keep && mask_nonzero(P, lo, P.mask_shift == 3 ? pre.mk64[1] : 0u);
        }
        if (m < P.M) c.fat(c.L.tokb)[c.tid] = keep ? 0.f : kNegBig;
    }

    // lane's 4*DT consecutive elements (columns 4*DT*q ..: chunk_col's RUN form, which the R and L rounds use) of an LDS row
    static __device__ __forceinline__ void lds_store_row(T* row, const f32x4 (&O)[DT], int q) {
        T* dst = row + 4 * DT * q;
        if (DT % 2 == 0) {
#pragma unroll
            for (int p = 0; p < DT / 2; ++p) {
                V4 a = {from_f<T>(O[2 * p][0]), from_f<T>(O[2 * p][1]), from_f<T>(O[2 * p][2]), from_f<T>(O[2 * p][3])};
                V4 b = {from_f<T>(O[2 * p + 1][0]), from_f<T>(O[2 * p + 1][1]), from_f<T>(O[2 * p + 1][2]), from_f<T>(O[2 * p + 1][3])};
                const u32x2 lo = __builtin_bit_cast(u32x2, a), hi = __builtin_bit_cast(u32x2, b);
                *reinterpret_cast<u32x4*>(dst + 8 * p) = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
        } else {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                V4 a = {from_f<T>(O[dt][0]), from_f<T>(O[dt][1]), from_f<T>(O[dt][2]), from_f<T>(O[dt][3])};
                *reinterpret_cast<u32x2*>(dst + 4 * dt) = __builtin_bit_cast(u32x2, a);
            }
        }
    }
    // sm_scale * round(O), rounded again on its way into the row (ma_torch.py:21): O holds the product in
    // fp32.  For f16 with a scale that is an f16 value itself (1 / sqrt(D) is for D = 4^n) both roundings
    // and the multiplication run two values per instruction: the product of two f16 values rounded to f16
    // is what the fp32 multiplication followed by the rounding gives.
    // (PACK = false leaves the two-value form out: its second code path costs the two-tile kernel registers it does not have)
    template <bool PACK = true>
    static __device__ __forceinline__ void lds_store_row_scaled(T* row, const f32x4 (&O)[DT], int q, float sm_scale, bool scale_is_f16) {
        if constexpr (PACK && std::is_same<T, f16>::value && DT % 2 == 0) {
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
            if (scale_is_f16) {   // uniform
                const _Float16 s = static_cast<_Float16>(sm_scale);
                T* dst = row + 4 * DT * q;
                const h2 s2 = {s, s};
#pragma unroll
                for (int p = 0; p < DT / 2; ++p) {
                    unsigned w[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        h2 x = {static_cast<_Float16>(O[2 * p + i / 2][2 * (i % 2)]), static_cast<_Float16>(O[2 * p + i / 2][2 * (i % 2) + 1])};
                        x *= s2;
                        w[i] = __builtin_bit_cast(unsigned, x);
                    }
                    *reinterpret_cast<u32x4*>(dst + 8 * p) = u32x4{w[0], w[1], w[2], w[3]};
                }
                return;
            }
        }
        f32x4 S[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int v = 0; v < 4; ++v) S[dt][v] = sm_scale * round_to<T>(O[dt][v]);
        lds_store_row(row, S, q);
    }
    // transposed A operand from arbitrary LDS rows: p_lo / p_hi point at this lane's source row
    // (k slot e resp. 4 + e of its 16-lane group) at the lane's column of the output tile
    static __device__ __forceinline__ V8 tr8(const T* p_lo, const T* p_hi) {
        typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
        typedef short i16x8 __attribute__((ext_vector_type(8)));
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_lo));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_hi));
        const i16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(V8, v);
    }
    // GEMM2 with the rows of the transposed operand `pitch` bytes apart (RB: the rows of a block; the block pitch:
    // the rows of a position): O[dt][v] = sum_x row(x)[chunk_col(q, dt) + v] * P[x][lane column], x < rows
    // (rows beyond read the row of zeros; R rounds pass rows = 16 * NT: the zero rows behind the tiles cover their tails)
    template <int NT_, bool RUN>
    static __device__ __forceinline__ void gemm2_rows(f32x4 (&O)[DT], const Ctx& c, const T* tile0, unsigned pitch, int rows,
                                                      const V8 (&pb)[(NT_ + 1) / 2]) {
        const int e4 = c.r >> 2, c4 = c.r & 3;
        const T* zr = c.at(c.L.ZR);
        const T* lo[(NT_ + 1) / 2];
        const T* hi[(NT_ + 1) / 2];
#pragma unroll
        for (int g = 0; g < (NT_ + 1) / 2; ++g) {   // k slot s <-> row 32g + 16(s/4) + 4q + s%4
            const int x = 32 * g + 4 * c.q + e4;
            lo[g] = x < rows ? reinterpret_cast<const T*>(reinterpret_cast<const char*>(tile0) + x * pitch) : zr;
            hi[g] = (2 * g + 1 < NT_ && x + 16 < rows) ? reinterpret_cast<const T*>(reinterpret_cast<const char*>(tile0) + (x + 16) * pitch) : zr;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            const int col = chunk_col<DT, RUN>(c4, dt);
#pragma unroll
            for (int g = 0; g < (NT_ + 1) / 2; ++g) acc = Ops<T>::mma(tr8(lo[g] + col, hi[g] + col), pb[g], acc);
            O[dt] = acc;
        }
    }

    // ---------------------------------------------------------------- the three kinds of rounds
    // R round: al_cl_ref / al_y_cl_ref (ma/ma_torch.py:10-23, :38-52).  Problem m: keys and values are the rows of
    // block m, queries the rows aR(m, .) - Q's rows of the block in the first step.
    // TWO: the two-tile form (ma_resident_head2.h).  The first step's query rows are in S as well (S starts out as
    // Q), and V is not in LDS: the waves of the problem load block m's V rows at the top of the round and write them
    // over the block's K rows once every wave of the problem has had its last look at those.
    static constexpr int NV = (ROWSB * CH + 64 * WPB - 1) / (64 * WPB);   // 16-byte chunks of a block's V rows per lane of the problem
    template <bool TWO = false>
    static __device__ __forceinline__ void round_r(const Problem& P, const Ctx& c, int rnd, bool first, bool with_v, bool scale_is_f16,
                                                   const Head* hd = nullptr) {
        const int B = P.B, M = P.M;
        const int grp = c.wave / WPB, wig = c.wave % WPB;
        const int m = rnd * PPB + grp;
        const bool active = m < M;   // uniform per wave
        const int r = c.r, q = c.q;
        const int j = 16 * wig + r;
        const bool ok = j < B;
        V8 pb[(NTB + 1) / 2];
        u32x4 vv[TWO ? NV : 1];
        if constexpr (TWO) {
            if (with_v && active) {   // uniform per wave
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int cc = wig * 64 + c.lane + i * 64 * WPB, row = cc / CH, ch = cc % CH;
                    const int t = m * B + row - P.pad_off;
                    const bool in = row < B && static_cast<unsigned>(t) < static_cast<unsigned>(P.N) && ch * 8 < P.D;
                    vv[i] = bload16<false>(hd->v, in ? static_cast<unsigned>(t) * c.vst + ch * 16 : kOob);
                }
            }
        }
        if (active) {
            const T* Kt = c.row(c.L.K, m, 0);
            const T* xrow = ok ? c.row((first && !TWO) ? c.L.Q : c.L.S, m, j) : c.at(c.L.ZR);
            V8 xb[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xb[ks] = lds_row8<T>(xrow + 32 * ks + 8 * q);
            const float crv = c.fat(c.L.cR)[ok ? m * B + j : 0];
            const float cr = (ok && !first) ? crv : 1.0f;
            const float cj = c.scale2 * rcp(cr + P.eps);   // logits in log2 units
            const float* kbias = c.fat(c.L.tokb) + m * ROWSB;
            f32x4 C[NTB];
#pragma unroll
            for (int wt = 0; wt < NTB; ++wt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(Kt + (16 * wt + r) * LD + 32 * ks + 8 * q), xb[ks], acc);
                const f32x4 kb = *reinterpret_cast<const f32x4*>(kbias + 16 * wt + 4 * q);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[v] = fmaf(round_to<T>(acc[v]), cj, kb[v]);
                C[wt] = acc;
            }
            float mx = C[0][0];
#pragma unroll
            for (int wt = 0; wt < NTB; ++wt)
#pragma unroll
                for (int v = 0; v < 4; ++v) mx = fmaxf(mx, C[wt][v]);
            mx = fmaxf(quad_rows_max(mx), P.eps * kLog2e);   // clamped row maximum (ma_torch.py:15)
            float sum = 0.f, ent = 0.f;
#pragma unroll
            for (int wt = 0; wt < NTB; ++wt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float d = C[wt][v] - mx;
                    const float p = __builtin_amdgcn_exp2f(d);
                    sum += p;
                    ent = fmaf(p, d, ent);
                    C[wt][v] = p;
                }
            sum = quad_rows_sum(sum);
            ent = quad_rows_sum(ent);
            const float den = sum + P.eps, inv = rcp(den);
#pragma unroll
            for (int wt = 0; wt < NTB; ++wt)
#pragma unroll
                for (int v = 0; v < 4; ++v) C[wt][v] *= inv;
            // cL = sum_i r log r with r = p / den (ma_torch.py:20), kept as the softmax bias -log2(e) * cL of the
            // L and Z problems of position j; the four lanes of a row all hold it
            *(ok ? c.fat(c.L.cb) + j * ROWSM + m : c.fat(c.L.trash)) = -kLog2e * (kLn2 * (ent * inv - log2_normal(den) * (sum * inv)));   // (the same roundings as where cL itself is kept)
            pack_p<T, NTB>(pb, C);
            f32x4 O[DT];
            gemm2_rows<NTB, true>(O, c, Kt, RB, ROWSB, pb);
            lds_store_row_scaled<!TWO>(ok ? c.row(c.L.S, m, j) : c.at(c.L.TR), O, q, P.sm_scale, scale_is_f16);
        }
        if constexpr (TWO) {
            if (with_v) {   // uniform
                problem_sync<WPB>();   // every wave of the problem has read the block's K rows for the last time
                if (active) {
#pragma unroll
                    for (int i = 0; i < NV; ++i) {
                        const int cc = wig * 64 + c.lane + i * 64 * WPB, row = cc / CH, ch = cc % CH;
                        // (rows behind a block that is no multiple of 16 rows long belong to the next block: they stay as
                        // they are - their probabilities are zero)
                        *reinterpret_cast<u32x4*>(row < B ? reinterpret_cast<char*>(c.row(c.L.K, m, row)) + ch * 16 : c.smem + c.L.TR + ch * 16) = vv[i];
                    }
                }
                problem_sync<WPB>();
            }
        }
        if (with_v) {   // uniform
            f32x4 O[DT];
            if (active) gemm2_rows<NTB, true>(O, c, c.row(c.L.V, m, 0), RB, ROWSB, pb);
            // Y(j, m) goes where V's row j of block m was: every wave of the problem has read the block's V rows
            problem_sync<WPB>();
            if (active) lds_store_row(ok ? c.row(c.L.V, m, j) : c.at(c.L.TR), O, q);
        }
    }

    // L round: ar_cr_ref (ma/ma_torch.py:26-35).  Problem j: the rows at position j of every block.  Two passes
    // over the logits, as in LProb: pass 1 with a wave per strip of query blocks l (accumulator rows = key
    // blocks k) for the row statistics, pass 2 with a wave per strip of key blocks k (rows = query blocks l),
    // whose probabilities are the B operand of aR[k] = sum_l L[l, k] Q[l] as they stand.
    static __device__ __forceinline__ void round_l(const Problem& P, const Ctx& c, int rnd) {
        const int B = P.B, M = P.M;
        const int grp = c.wave / WPM, wig = c.wave % WPM;
        const int j = rnd * PPM + grp;
        const bool active = j < B;   // uniform per wave
        const int r = c.r, q = c.q;
        const int lk = 16 * wig + r;   // pass 1: this lane's query block l; pass 2: its key block k
        const T* zr = c.at(c.L.ZR);
        const T* Qj = c.row(c.L.Q, 0, j);   // row l of the problem's Q^T tile: l block pitches behind
        const T* Sj = c.row(c.L.S, 0, j);   // aL(j, k): k block pitches behind, and aR(k, j) goes there
        const auto blk = [&](const T* base, int x) { return reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + static_cast<unsigned>(x) * c.BP); };
        const float* cb = c.fat(c.L.cb) + j * ROWSM;
        float* mxs = c.fat(c.L.stats) + grp * 2 * ROWSM;
        float* invs = mxs + ROWSM;
        if (active) {
            const T* xrow = lk < M ? blk(Qj, lk) : zr;
            V8 xq[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xq[ks] = lds_row8<T>(xrow + 32 * ks + 8 * q);
            f32x4 C[NTM];
            float mx = kNegBig;
#pragma unroll
            for (int kt = 0; kt < NTM; ++kt) {
                const int k = 16 * kt + r;
                const T* arow = k < M ? blk(Sj, k) : zr;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(arow + 32 * ks + 8 * q), xq[ks], acc);
                const f32x4 b = *reinterpret_cast<const f32x4*>(cb + 16 * kt + 4 * q);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    acc[v] = fmaf(round_to<T>(acc[v]), kLog2e, b[v]);
                    mx = fmaxf(mx, acc[v]);
                }
                C[kt] = acc;
            }
            mx = quad_rows_max(mx);
            float sum = 0.f;
#pragma unroll
            for (int kt = 0; kt < NTM; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v) sum += __builtin_amdgcn_exp2f(C[kt][v] - mx);
            sum = quad_rows_sum(sum);
            // padded / masked query tokens are zeroed after the softmax (ma_torch.py:30); the four lanes of a row all hold its statistics
            const float tb = c.fat(c.L.tokb)[lk < M ? lk * ROWSB + j : 0];
            mxs[lk] = mx;
            invs[lk] = (lk < M && tb == 0.f) ? rcp(sum) : 0.f;
        }
        problem_sync<WPM>();
        if (active) {
            const bool kv = lk < M;
            T* krow = kv ? const_cast<T*>(blk(Sj, lk)) : c.at(c.L.TR);
            V8 xk[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xk[ks] = lds_row8<T>((kv ? krow : zr) + 32 * ks + 8 * q);
            const float cbk = cb[lk];
            f32x4 C[NTM];
            float crs = 0.f;
#pragma unroll
            for (int lt = 0; lt < NTM; ++lt) {
                const int l = 16 * lt + r;
                const T* qrow = l < M ? blk(Qj, l) : zr;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(qrow + 32 * ks + 8 * q), xk[ks], acc);
                const f32x4 mx4 = *reinterpret_cast<const f32x4*>(mxs + 16 * lt + 4 * q);
                const f32x4 inv4 = *reinterpret_cast<const f32x4*>(invs + 16 * lt + 4 * q);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float u = fmaf(round_to<T>(acc[v]), kLog2e, cbk);
                    const float lv = __builtin_amdgcn_exp2f(u - mx4[v]) * inv4[v];
                    crs += lv;
                    acc[v] = lv;
                }
                C[lt] = acc;
            }
            crs = quad_rows_sum(crs);
            // aR[k, :] = sum_l round(L[l, k]) Q[l, :]
            V8 pb[(NTM + 1) / 2];
            pack_p<T, NTM>(pb, C);
            f32x4 O[DT];
            gemm2_rows<NTM, true>(O, c, Qj, c.BP, M, pb);
            lds_store_row(krow, O, q);
            *(kv ? c.fat(c.L.cR) + lk * B + j : c.fat(c.L.trash)) = crs;
        }
        // (the next round's first pass overwrites the statistics a slower wave of this problem may still be reading)
        if (WPM > 1) __syncthreads();
    }

    // Z round: z_ref (ma/ma_torch.py:55-62) and the final slice (:106-108)
    // the query row (l, j) of this lane in Z round rnd, straight from memory (two-tile form: Q is not in LDS then)
    static __device__ __forceinline__ void load_zq(const Problem& P, const Ctx& c, const Head& hd, int rnd, V8 (&xq)[KS]) {
        const int grp = c.wave / WPM, wig = c.wave % WPM;
        const int j = rnd * PPM + grp, l = 16 * wig + c.r;
        const int t = l * P.B + j - P.pad_off;
        const bool in = j < P.B && l < P.M && static_cast<unsigned>(t) < static_cast<unsigned>(P.N);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int col = 32 * ks + 8 * c.q;
            xq[ks] = __builtin_bit_cast(V8, bload16<false>(hd.q, (in && col < P.D) ? static_cast<unsigned>(t) * c.qst + col * 2 : kOob));
        }
    }
    template <bool TWO = false>
    static __device__ __forceinline__ void round_z(const Problem& P, const Ctx& c, const Head& hd, int rnd, const V8* zq = nullptr) {
        const int B = P.B, M = P.M;
        const int grp = c.wave / WPM, wig = c.wave % WPM;
        const int j = rnd * PPM + grp;
        if (j >= B) return;   // uniform per wave; no barrier inside a Z round
        const int r = c.r, q = c.q;
        const int l = 16 * wig + r;
        const T* zr = c.at(c.L.ZR);
        const T* Qj = c.row(c.L.Q, 0, j);
        const T* Sj = c.row(c.L.S, 0, j);
        const auto blk = [&](const T* base, int x) { return reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + static_cast<unsigned>(x) * c.BP); };
        const float* cb = c.fat(c.L.cb) + j * ROWSM;
        const T* xrow = l < M ? blk(Qj, l) : zr;
        V8 xq[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if constexpr (TWO) xq[ks] = zq[ks];
            else xq[ks] = lds_row8<T>(xrow + 32 * ks + 8 * q);
        }
        f32x4 C[NTM];
#pragma unroll
        for (int wt = 0; wt < NTM; ++wt) {
            const int k = 16 * wt + r;
            const T* arow = k < M ? blk(Sj, k) : zr;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(arow + 32 * ks + 8 * q), xq[ks], acc);
            const f32x4 b = *reinterpret_cast<const f32x4*>(cb + 16 * wt + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = fmaf(round_to<T>(acc[v]), kLog2e, b[v]);
            C[wt] = acc;
        }
        float mx = C[0][0];
#pragma unroll
        for (int wt = 0; wt < NTM; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) mx = fmaxf(mx, C[wt][v]);
        mx = quad_rows_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int wt = 0; wt < NTM; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float p = __builtin_amdgcn_exp2f(C[wt][v] - mx);
                sum += p;
                C[wt][v] = p;
            }
        const float inv = rcp(quad_rows_sum(sum));
#pragma unroll
        for (int wt = 0; wt < NTM; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) C[wt][v] *= inv;
        V8 pb[(NTM + 1) / 2];
        pack_p<T, NTM>(pb, C);
        f32x4 O[DT];
        gemm2_rows<NTM, false>(O, c, c.row(c.L.V, 0, j), c.BP, M, pb);   // Y(j, k) sits in V's row j of block k
        const int t = l * B + j - P.pad_off;
        store_row<T, DT>(hd.out, l < M ? tok_off(t, P.N, c.ost) : kOob, P.D, O, q, false);   // padded query rows are dropped
    }
};

template <class T, int DT, int NTB, int NTM, int W, int NI, int WGS = 1>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(W * WGS / 4))) void resident_head_mfma(Problem P) {
    using HR = HeadRes<T, DT, NTB, NTM, W, NI>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int Np = P.M * P.B;
    typename HR::Ctx c;
    c.smem = smem;
    c.L = HR::layout(Np, P.B, P.M);
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
    // once per launch: zeros in the tiles (the gaps between the blocks' rows are never written again, and a
    // 16-row strip of a shorter block reads across them), in the row of zeros; the softmax bias of key
    // blocks that do not exist
    // (with blocks of exactly 16, 32 or 64 rows no strip reaches across a gap or into the columns behind a row's last, and
    // with a head dim that fills its tile columns every column a product reads is written first: only the row of zeros then)
    const bool fill_tiles = HR::ROWSB != P.B || (DT & 1) != 0;   // uniform
    for (unsigned i = (fill_tiles ? 0u : c.L.ZR) + c.tid * 16u; i < c.L.TR; i += HR::NT * 16u) *reinterpret_cast<u32x4*>(smem + i) = u32x4{0u, 0u, 0u, 0u};
    for (int i = c.tid; i < P.B * HR::ROWSM; i += HR::NT) c.fat(c.L.cb)[i] = kNegBig;
    // (the state rows are written 16*DT columns wide but read as GEMM operands over all 32*KS columns: for head
    // dims of 65..80 the columns in between are never written and keep those zeros)
    __syncthreads();   // no wave writes a tile row before every wave's zeros are in

    const int heads = P.E * P.H, stride = static_cast<int>(gridDim.x);
    int head = static_cast<int>(blockIdx.x);
    if (head >= heads) return;
    typename HR::Pre pre = {};
    typename HR::Head hd = HR::head_of(P, c, head);
    HR::template issue_q<kPolStream>(P, c, hd, pre);
    HR::template issue_k<kPolStream>(P, c, hd, pre);
    HR::template issue_v<kPolStream>(P, c, hd, pre);
    HR::commit_tile(P, c, c.L.Q, pre.q);
    HR::commit_tile(P, c, c.L.K, pre.k);
    HR::commit_tile(P, c, c.L.V, pre.v);
    HR::commit_tokb(P, c, pre);
    __syncthreads();
    const int nr = (P.M + HR::PPB - 1) / HR::PPB, nl = (P.B + HR::PPM - 1) / HR::PPM;
    const int nph = 2 * P.T;   // phases of a head: R [L R ...] Z
    for (;;) {
        const int next = head + stride;
        const bool more = next < heads;
        typename HR::Head hn = hd;
        // The next head's rows fly while this one computes.  All of them are started here, at ONE place outside the
        // loops over phases and rounds: loads started at several places of a loop are carried from iteration to
        // iteration through register copies, and a copy of a register waits for the load that is still filling it.
        // (While they arrive - 96 KB into the registers of a compute unit - the first phase runs at half its speed;
        // starting them in front of a later phase, or a tile per phase, measured 1 - 2 us slower per forward.)
        if (more) {
            hn = HR::head_of(P, c, next);
            HR::template issue_q<kPolStream>(P, c, hn, pre);
            HR::template issue_k<kPolStream>(P, c, hn, pre);
            HR::template issue_v<kPolStream>(P, c, hn, pre);
        }
        for (int ph = 0; ph < nph - 1; ++ph) {
            if (ph & 1) {
                for (int rnd = 0; rnd < nl; ++rnd) HR::round_l(P, c, rnd);
            } else {
                for (int rnd = 0; rnd < nr; ++rnd) HR::round_r(P, c, rnd, ph == 0, ph == nph - 2, scale_is_f16);
            }
            __syncthreads();   // the next phase reads what this one wrote, transposed
        }
        // K has had its last reader (the barrier behind the last R phase): the next head's moves in while the Z problems run
        if (more) HR::commit_tile(P, c, c.L.K, pre.k);
        for (int rnd = 0; rnd < nl; ++rnd) HR::round_z(P, c, hd, rnd);
        if (!more) break;
        __syncthreads();   // everybody is done with this head's rows
        HR::commit_tile(P, c, c.L.Q, pre.q);
        HR::commit_tile(P, c, c.L.V, pre.v);
        HR::commit_tokb(P, c, pre);
        __syncthreads();
        head = next;
        hd = hn;
    }
}

}  // namespace mfma
}  // namespace ma
