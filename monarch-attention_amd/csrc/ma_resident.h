// Resident forward: one workgroup runs a whole head - all T alternating steps,
// the product with V and the output stage - with the per-head state (aL, aR, Y,
// cL, cR of monarch_attention_torch, ma/ma_torch.py:88-104) held in LDS from the
// first step to the last.  Nothing but Q, K, V is read from memory and nothing
// but the output is written: the state never leaves the compute unit.
//
// It applies when the state fits: two or three Np x D tiles (aL, aR, Y) plus the
// operand staging of the problems in flight within the 160 KB of LDS, i.e. heads
// of up to ~256 padded tokens at D = 64, and blocks / block counts of at most 64.
// Heads of up to ~512 tokens run with ONE tile (kOneTile): aL and aR share it in
// place - the R problem of block m reads the rows aR(m, .) and writes aL(., m)
// over them, the L problem of position j reads aL(j, .) and writes aR(., j) over
// those - and Y, which is written once and read once, goes through the caller's
// workspace (the workgroup that wrote a head's Y is the one that reads it back).
//
// The head is processed as a sequence of ROUNDS; a round runs up to PPW block
// problems of one phase concurrently on the workgroup's W waves (R phase: key
// blocks m, L / Z phase: positions j).  Every global load a round needs - the K
// and V tiles of its blocks, the strided Q rows of its positions, the mask bytes
// - depends only on the inputs, never on the state, so the loads of round i+1
// are issued into registers BEFORE round i is computed and are committed to LDS
// when round i is done: memory latency is covered by the previous round's math,
// also across phase and head boundaries.  A round itself contains no wait on
// memory at all (its operands are in LDS or in prefetched registers).
//
// State layout in LDS (row pitch LD, like the operand tiles):
//   SA  aL rows (j, m) -> j*M + m      read as the "aL[j]" tile of the L / Z problems
//   SX  aR rows (m, j) -> m*B + j      read as the "aR[m]" rows of the R problems
//   SY  Y  rows (j, m) -> j*M + m      read (transposed) by the Z problems; in aR's place when
//       the last R phase is a single round (see y_on_x), else a tile of its own
//   kOneTile: SA = SX, aL(j, m) and aR(m, j) both live in row m*B + j; no SY
//   cLs[j*M + m], cRs[m*B + j] (fp32), ZR: one row of zeros that stands in for
//   rows beyond the tile tails (k >= M, j >= B).
#pragma once

#include "ma_mfma.h"

namespace ma {
namespace mfma {

template <class T, int DT, int NTB, int NTM, int W, bool ONE = false>
struct Resident {
    using G = Geom<DT>;
    using V8 = typename Ops<T>::v8;
    using V4 = typename Ops<T>::v4;
    static_assert(NTB <= 4 && NTM <= 4, "one strip per wave: blocks and block counts of at most 64");
    static constexpr int LD = G::LD, KS = G::KS;
    static constexpr int WPB = NTB, PPB = W / WPB;   // waves per R problem, R problems per round
    static constexpr int WPM = NTM, PPM = W / WPM;   // same for the L / Z problems
    static constexpr int ROWSB = 16 * NTB, ROWSM = 16 * NTM, ROWS2M = 32 * ((NTM + 1) / 2), LDP = ROWS2M + 8;
    // staging of one problem slot
    static constexpr size_t kStageR = 2 * ROWSB * LD * sizeof(T) + ROWSB * sizeof(float);
    static constexpr size_t kStageL = (ROWSM * LD + ROWSM * LDP) * sizeof(T) + (1 + WPM) * ROWSM * sizeof(float);
    static constexpr size_t kSlotR = (kStageR + 15) / 16 * 16, kSlotL = (kStageL + 15) / 16 * 16;

    // Y is written by the last R phase, which is also the last reader of aR.  When that phase is
    // a single round (all its block problems run at once) its waves read their aR rows first, meet
    // at a barrier, and only then write Y - so Y can take aR's place and the state is two tiles.
    // It costs that barrier, so it is only used where three tiles do not fit (the launcher decides).
    static __host__ __device__ bool y_on_x_possible(int M) { return M <= PPB; }
    // how the state is kept: three tiles, two (Y in aR's place), or one (aL and aR in place, Y through memory)
    enum { kThreeTiles = 0, kYOnX = 1, kOneTile = 2 };
    static __host__ __device__ int tiles_of(int mode) { return mode == kOneTile ? 1 : mode == kYOnX ? 2 : 3; }
    static __host__ __device__ size_t state_bytes(int Np, int mode) {   // SA, (SX,) (SY,) ZR, cLs, cRs
        const size_t np4 = (static_cast<size_t>(Np) + 3) / 4 * 4;
        return (tiles_of(mode) * static_cast<size_t>(Np) + 1) * LD * sizeof(T) + 2 * np4 * sizeof(float);
    }
    // staging is only needed for the problems a round can actually hold
    static __host__ __device__ size_t lds_bytes(int Np, int M, int B, int mode) {
        const size_t sr = static_cast<size_t>(M < PPB ? M : PPB) * kSlotR, sl = static_cast<size_t>(B < PPM ? B : PPM) * kSlotL;
        return state_bytes(Np, mode) + (sr > sl ? sr : sl);
    }

    // registers that carry one round's global loads from issue to execute
    // All tile copies are CNT 16-byte chunks per thread, whatever the tile's row count (the
    // threads of a problem grow with its rows), so the K tile of an R round and the Q^T tile of an
    // L round share one register array.
    static constexpr int CH = G::COLS / 8, CNT = CH / 4;
    static_assert(CH % 4 == 0, "tile rows are whole groups of four 16-byte chunks");
    struct Pre {
        u32x4 a[CNT];                              // R: K tile chunks; L: Q^T tile chunks
        u32x4 b[CNT];                              // last R: V tile chunks
        V8 xq[KS];                                 // Q rows: first R step / Z step
        float kb;                                  // key bias of staging row `tix` (R)
        unsigned qok;                              // 4 bits: query rows l0 + 4q + v are real and unmasked (L)
    };
    // start the loads of this thread's chunks of a tile of a problem with `nth` threads: rowoff(row)
    // is the row's byte offset in `src` or kOob; columns at or beyond D read as zero
    template <bool SHARED = false, class RowOff>
    static __device__ __forceinline__ void tile_issue(u32x4 (&val)[CNT], rsrc_t src, int D, RowOff rowoff, int tix, int nth) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * nth;
            const int row = c / CH, ch = c % CH;
            const unsigned ro = rowoff(row);
            val[i] = bload16<SHARED>(src, (ch * 8 < D) ? ro + ch * 16 : kOob);
        }
    }
    static __device__ __forceinline__ void tile_commit(T* tile, const u32x4 (&val)[CNT], int tix, int nth) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = tix + i * nth;
            *reinterpret_cast<u32x4*>(tile + (c / CH) * LD + (c % CH) * 8) = val[i];
        }
    }

    struct Round {
        int head;   // E*H fits int32 (validated by the host)
        int p, rnd;
    };

    struct Ctx {
        T *SA, *SX, *SY, *ZR;
        float *cLs, *cRs;
        char* stage;
        int wave, lane, r, q;
        bool y_on_x;   // Y shares the LDS of aR
        // row of aL(j, m) (m < M, j < B); ONE (kOneTile): SA == SX, aL(j, m) and aR(m, j) share row m*B + j, Y is in the workspace
        __device__ __forceinline__ T* al_row(int j, int m, int B, int M) const { return SA + (ONE ? m * B + j : j * M + m) * LD; }
    };
    // the head's Y rows (j, m) -> j*M + m in the workspace (kOneTile)
    static __device__ __forceinline__ rsrc_t y_slice(const Problem& P, int head) {
        const long long bytes = static_cast<long long>(P.M) * P.B * P.D * static_cast<long long>(sizeof(T));
        return make_rsrc(P.Y + head * bytes, static_cast<unsigned>(bytes));
    }
    // start the loads of the Y tile of position j of a Z problem (kOneTile)
    static __device__ __forceinline__ void y_issue(const Problem& P, int head, u32x4 (&val)[CNT], int j, int tix) {
        const unsigned db = static_cast<unsigned>(P.D) * sizeof(T);
        const int M = P.M;
        tile_issue<true>(val, y_slice(P, head), P.D, [&](int k) { return k < M ? static_cast<unsigned>(j * M + k) * db : kOob; }, tix, WPM * 64);
    }

    static __device__ __forceinline__ int rounds_of(const Problem& P, int p) {
        return (p & 1) ? (P.B + PPM - 1) / PPM : (P.M + PPB - 1) / PPB;   // p odd: L or Z (positions j), p even: R (blocks m)
    }
    static __device__ __forceinline__ bool advance(const Problem& P, Round& rd, int heads, int stride) {
        if (++rd.rnd < rounds_of(P, rd.p)) return true;
        rd.rnd = 0;
        if (++rd.p < 2 * P.T) return true;
        rd.p = 0;
        rd.head += stride;
        return rd.head < heads;
    }

    // lane's 4*DT consecutive elements (columns 4*DT*q ..: chunk_col's RUN form, used throughout this kernel) of an LDS row
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

    // transposed A operand from arbitrary LDS rows: p_lo / p_hi point at this lane's source row
    // (k slot e resp. 4 + e of its 16-lane group) at column chunk_col(c, dt)
    static __device__ __forceinline__ V8 tr8(const T* p_lo, const T* p_hi) {
        typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
        typedef short i16x8 __attribute__((ext_vector_type(8)));
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_lo));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_hi));
        const i16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(V8, v);
    }

    // ---------------------------------------------------------------- issue: start the round's global loads
    static __device__ __forceinline__ void issue(const Problem& P, const Round& rd, Pre& pre, const Ctx& c) {
        const int e = rd.head / P.H, h = rd.head % P.H;
        const Slices S = make_slices<T>(P, e, h, 0);
        const int B = P.B, M = P.M, D = P.D;
        const int nph = 2 * P.T;
        if (!(rd.p & 1)) {   // R round
            const int slot = c.wave / WPB, wig = c.wave % WPB, tix = wig * 64 + c.lane;
            const int m = rd.rnd * PPB + slot;
            if (m >= M) return;
            const int t0 = m * B - P.pad_off;
            tile_issue(pre.a, S.k, D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.kst) : kOob; }, tix, WPB * 64);
            if (rd.p == nph - 2)
                tile_issue(pre.b, S.v, D, [&](int i) { return i < B ? tok_off(t0 + i, P.N, S.vst) : kOob; }, tix, WPB * 64);
            if (rd.p == 0) {
                const int j = 16 * wig + c.r;
                load_x<T, DT, false>(pre.xq, S.q, j < B ? tok_off(t0 + j, P.N, S.qst) : kOob, D, c.q);
            }
            pre.kb = (tix < B && token_ok(P, e, t0 + tix)) ? 0.f : kNegBig;
        } else {
            const int slot = c.wave / WPM, wig = c.wave % WPM, tix = wig * 64 + c.lane;
            const int j = rd.rnd * PPM + slot;
            if (j >= B) return;
            if (rd.p == nph - 1) {   // Z round: the strip's Q rows
                const int l = 16 * wig + c.r;
                load_x<T, DT, false>(pre.xq, S.q, l < M ? tok_off(l * B + j - P.pad_off, P.N, S.qst) : kOob, D, c.q);
                // Y from the workspace: complete once the last R phase has ended, i.e. for every Z round
                // but the first, whose loads would start while that phase still runs (round_z loads them itself)
                if constexpr (ONE) if (rd.rnd > 0) y_issue(P, rd.head, pre.a, j, tix);
            } else {                 // L round: the Q^T tile and the query mask of the strip's rows
                tile_issue(pre.a, S.q, D, [&](int l) { return l < M ? tok_off(l * B + j - P.pad_off, P.N, S.qst) : kOob; }, tix, WPM * 64);
                unsigned ok = 0;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int l = 16 * wig + 4 * c.q + v;
                    if (l < M && token_ok(P, e, l * B + j - P.pad_off)) ok |= 1u << v;
                }
                pre.qok = ok;
            }
        }
    }

    // End of a round.  What a round writes to the state is read in the NEXT phase, and its staging
    // is reused by the next round: the workgroup barrier is needed after the last round of a phase
    // and whenever several waves share a problem's staging; single-wave problems in the middle of a
    // phase run on (their staging accesses are ordered within the wave).
    template <int WP>
    static __device__ __forceinline__ void round_end(const Problem& P, const Round& rd) {
        if (WP > 1 || rd.rnd + 1 == rounds_of(P, rd.p)) __syncthreads();
        else __builtin_amdgcn_wave_barrier();
    }

    // ---------------------------------------------------------------- the three kinds of rounds
    // R round: al_cl_ref / al_y_cl_ref (ma/ma_torch.py:10-23, :38-52) on the LDS state
    static __device__ __forceinline__ void round_r(const Problem& P, const Round& rd, const Pre& pre, const Ctx& c) {
        const int B = P.B, M = P.M;
        const bool first = rd.p == 0, with_v = rd.p == 2 * P.T - 2;
        const int slot = c.wave / WPB, wig = c.wave % WPB, tix = wig * 64 + c.lane;
        const int m = rd.rnd * PPB + slot;
        const bool active = m < M;
        const int r = c.r, q = c.q;
        T* Kt = reinterpret_cast<T*>(c.stage + slot * kSlotR);
        T* Vt = Kt + ROWSB * LD;
        float* kbias = reinterpret_cast<float*>(Vt + ROWSB * LD);
        if (active) {
            tile_commit(Kt, pre.a, tix, WPB * 64);
            if (with_v) tile_commit(Vt, pre.b, tix, WPB * 64);
            if (tix < ROWSB) kbias[tix] = pre.kb;
        }
        problem_sync<WPB>();
        const int j = 16 * wig + r;
        const bool jv = j < B;
        V8 xb[KS];
        float cr = 1.0f;
        if (active) {
            if (first) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) xb[ks] = pre.xq[ks];
            } else {
                const T* xrow = jv ? c.SX + (m * B + j) * LD : c.ZR;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) xb[ks] = lds_row8<T>(xrow + 32 * ks + 8 * q);
                if (jv) cr = c.cRs[m * B + j];
            }
        }
        // Y takes the place of aR (see the kernel): every wave has read its aR rows before any
        // wave writes Y rows.  Uniform condition; the barrier also waits for the reads' data.
        if (c.y_on_x && with_v && !first) __syncthreads();
        if (active) {
            const float cj = (P.sm_scale * kLog2e) * rcp(cr + P.eps);
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
            const int lrow = j * M + m;
            if (jv && q == 0) c.cLs[lrow] = kLn2 * (ent * inv - log2_normal(den) * (sum * inv));
            V8 pb[(NTB + 1) / 2];
            pack_p<T, NTB>(pb, C);
            {
                f32x4 O[DT];
                gemm2<T, DT, NTB, true>(O, Kt, pb, r, q);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) O[dt][v] = P.sm_scale * round_to<T>(O[dt][v]);
                if (jv) lds_store_row(c.al_row(j, m, B, M), O, q);
            }
            if (with_v) {
                f32x4 O[DT];
                gemm2<T, DT, NTB, true>(O, Vt, pb, r, q);
                if (ONE) store_row<T, DT, true>(y_slice(P, rd.head), jv ? static_cast<unsigned>(lrow) * (static_cast<unsigned>(P.D) * sizeof(T)) : kOob, P.D, O, q);
                else if (jv) lds_store_row(c.SY + lrow * LD, O, q);
            }
        }
        // Y rows in the workspace: written (acknowledged) before the barrier that ends the phase lets the Z rounds load them
        if (ONE && with_v && rd.rnd + 1 == rounds_of(P, rd.p)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        round_end<WPB>(P, rd);
    }

    // L round: ar_cr_ref (ma/ma_torch.py:26-35) on the LDS state
    static __device__ __forceinline__ void round_l(const Problem& P, const Round& rd, const Pre& pre, const Ctx& c) {
        const int B = P.B, M = P.M;
        const int slot = c.wave / WPM, wig = c.wave % WPM, tix = wig * 64 + c.lane;
        const int j = rd.rnd * PPM + slot;
        const bool active = j < B;
        const int r = c.r, q = c.q;
        constexpr int NG = (NTM + 1) / 2;
        T* Qt = reinterpret_cast<T*>(c.stage + slot * kSlotL);
        T* PT = Qt + ROWSM * LD;
        float* cb = reinterpret_cast<float*>(PT + ROWSM * LDP);
        float* crp = cb + ROWSM;
        if (active) {
            tile_commit(Qt, pre.a, tix, WPM * 64);
            if (tix < ROWSM) cb[tix] = tix < M ? -kLog2e * c.cLs[j * M + tix] : kNegBig;
            constexpr int PH = ROWS2M > ROWSM ? ROWS2M - ROWSM : 1;   // phantom query-block columns that phase 2 reads
            if (ROWS2M > ROWSM)
                for (int i = tix; i < ROWSM * PH; i += WPM * 64) PT[(i / PH) * LDP + ROWSM + i % PH] = from_f<T>(0.f);
        }
        problem_sync<WPM>();
        if (active) {
            const int l0 = 16 * wig;
            V8 xa[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xa[ks] = lds_row8<T>(Qt + (l0 + r) * LD + 32 * ks + 8 * q);
            f32x4 C[NTM];
#pragma unroll
            for (int kt = 0; kt < NTM; ++kt) {
                const int k = 16 * kt + r;
                const T* brow = k < M ? c.al_row(j, k, B, M) : c.ZR;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(xa[ks], lds_row8<T>(brow + 32 * ks + 8 * q), acc);
                const float b = cb[k];
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[v] = fmaf(round_to<T>(acc[v]), kLog2e, b);
                C[kt] = acc;
            }
            f32x4 mx = C[0];
#pragma unroll
            for (int kt = 1; kt < NTM; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v) mx[v] = fmaxf(mx[v], C[kt][v]);
#pragma unroll
            for (int v = 0; v < 4; ++v) mx[v] = row16_max(mx[v]);
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kt = 0; kt < NTM; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float p = __builtin_amdgcn_exp2f(C[kt][v] - mx[v]);
                    sum[v] += p;
                    C[kt][v] = p;
                }
            f32x4 inv;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float s = row16_sum(sum[v]);
                inv[v] = ((pre.qok >> v) & 1u) ? rcp(s) : 0.f;   // padded / masked queries are zeroed (ma_torch.py:30)
            }
#pragma unroll
            for (int kt = 0; kt < NTM; ++kt) {
                V4 o;
                float part = 0.f;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float lv = C[kt][v] * inv[v];
                    part += lv;
                    o[v] = from_f<T>(lv);
                }
                *reinterpret_cast<u32x2*>(PT + (16 * kt + r) * LDP + l0 + 4 * q) = __builtin_bit_cast(u32x2, o);
                const float s = quad_rows_sum(part);
                if (q == 0) crp[wig * ROWSM + 16 * kt + r] = s;
            }
        }
        problem_sync<WPM>();
        if (active) {
            const int k = 16 * wig + r;   // this wave's tile of key blocks
            const bool kv = k < M;
            V8 pb[NG];
#pragma unroll
            for (int g = 0; g < NG; ++g) pb[g] = lds_row8<T>(PT + k * LDP + 32 * g + 8 * q);
            f32x4 O[DT];
            const int e4 = r >> 2, c4 = r & 3;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int g = 0; g < NG; ++g) {   // natural k-slot order: slot s <-> query block 32g + 8q + s
                    const int lo = 32 * g + 8 * q + e4, hi = lo + 4;
                    const T* p_lo = (lo < ROWSM ? Qt + lo * LD : c.ZR) + chunk_col<DT, true>(c4, dt);
                    const T* p_hi = (hi < ROWSM ? Qt + hi * LD : c.ZR) + chunk_col<DT, true>(c4, dt);
                    acc = Ops<T>::mma(tr8(p_lo, p_hi), pb[g], acc);
                }
                O[dt] = acc;
            }
            if (kv) {
                lds_store_row(c.SX + (k * B + j) * LD, O, q);
                if (q == 0) {
                    float s = 0.f;
#pragma unroll
                    for (int w = 0; w < WPM; ++w) s += crp[w * ROWSM + k];
                    c.cRs[k * B + j] = s;
                }
            }
        }
        round_end<WPM>(P, rd);
    }

    // Z round: z_ref (ma/ma_torch.py:55-62) and the final slice (:106-108)
    static __device__ __forceinline__ void round_z(const Problem& P, const Round& rd, const Pre& pre, const Ctx& c) {
        const int B = P.B, M = P.M, D = P.D;
        const int slot = c.wave / WPM, wig = c.wave % WPM, tix = wig * 64 + c.lane;
        const int j = rd.rnd * PPM + slot;
        const bool active = j < B;
        const int r = c.r, q = c.q;
        // staging as in an L round: the Y tile (kOneTile) where that has its Q^T tile, the bias behind the P^T tile
        T* Yt = reinterpret_cast<T*>(c.stage + slot * kSlotL);
        float* cb = reinterpret_cast<float*>(Yt + ROWSM * LD + ROWSM * LDP);
        if (active && tix < ROWSM) cb[tix] = tix < M ? -kLog2e * c.cLs[j * M + tix] : kNegBig;
        if (ONE && active) {
            if (rd.rnd == 0) {   // uniform: the first Z round loads its Y tile here, after the barrier that ended the last R phase
                u32x4 ya[CNT];
                y_issue(P, rd.head, ya, j, tix);
                tile_commit(Yt, ya, tix, WPM * 64);
            } else {
                tile_commit(Yt, pre.a, tix, WPM * 64);
            }
        }
        problem_sync<WPM>();
        if (active) {
            const int e = rd.head / P.H, h = rd.head % P.H;
            const Slices S = make_slices<T>(P, e, h, 0);
            const int l = 16 * wig + r;
            const int t = l * B + j - P.pad_off;
            f32x4 C[NTM];
#pragma unroll
            for (int wt = 0; wt < NTM; ++wt) {
                const int k = 16 * wt + r;
                const T* arow = k < M ? c.al_row(j, k, B, M) : c.ZR;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = Ops<T>::mma(lds_row8<T>(arow + 32 * ks + 8 * q), pre.xq[ks], acc);
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
            const int e4 = r >> 2, c4 = r & 3;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int g = 0; g < (NTM + 1) / 2; ++g) {   // k slot s <-> key block 32g + 16(s/4) + 4q + s%4
                    const int lo = 32 * g + 4 * q + e4, hi = lo + 16;
                    const T* ylo = ONE ? Yt + lo * LD : c.SY + (j * M + lo) * LD;
                    const T* yhi = ONE ? Yt + hi * LD : c.SY + (j * M + hi) * LD;
                    const T* p_lo = (lo < M ? ylo : c.ZR) + chunk_col<DT, true>(c4, dt);
                    const T* p_hi = (hi < M ? yhi : c.ZR) + chunk_col<DT, true>(c4, dt);
                    acc = Ops<T>::mma(tr8(p_lo, p_hi), pb[g], acc);
                }
                O[dt] = acc;
            }
            store_row<T, DT, true>(S.out, l < M ? tok_off(t, P.N, S.ost) : kOob, D, O, q, S.stream_out);   // padded query rows are dropped
        }
        round_end<WPM>(P, rd);
    }

    static __device__ __forceinline__ void execute(const Problem& P, const Round& rd, const Pre& pre, const Ctx& c) {
        if (!(rd.p & 1)) round_r(P, rd, pre, c);
        else if (rd.p == 2 * P.T - 1) round_z(P, rd, pre, c);
        else round_l(P, rd, pre, c);
    }
};

template <class T, int DT, int NTB, int NTM, int W, bool ONE>
__global__ __launch_bounds__(64 * W) void resident_fwd_mfma(Problem P, int mode) {
    using RS = Resident<T, DT, NTB, NTM, W, ONE>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int Np = P.M * P.B;
    typename RS::Ctx c;
    c.SA = reinterpret_cast<T*>(smem);
    c.y_on_x = mode == RS::kYOnX;
    const int tiles = RS::tiles_of(mode);
    c.SX = ONE ? c.SA : c.SA + Np * RS::LD;
    c.SY = c.y_on_x ? c.SX : c.SX + Np * RS::LD;   // unused with one tile
    c.ZR = c.SA + tiles * Np * RS::LD;
    c.cLs = reinterpret_cast<float*>(c.ZR + RS::LD);
    c.cRs = c.cLs + (Np + 3) / 4 * 4;
    c.stage = smem + RS::state_bytes(Np, mode);
    c.wave = wave_id();
    c.lane = threadIdx.x & 63;
    c.r = c.lane & 15;
    c.q = c.lane >> 4;
    for (int i = threadIdx.x; i < RS::LD; i += 64 * W) c.ZR[i] = from_f<T>(0.f);
    // The state rows are written 16*DT columns wide but read as GEMM operands over all 32*KS
    // columns: where the two differ (head dims of 65..80) the columns in between are never
    // written and must not hold leftovers (0 * NaN) of whatever used the LDS before.
    if constexpr (16 * DT < 32 * RS::KS) {
        constexpr int kTail = 32 * RS::KS - 16 * DT;
        for (int i = threadIdx.x; i < tiles * Np * kTail; i += 64 * W) c.SA[(i / kTail) * RS::LD + 16 * DT + i % kTail] = from_f<T>(0.f);
    }
    __syncthreads();

    const int heads = P.E * P.H;
    typename RS::Round cur = {static_cast<int>(blockIdx.x), 0, 0};
    if (cur.head >= heads) return;
    typename RS::Pre pc;
    RS::issue(P, cur, pc, c);
    for (;;) {
        typename RS::Round nxt = cur;
        const bool more = RS::advance(P, nxt, heads, gridDim.x);
        typename RS::Pre pn = {};   // fully defined before the conditional loads: no merge of an old and a new set
        if (more) RS::issue(P, nxt, pn, c);   // next round's loads fly while this round computes
        RS::execute(P, cur, pc, c);
        if (!more) break;
        cur = nxt;
        pc = pn;
    }
}

}  // namespace mfma
}  // namespace ma
