// Backward stages on the matrix cores (v_mfma_f32_16x16x4_f32), for every
// operand dtype: a workgroup stages the operand tiles of its block problem in
// LDS (zero-padded to the tile grid; tiles of q, k, v and of the 16-bit state in
// their own dtype, gradients and probabilities as fp32), and every product of the stage
// derivative - the formulas are at the top of ma_bwd.hip - is a small GEMM
// between LDS matrices, read with arbitrary row / column strides so that
// transposed operands cost nothing.  Selected when the tiles of a problem fit
// the LDS and q, k, v share a dtype; the FMA kernels of ma_bwd.hip cover the
// rest.  Ownership and summation order are as there: a workgroup owns every
// row it accumulates into, so results are reproducible bit for bit.
#pragma once

#include "ma_generic_dev.h"
#include "ma_mfma_launch.h"

#include <type_traits>

namespace ma {
namespace {

using f32x4 = float __attribute__((ext_vector_type(4)));

// Row stride of an LDS matrix with n (a multiple of 16) columns.  The GEMM operands are read both
// as (row = lane % 16, column = lane / 16) and as (row = lane / 16, column = lane % 16); a stride of
// 12 or 20 (mod 32) floats keeps the first pattern free of bank conflicts and the second nearly so.
__host__ __device__ constexpr int ld_of(int n) { return n + (n % 32 == 0 ? 12 : 4); }
// The same for a matrix of T: 16-bit rows take a stride of 2 w elements with w = 9 (mod 16) 32-bit
// words, which does for the two read patterns what 12 / 20 (mod 32) does for fp32.
template <class T>
__host__ __device__ constexpr int ld_t(int n) {
    return sizeof(T) == 4 ? ld_of(n) : 2 * ((n / 2 + 6) / 16 * 16 + 9);
}
constexpr size_t kLdsBudget = 156 * 1024;

__host__ __device__ constexpr int up(int x, int m) { return (x + m - 1) / m * m; }

// all-reduce over the wave on the VALU (DPP within 16-lane rows, lane swaps across them)
__device__ __forceinline__ float wmax(float x) { return mfma::quad_rows_max(mfma::row16_max(x)); }
__device__ __forceinline__ float wsum(float x) { return mfma::quad_rows_sum(mfma::row16_sum(x)); }

// all-reduce over aligned groups of G lanes (G = 4 .. 64, a power of two).  The row passes give a
// matrix row to G lanes, so that a wave works on 64 / G rows at once: short rows (small blocks)
// would otherwise leave most lanes idle and walk the rows one after the other.
template <int G>
__device__ __forceinline__ float seg_max(float x) {
    x = fmaxf(x, mfma::dpp<0xB1>(x));
    x = fmaxf(x, mfma::dpp<0x4E>(x));
    if (G >= 8) x = fmaxf(x, mfma::dpp<0x141>(x));
    if (G >= 16) x = fmaxf(x, mfma::dpp<0x140>(x));
    if (G >= 32) {
        float a = x, b = x;
        mfma::swap_rows16(a, b);
        x = fmaxf(a, b);
    }
    if (G >= 64) {
        float a = x, b = x;
        mfma::swap_halves32(a, b);
        x = fmaxf(a, b);
    }
    return x;
}
template <int G>
__device__ __forceinline__ float seg_sum(float x) {
    x += mfma::dpp<0xB1>(x);
    x += mfma::dpp<0x4E>(x);
    if (G >= 8) x += mfma::dpp<0x141>(x);
    if (G >= 16) x += mfma::dpp<0x140>(x);
    if (G >= 32) {
        float a = x, b = x;
        mfma::swap_rows16(a, b);
        x = a + b;
    }
    if (G >= 64) {
        float a = x, b = x;
        mfma::swap_halves32(a, b);
        x = a + b;
    }
    return x;
}
// lanes per row for rows of n (a multiple of 16) entries: four entries per lane for short rows, the
// whole wave for rows of more than 32 entries (measured: there the one-row-per-wave walk, with its
// conflict-free LDS accesses, is the faster one)
inline int group_lanes(int n) { return n <= 16 ? 4 : n <= 32 ? 8 : 64; }
// f(std::integral_constant<int, E>) with E = entries of a row of n per lane of a group of G lanes, for the
// rows that a lane can keep in registers (at most four entries); false if the row is longer
template <int G, class F>
__device__ __forceinline__ bool with_entries(int n, F&& f) {
    if (n > 4 * G) return false;
    if (G < 64) {   // groups of 4 / 8 lanes are only used for rows of 16 / 32: four entries
        f(std::integral_constant<int, 4>{});
        return true;
    }
    switch ((n + G - 1) / G) {
        case 1: f(std::integral_constant<int, 1>{}); break;
        case 2: f(std::integral_constant<int, 2>{}); break;
        case 3: f(std::integral_constant<int, 3>{}); break;
        default: f(std::integral_constant<int, 4>{}); break;
    }
    return true;
}

// acc[t] += sum_k A(r,k) B(k, 16 t + c) for one 16-row strip of up to four 16-column tiles.
// A(r,k) = A[r*ars + k*acs], B(k,c) = B[k*brs + c*bcs]; K is a multiple of 16.  Lane (r = lane % 16,
// q = lane / 16) feeds A(r, k0+q) and B(k0+q, r); acc[t][v] is C(4q+v, 16t+r).  The operands of four
// k-steps are read before their MFMAs are issued, so that the LDS reads overlap.
template <int NT, class TA, class TB>
__device__ __forceinline__ void strip_mma_n(f32x4 (&acc)[4], const TA* A, int ars, int acs, const TB* B, int brs, int bcs, int K) {
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
    const TA* a = A + r * ars + q * acs;
    const TB* b = B + q * brs + r * bcs;
    for (int k0 = 0; k0 < K; k0 += 16) {
        float av[4], bv[4][NT];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            av[u] = to_f(a[(k0 + 4 * u) * acs]);
#pragma unroll
            for (int t = 0; t < NT; ++t) bv[u][t] = to_f(b[(k0 + 4 * u) * brs + 16 * t * bcs]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], bv[u][t], acc[t], 0, 0, 0);
    }
}
template <class TA, class TB>
__device__ __forceinline__ void strip_mma(f32x4 (&acc)[4], int nt, const TA* A, int ars, int acs, const TB* B, int brs, int bcs,
                                          int K) {
    switch (nt) {   // nt is the same for every lane of the wave
        case 1: return strip_mma_n<1>(acc, A, ars, acs, B, brs, bcs, K);
        case 2: return strip_mma_n<2>(acc, A, ars, acs, B, brs, bcs, K);
        case 3: return strip_mma_n<3>(acc, A, ars, acs, B, brs, bcs, K);
        default: return strip_mma_n<4>(acc, A, ars, acs, B, brs, bcs, K);
    }
}

// f(row, col, value) for every element of the strip
template <class F>
__device__ __forceinline__ void strip_each(const f32x4 (&acc)[4], int nt, int r0, int c0, F&& f) {
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (t < nt) {
#pragma unroll
            for (int v = 0; v < 4; ++v) f(r0 + 4 * q + v, c0 + 16 * t + r, acc[t][v]);
        }
}

// base[row * row_stride + col] = (accumulate ? old : 0) + value for every element of the strip with
// row < rows_valid and col < cols_valid.  All old values are loaded before the first store (the loads
// are in flight together instead of one memory round trip per element), and only the strip's NT
// tiles cost address arithmetic.
template <int NT>
__device__ __forceinline__ void strip_rmw_n(const f32x4 (&acc)[4], int r0, int c0, bool accumulate, float* base, long long row_stride,
                                            int rows_valid, int cols_valid) {
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
    float* rowp[4];
    bool rok[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row = r0 + 4 * q + v;
        rok[v] = row < rows_valid;
        rowp[v] = base + row * row_stride + (c0 + r);
    }
    float old[NT][4];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const bool cok = c0 + 16 * t + r < cols_valid;
#pragma unroll
        for (int v = 0; v < 4; ++v) old[t][v] = (accumulate && rok[v] && cok) ? rowp[v][16 * t] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const bool cok = c0 + 16 * t + r < cols_valid;
#pragma unroll
        for (int v = 0; v < 4; ++v)
            if (rok[v] && cok) rowp[v][16 * t] = old[t][v] + acc[t][v];
    }
}
__device__ __forceinline__ void strip_rmw(const f32x4 (&acc)[4], int nt, int r0, int c0, bool accumulate, float* base,
                                          long long row_stride, int rows_valid, int cols_valid) {
    switch (nt) {   // nt is the same for every lane of the wave
        case 1: return strip_rmw_n<1>(acc, r0, c0, accumulate, base, row_stride, rows_valid, cols_valid);
        case 2: return strip_rmw_n<2>(acc, r0, c0, accumulate, base, row_stride, rows_valid, cols_valid);
        case 3: return strip_rmw_n<3>(acc, r0, c0, accumulate, base, row_stride, rows_valid, cols_valid);
        default: return strip_rmw_n<4>(acc, r0, c0, accumulate, base, row_stride, rows_valid, cols_valid);
    }
}

// base[row * row_stride + col] = value rounded to T, for the elements of the strip inside the valid range
template <class T>
__device__ __forceinline__ void strip_store16(const f32x4 (&acc)[4], int nt, int r0, int c0, T* base, long long row_stride,
                                              int rows_valid, int cols_valid) {
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t >= nt) break;
        const int col = c0 + 16 * t + r;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = r0 + 4 * q + v;
            if (row < rows_valid && col < cols_valid) base[row * row_stride + col] = from_f<T>(acc[t][v]);
        }
    }
}

// Strips of a rows x cols output (both multiples of 16) dealt to the waves; body(r0, c0, nt).
// A strip is as wide as lets every wave have one (1, 2 or 4 tiles).
template <int NTH, class F>
__device__ __forceinline__ void for_strips(int rows, int cols, F&& body) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tiles = (rows / 16) * (cols / 16);
    const int wt = tiles >= 4 * (NTH / 64) ? 4 : tiles >= 2 * (NTH / 64) ? 2 : 1;
    const int cg = (cols / 16 + wt - 1) / wt, total = (rows / 16) * cg;
    // (row tile, column group) of strip s; a power-of-two group count (the usual case) needs no division
    const bool pow2 = (cg & (cg - 1)) == 0;
    const int shift = __builtin_ctz(cg);
    for (int s = wave; s < total; s += NTH / 64) {
        const int rt = pow2 ? s >> shift : s / cg;
        const int g = pow2 ? s & (cg - 1) : s - rt * cg;
        body(16 * rt, 16 * wt * g, min(wt, cols / 16 - wt * g));
    }
}

__device__ __forceinline__ void zero_acc(f32x4 (&acc)[4]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// rows x width elements of TD (row stride ld) <- rows of a (.., rows, W) tensor of dtype T, converted
// and multiplied by scale; rows for which row_ptr(i) is null and columns >= W are zero.  Sixteen lanes take a row, four elements each (one 8- or 16-byte load where
// the row allows it), so a wave loads four rows per instruction; two such groups are in flight
// together.
template <int NTH, class T, class TD, class RowPtr>
__device__ __forceinline__ void stage_rows(TD* dst, int ld, int rows, int width, int W, float scale, RowPtr&& row_ptr) {
    constexpr int NW = NTH / 64;
    struct alignas(4 * sizeof(T)) Quad { T v[4]; };
    struct alignas(2 * sizeof(TD)) Pair { TD a, b; };
    const int lane = threadIdx.x & 63, sub = lane >> 4, c0 = lane & 15;
    for (int i0 = 4 * (threadIdx.x >> 6) + sub; i0 < rows; i0 += 8 * NW) {
        const T* p[2];
        bool vec[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int i = i0 + 4 * NW * u;
            p[u] = i < rows ? row_ptr(i) : nullptr;
            vec[u] = W % 4 == 0 && reinterpret_cast<uintptr_t>(p[u]) % sizeof(Quad) == 0;
        }
        for (int c = c0; 4 * c < width; c += 16) {
            Quad x[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (p[u] != nullptr && vec[u] && 4 * c < W) {
                    x[u] = *reinterpret_cast<const Quad*>(p[u] + 4 * c);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) x[u].v[e] = (p[u] != nullptr && 4 * c + e < W) ? p[u][4 * c + e] : from_f<T>(0.f);
                }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = i0 + 4 * NW * u;
                if (i >= rows) continue;
                if constexpr (sizeof(TD) == 4) {
                    *reinterpret_cast<f32x4*>(dst + i * ld + 4 * c) = f32x4{scale * to_f(x[u].v[0]), scale * to_f(x[u].v[1]),
                                                                           scale * to_f(x[u].v[2]), scale * to_f(x[u].v[3])};
                } else if (std::is_same<T, TD>::value && scale == 1.f) {   // copied as they are
                    *reinterpret_cast<Pair*>(dst + i * ld + 4 * c) = Pair{from_f<TD>(to_f(x[u].v[0])), from_f<TD>(to_f(x[u].v[1]))};
                    *reinterpret_cast<Pair*>(dst + i * ld + 4 * c + 2) = Pair{from_f<TD>(to_f(x[u].v[2])), from_f<TD>(to_f(x[u].v[3]))};
                } else {   // 16-bit rows start on 4-byte boundaries only
                    *reinterpret_cast<Pair*>(dst + i * ld + 4 * c) =
                        Pair{from_f<TD>(scale * to_f(x[u].v[0])), from_f<TD>(scale * to_f(x[u].v[1]))};
                    *reinterpret_cast<Pair*>(dst + i * ld + 4 * c + 2) =
                        Pair{from_f<TD>(scale * to_f(x[u].v[2])), from_f<TD>(scale * to_f(x[u].v[3]))};
                }
            }
        }
    }
}

// Several tiles staged together: the loads of all of them are issued before any is written to LDS,
// so a stage waits for one memory round trip instead of one per tile.  Same work split and same
// zero-filling as stage_rows; the tiles may differ in rows, width and types.  Costs registers: used
// by the single-wave workgroups of small blocks, whose stages are one chain of memory round trips.
template <class T, class TD, class RowPtr>
struct TileSpec {
    struct alignas(4 * sizeof(T)) Quad { T v[4]; };
    struct alignas(2 * sizeof(TD)) Pair { TD a, b; };
    TD* dst;
    int ld, rows, width, W;
    float scale;
    RowPtr row_ptr;
    const T* p[2];
    Quad x[2];

    __device__ __forceinline__ void rows_begin(int i0, int step) {
#pragma unroll
        for (int u = 0; u < 2; ++u) p[u] = i0 + step * u < rows ? row_ptr(i0 + step * u) : nullptr;
    }
    __device__ __forceinline__ void load(int c) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (p[u] != nullptr && W % 4 == 0 && reinterpret_cast<uintptr_t>(p[u]) % sizeof(Quad) == 0 && 4 * c < W) {
                x[u] = *reinterpret_cast<const Quad*>(p[u] + 4 * c);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) x[u].v[e] = (p[u] != nullptr && 4 * c + e < W) ? p[u][4 * c + e] : from_f<T>(0.f);
            }
        }
    }
    __device__ __forceinline__ void store(int i0, int step, int c) const {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int i = i0 + step * u;
            if (i >= rows || 4 * c >= width) continue;
            TD* d = dst + i * ld + 4 * c;
            if constexpr (sizeof(TD) == 4) {
                *reinterpret_cast<f32x4*>(d) = f32x4{scale * to_f(x[u].v[0]), scale * to_f(x[u].v[1]), scale * to_f(x[u].v[2]),
                                                     scale * to_f(x[u].v[3])};
            } else if (std::is_same<T, TD>::value && scale == 1.f) {   // copied as they are
                *reinterpret_cast<Pair*>(d) = Pair{from_f<TD>(to_f(x[u].v[0])), from_f<TD>(to_f(x[u].v[1]))};
                *reinterpret_cast<Pair*>(d + 2) = Pair{from_f<TD>(to_f(x[u].v[2])), from_f<TD>(to_f(x[u].v[3]))};
            } else {
                *reinterpret_cast<Pair*>(d) = Pair{from_f<TD>(scale * to_f(x[u].v[0])), from_f<TD>(scale * to_f(x[u].v[1]))};
                *reinterpret_cast<Pair*>(d + 2) = Pair{from_f<TD>(scale * to_f(x[u].v[2])), from_f<TD>(scale * to_f(x[u].v[3]))};
            }
        }
    }
};
template <class T, class TD, class RowPtr>
__device__ __forceinline__ TileSpec<T, TD, RowPtr> tile_of(TD* dst, int ld, int rows, int width, int W, float scale, RowPtr row_ptr) {
    return TileSpec<T, TD, RowPtr>{dst, ld, rows, width, W, scale, row_ptr, {nullptr, nullptr}, {}};
}
template <int NTH, class... Ts>
__device__ __forceinline__ void stage_tiles(Ts... t) {
    constexpr int NW = NTH / 64;
    const int lane = threadIdx.x & 63, sub = lane >> 4, c0 = lane & 15;
    int rows = 0, width = 0;
    ((rows = max(rows, t.rows), width = max(width, t.width)), ...);
    for (int i0 = 4 * (threadIdx.x >> 6) + sub; i0 < rows; i0 += 8 * NW) {
        (t.rows_begin(i0, 4 * NW), ...);
        for (int c = c0; 4 * c < width; c += 16) {
            (t.load(c), ...);
            (t.store(i0, 4 * NW, c), ...);
        }
    }
}

// softmax over columns [0, cols) of every row of U[rows][ld], in place (entries may be -inf)
template <int NTH>
__device__ __forceinline__ void softmax_rows_lds(float* U, int ld, int rows, int cols) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int ll = wave; ll < rows; ll += NTH / 64) {
        float* Ul = U + ll * ld;
        float mx = -INFINITY;
        for (int k = lane; k < cols; k += 64) mx = fmaxf(mx, Ul[k]);
        mx = wmax(mx);
        float sum = 0.f;
        for (int k = lane; k < cols; k += 64) {
            const float p = __expf(Ul[k] - mx);
            Ul[k] = p;
            sum += p;
        }
        sum = wsum(sum);
        const float inv = 1.0f / sum;
        for (int k = lane; k < cols; k += 64) Ul[k] = Ul[k] * inv;
    }
}

// ---------------------------------------------------------------- Z and L stages
// LDS of the Z / L stage for tiles of TL query blocks: byte offsets and row strides (elements).
//   aL[M16][ldd] TQ, W[M16][ldw] (Z: Y_j, TQ; L: gaR_j, float), cl[M16], cw[M16] (L: gcR_j),
//   Qt[TL][ldd] TQ, dO[TL][ldo] TQ (Z only), qok[TL], U[TL][ldm], Gg[TL][ldm]
struct LzLayout {
    int ldd, ldw, ldo, ldm;
    unsigned aLt, Wt, cl, cw, Qt, dO, qok, U, Gg, total;
};
template <class TQ>
__host__ __device__ inline LzLayout lz_layout(int M, int D, int W, bool z, int TL) {
    const int M16 = up(M, 16), D16 = up(D, 16), W16 = up(W, 16);
    LzLayout L;
    L.ldd = ld_t<TQ>(D16);
    L.ldw = z ? ld_t<TQ>(W16) : ld_of(W16);
    L.ldo = ld_t<TQ>(W16);
    L.ldm = ld_of(M16);
    unsigned off = 0;
    auto take = [&](size_t bytes) { const unsigned at = off; off += static_cast<unsigned>((bytes + 15) / 16 * 16); return at; };
    L.aLt = take(sizeof(TQ) * M16 * L.ldd);
    L.Wt = take((z ? sizeof(TQ) : sizeof(float)) * M16 * L.ldw);
    L.cl = take(4 * M16);
    L.cw = take(4 * M16);
    L.Qt = take(sizeof(TQ) * TL * L.ldd);
    L.dO = take(z ? sizeof(TQ) * TL * L.ldo : 0);
    L.qok = take(4 * TL);
    L.U = take(4 * TL * L.ldm);
    L.Gg = take(4 * TL * L.ldm);
    L.total = off;
    return L;
}

// One workgroup per (e,h,j), TL query blocks l at a time (TL a multiple of 16).
template <class TQ, bool kZ, int NTH>
__global__ __launch_bounds__(NTH) void lz_bwd_mfma(Problem P, BwdBuffers G, int TL) {
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    using TW = typename std::conditional<kZ, TQ, float>::type;
    const int M = P.M, D = P.D, B = P.B, W = kZ ? P.Dv : P.D;
    const int M16 = up(M, 16), D16 = up(D, 16), W16 = up(W, 16);
    const LzLayout L = lz_layout<TQ>(M, D, W, kZ, TL);
    const int ldd = L.ldd, ldw = L.ldw, ldo = L.ldo, ldm = L.ldm;
    int w = blockIdx.x;
    const int j = w % B; w /= B;
    const int h = w % P.H, e = w / P.H;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long jm = (eh * B + j) * M;
    TQ* aLt = reinterpret_cast<TQ*>(lds_raw + L.aLt);
    TW* Wt = reinterpret_cast<TW*>(lds_raw + L.Wt);
    float* cl = reinterpret_cast<float*>(lds_raw + L.cl);
    float* cw = reinterpret_cast<float*>(lds_raw + L.cw);
    TQ* Qt = reinterpret_cast<TQ*>(lds_raw + L.Qt);
    TQ* dO = reinterpret_cast<TQ*>(lds_raw + L.dO);
    float* qok = reinterpret_cast<float*>(lds_raw + L.qok);
    float* U = reinterpret_cast<float*>(lds_raw + L.U);
    float* Gg = reinterpret_cast<float*>(lds_raw + L.Gg);

    const TQ* aL = reinterpret_cast<const TQ*>(P.aL) + jm * D;
    stage_rows<NTH, TQ, TQ>(aLt, ldd, M16, D16, D, 1.f, [&](int k) { return k < M ? aL + k * D : nullptr; });
    if (kZ) {
        const TQ* Y = reinterpret_cast<const TQ*>(P.Y) + jm * W;
        stage_rows<NTH, TQ, TQ>(reinterpret_cast<TQ*>(Wt), ldw, M16, W16, W, 1.f,
                                [&](int k) { return k < M ? Y + k * static_cast<long long>(W) : nullptr; });
    } else {
        stage_rows<NTH, float, float>(reinterpret_cast<float*>(Wt), ldw, M16, W16, W, 1.f,
                                      [&](int k) { return k < M ? G.gaR + ((eh * M + k) * B + j) * D : nullptr; });
    }
    for (int k = threadIdx.x; k < M16; k += NTH) {
        cl[k] = k < M ? P.cL[jm + k] : 0.f;
        cw[k] = (!kZ && k < M) ? G.gcR[(eh * M + k) * B + j] : 0.f;
    }

    for (int l0 = 0; l0 < M; l0 += TL) {
        stage_rows<NTH, TQ, TQ>(Qt, ldd, TL, D16, D, 1.f, [&](int ll) {
            return l0 + ll < M ? tok_row<TQ>(P.q, P.qs, e, h, (l0 + ll) * B + j - P.pad_off, P.N) : nullptr;
        });
        if (kZ)
            stage_rows<NTH, TQ, TQ>(dO, ldo, TL, W16, W, 1.f, [&](int ll) {
                return l0 + ll < M ? tok_row<TQ>(G.dout, G.dos, e, h, (l0 + ll) * B + j - P.pad_off, P.N) : nullptr;
            });
        for (int ll = threadIdx.x; ll < TL; ll += NTH)
            qok[ll] = (l0 + ll < M && token_ok(P, e, (l0 + ll) * B + j - P.pad_off)) ? 1.f : 0.f;
        __syncthreads();

        // U = round(Qt aL^T) - cL, -inf in the columns beyond M
        for_strips<NTH>(TL, M16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, Qt + r0 * ldd, ldd, 1, aLt + c0 * ldd, 1, ldd, D16);
            strip_each(acc, nt, r0, c0, [&](int ll, int k, float x) { U[ll * ldm + k] = k < M ? round_to<TQ>(x) - cl[k] : -INFINITY; });
        });
        // Z: gLz = dO Y^T;  L: gLm = mask_q (Qt gaR^T + gcR)
        for_strips<NTH>(TL, M16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            if (kZ) strip_mma(acc, nt, dO + r0 * ldo, ldo, 1, Wt + c0 * ldw, 1, ldw, W16);
            else strip_mma(acc, nt, Qt + r0 * ldd, ldd, 1, Wt + c0 * ldw, 1, ldw, W16);
            strip_each(acc, nt, r0, c0, [&](int ll, int k, float x) {
                if (!kZ) x = (k < M && qok[ll] != 0.f) ? x + cw[k] : 0.f;
                Gg[ll * ldm + k] = x;
            });
        });
        __syncthreads();
        softmax_rows_lds<NTH>(U, ldm, TL, M16);   // a wave has the same rows here and in the pass below
        {   // dU = p (g - sum g p); afterwards U holds the rounded (L: query-masked) probabilities
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            for (int ll = wave; ll < TL; ll += NTH / 64) {
                float dot = 0.f;
                for (int k = lane; k < M16; k += 64) dot = fmaf(Gg[ll * ldm + k], U[ll * ldm + k], dot);
                dot = wsum(dot);
                const float keep = kZ ? 1.f : qok[ll];
                for (int k = lane; k < M16; k += 64) {
                    const float p = U[ll * ldm + k];
                    Gg[ll * ldm + k] = p * (Gg[ll * ldm + k] - dot);
                    U[ll * ldm + k] = keep * round_to<TQ>(p);
                }
            }
        }
        __syncthreads();
        if (kZ) {   // gY (+)= round(Lz)^T dO
            for_strips<NTH>(M16, W16, [&](int r0, int c0, int nt) {
                f32x4 acc[4];
                zero_acc(acc);
                strip_mma(acc, nt, U + r0, 1, ldm, dO + c0, ldo, 1, TL);
                strip_rmw(acc, nt, r0, c0, l0 != 0, G.gY + jm * W, W, M, W);
            });
        }
        // gaL (+)= dU^T Qt
        for_strips<NTH>(M16, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, Gg + r0, 1, ldm, Qt + c0, ldd, 1, TL);
            strip_rmw(acc, nt, r0, c0, l0 != 0, G.gaL + jm * D, D, M, D);
        });
        for (int k = threadIdx.x; k < M; k += NTH) {   // gcL (+)= -sum_l dU
            float acc = l0 ? G.gcL[jm + k] : 0.f;
#pragma unroll 8
            for (int ll = 0; ll < TL; ++ll) acc -= Gg[ll * ldm + k];
            G.gcL[jm + k] = acc;
        }
        // dq rows (l, j) += dU aL  (L: + round(Lm) gaR)
        for_strips<NTH>(TL, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, Gg + r0 * ldm, ldm, 1, aLt + c0, ldd, 1, M16);
            if (!kZ) strip_mma(acc, nt, U + r0 * ldm, ldm, 1, Wt + c0, ldw, 1, M16);
            // the Z stage runs first and every dq row belongs to one tile of one workgroup: it is written, not added to
            strip_rmw(acc, nt, r0, c0, !kZ, G.dq + (eh * M * B + static_cast<long long>(l0) * B + j) * D, static_cast<long long>(B) * D,
                      M - l0, D);
        });
        __syncthreads();
    }
}

// ---------------------------------------------------------------- R stage
// LDS of the R stage for tiles of TJ query rows: byte offsets and row strides (elements).
//   Kt[B16][ldd] TQ, Vt[B16][ldv] TQ, kok[B16], X[TJ][ldd] TQ, Ga[TJ][lga] (sm * gaL), Gy[TJ][lgy],
//   c[TJ], gcl[TJ], S[TJ][ldb], R[TJ][ldb], Gg[TJ][ldb]
struct RLayout {
    int ldd, ldv, lga, lgy, ldb;
    unsigned Kt, Vt, kok, X, Ga, Gy, c, gcl, S, R, Gg, total;
};
template <class TQ>
__host__ __device__ inline RLayout r_layout(int B, int D, int Dv, bool with_v, int TJ) {
    const int B16 = up(B, 16), D16 = up(D, 16), V16 = up(Dv, 16);
    RLayout L;
    L.ldd = ld_t<TQ>(D16);
    L.ldv = ld_t<TQ>(V16);
    L.lga = ld_of(D16);
    L.lgy = ld_of(V16);
    L.ldb = ld_of(B16);
    unsigned off = 0;
    auto take = [&](size_t bytes) { const unsigned at = off; off += static_cast<unsigned>((bytes + 15) / 16 * 16); return at; };
    L.Kt = take(sizeof(TQ) * B16 * L.ldd);
    L.Vt = take(with_v ? sizeof(TQ) * B16 * L.ldv : 0);
    L.kok = take(4 * B16);
    L.X = take(sizeof(TQ) * TJ * L.ldd);
    L.Ga = take(4 * TJ * L.lga);
    L.Gy = take(with_v ? 4 * TJ * L.lgy : 0);
    L.c = take(4 * TJ);
    L.gcl = take(4 * TJ);
    L.S = take(4 * TJ * L.ldb);
    L.R = take(4 * TJ * L.ldb);
    L.Gg = take(4 * TJ * L.ldb);
    L.total = off;
    return L;
}

// One workgroup per key block (e,h,k), TJ query rows j at a time (TJ a multiple of 16).
template <class TQ, int NTH>
__global__ __launch_bounds__(NTH) void r_bwd_mfma(Problem P, BwdBuffers G, int TJ, int first, int with_v) {
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    const int B = P.B, M = P.M, D = P.D, Dv = P.Dv;
    const int B16 = up(B, 16), D16 = up(D, 16), V16 = up(Dv, 16);
    const RLayout L = r_layout<TQ>(B, D, Dv, with_v != 0, TJ);
    const int ldd = L.ldd, ldv = L.ldv, lga = L.lga, lgy = L.lgy, ldb = L.ldb;
    // G.jt_split > 0: the tiles of query rows of a block go to different workgroups (few, large blocks);
    // their dk / dv parts then land in per-tile partial buffers that a reduction adds up in a fixed order
    int w = blockIdx.x;
    const int jt = G.jt_split ? w % G.jt_split : 0;
    if (G.jt_split) w /= G.jt_split;
    const int k = w % M; w /= M;
    const int h = w % P.H, e = w / P.H;
    const int j_begin = G.jt_split ? jt * TJ : 0, j_end = G.jt_split ? min(B, j_begin + TJ) : B;
    const long long part = static_cast<long long>(jt) * P.E * P.H * M * B;   // row offset into the partial buffers
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aR = reinterpret_cast<const TQ*>(P.aR) + (eh * M + k) * B * D;
    const float* cR = P.cR + (eh * M + k) * B;
    const float sm = P.sm_scale;
    TQ* Kt = reinterpret_cast<TQ*>(lds_raw + L.Kt);
    TQ* Vt = reinterpret_cast<TQ*>(lds_raw + L.Vt);
    float* kok = reinterpret_cast<float*>(lds_raw + L.kok);
    TQ* X = reinterpret_cast<TQ*>(lds_raw + L.X);
    float* Ga = reinterpret_cast<float*>(lds_raw + L.Ga);
    float* Gy = reinterpret_cast<float*>(lds_raw + L.Gy);
    float* c = reinterpret_cast<float*>(lds_raw + L.c);
    float* gcl = reinterpret_cast<float*>(lds_raw + L.gcl);
    float* S = reinterpret_cast<float*>(lds_raw + L.S);
    float* R = reinterpret_cast<float*>(lds_raw + L.R);
    float* Gg = reinterpret_cast<float*>(lds_raw + L.Gg);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    stage_rows<NTH, TQ, TQ>(Kt, ldd, B16, D16, D, 1.f,
                   [&](int i) { return i < B ? tok_row<TQ>(P.k, P.ks, e, h, k * B + i - P.pad_off, P.N) : nullptr; });
    if (with_v)
        stage_rows<NTH, TQ, TQ>(Vt, ldv, B16, V16, Dv, 1.f,
                       [&](int i) { return i < B ? tok_row<TQ>(P.v, P.vs, e, h, k * B + i - P.pad_off, P.N) : nullptr; });
    for (int i = threadIdx.x; i < B16; i += NTH) kok[i] = (i < B && token_ok(P, e, k * B + i - P.pad_off)) ? 1.f : 0.f;

    for (int j0 = j_begin; j0 < j_end; j0 += TJ) {
        stage_rows<NTH, TQ, TQ>(X, ldd, TJ, D16, D, 1.f, [&](int jj) -> const TQ* {
            if (j0 + jj >= B) return nullptr;
            return first ? tok_row<TQ>(P.q, P.qs, e, h, k * B + j0 + jj - P.pad_off, P.N) : aR + (j0 + jj) * D;
        });
        stage_rows<NTH, float, float>(Ga, lga, TJ, D16, D, sm,
                          [&](int jj) { return j0 + jj < B ? G.gaL + ((eh * B + j0 + jj) * M + k) * D : nullptr; });
        if (with_v)
            stage_rows<NTH, float, float>(Gy, lgy, TJ, V16, Dv, 1.f, [&](int jj) {
                return j0 + jj < B ? G.gY + ((eh * B + j0 + jj) * M + k) * static_cast<long long>(Dv) : nullptr;
            });
        for (int jj = threadIdx.x; jj < TJ; jj += NTH) {
            const bool in = j0 + jj < B;
            c[jj] = 1.0f / (((first || !in) ? 1.0f : cR[j0 + jj]) + P.eps);   // c holds 1 / (cR + eps)
            gcl[jj] = in ? G.gcL[(eh * B + j0 + jj) * M + k] : 0.f;
        }
        __syncthreads();

        // S = sm round(X K^T) / (cR + eps), -inf for masked / padded keys
        for_strips<NTH>(TJ, B16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, X + r0 * ldd, ldd, 1, Kt + c0 * ldd, 1, ldd, D16);
            strip_each(acc, nt, r0, c0,
                       [&](int jj, int i, float x) { S[jj * ldb + i] = kok[i] != 0.f ? sm * round_to<TQ>(x) * c[jj] : -INFINITY; });
        });
        // sm gaL K^T + gY V^T, the part of g that does not need the probabilities
        for_strips<NTH>(TJ, B16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, Ga + r0 * lga, lga, 1, Kt + c0 * ldd, 1, ldd, D16);
            if (with_v) strip_mma(acc, nt, Gy + r0 * lgy, lgy, 1, Vt + c0 * ldv, 1, ldv, V16);
            strip_each(acc, nt, r0, c0, [&](int jj, int i, float x) { Gg[jj * ldb + i] = x; });
        });
        __syncthreads();
        for (int jj = wave; jj < TJ; jj += NTH / 64) {
            // probabilities (ma_torch.py:14-18)
            float mx = -INFINITY;
            for (int i = lane; i < B16; i += 64) mx = fmaxf(mx, S[jj * ldb + i]);
            mx = fmaxf(wmax(mx), P.eps);
            float sum = 0.f;
            for (int i = lane; i < B16; i += 64) {
                const float p = __expf(S[jj * ldb + i] - mx);
                R[jj * ldb + i] = p;
                sum += p;
            }
            const float inv = 1.0f / (wsum(sum) + P.eps);
            // g = gcL (log r + 1) + sm gaL K^T + gY V^T where the clamp did not act, else 0
            float dot = 0.f;
            for (int i = lane; i < B16; i += 64) {
                const float r = R[jj * ldb + i] * inv;
                const float rc = i < B ? fmaxf(r, kTiny) : 0.f;
                const float g = (i < B && r >= kTiny) ? fmaf(gcl[jj], __logf(rc) + 1.0f, Gg[jj * ldb + i]) : 0.f;
                R[jj * ldb + i] = rc;
                Gg[jj * ldb + i] = g;
                dot = fmaf(g, rc, dot);
            }
            dot = wsum(dot);
            // dS, gcR; Gg <- dDot = dS sm / (cR + eps); R <- round(r)
            float gc = 0.f;
            for (int i = lane; i < B16; i += 64) {
                const float s = S[jj * ldb + i], r = R[jj * ldb + i];
                const float ds = s == -INFINITY ? 0.f : r * (Gg[jj * ldb + i] - dot);
                if (s != -INFINITY) gc = fmaf(-ds, s * c[jj], gc);
                Gg[jj * ldb + i] = ds * sm * c[jj];
                R[jj * ldb + i] = round_to<TQ>(r);
            }
            gc = wsum(gc);
            if (!first && lane == 0 && j0 + jj < B) G.gcR[(eh * M + k) * B + j0 + jj] = gc;
        }
        __syncthreads();
        // gaR = dDot K (first step: aR is q, the rows of block k of dq)
        for_strips<NTH>(TJ, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, Gg + r0 * ldb, ldb, 1, Kt + c0, ldd, 1, B16);
            strip_rmw(acc, nt, r0, c0, first != 0, (first ? G.dq : G.gaR) + ((eh * M + k) * B + j0) * D, D, B - j0, D);
        });
        // dK += round(r)^T (sm gaL) + dDot^T X
        for_strips<NTH>(B16, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma(acc, nt, R + r0, 1, ldb, Ga + c0, lga, 1, TJ);
            strip_mma(acc, nt, Gg + r0, 1, ldb, X + c0, ldd, 1, TJ);
            strip_rmw(acc, nt, r0, c0, !G.jt_split, (G.jt_split ? G.pk + part * D : G.dk) + (eh * M + k) * B * D, D, B, D);
        });
        if (with_v)   // dV += round(r)^T gY
            for_strips<NTH>(B16, V16, [&](int r0, int c0, int nt) {
                f32x4 acc[4];
                zero_acc(acc);
                strip_mma(acc, nt, R + r0, 1, ldb, Gy + c0, lgy, 1, TJ);
                strip_rmw(acc, nt, r0, c0, j0 != j_begin,   // dv has this one writer
                          (G.jt_split ? G.pv + part * Dv : G.dv) + (eh * M + k) * B * static_cast<long long>(Dv), Dv, B, Dv);
            });
        __syncthreads();
    }
}

// largest tile (multiple of 16, at most the padded extent) whose LDS fits; 0 if none
template <class F>
int pick_tile(int extent, F&& bytes) {
    for (int t = up(extent, 16); t >= 16; t -= 16)
        if (bytes(t) <= kLdsBudget) return t;
    return 0;
}

// ================================================================ fp16 / bf16 operands
// The same stages with every GEMM operand as a 16-bit LDS matrix (row pitch n + 8 elements) and
// v_mfma_f32_16x16x16_{f16,bf16}: a lane's four k-values are one 8-byte LDS read - a plain one
// where k runs along the row, ds_read_b64_tr_b16 where it runs down the column (lane 4e+c of a
// 16-lane group addresses row e, columns 4c..4c+3 of a 4 x 16 block and receives column lane%16).
// Probabilities and their gradients are kept in fp32 for the softmax arithmetic and rounded to the
// operand dtype for the products, which is where autograd through the reference rounds them too.
typedef short i16x4 __attribute__((ext_vector_type(4)));
__host__ __device__ constexpr int ld16(int n) { return n + 8; }

template <class T>
struct Mma16;
template <>
struct Mma16<f16> {
    static __device__ __forceinline__ f32x4 mma(i16x4 a, i16x4 b, f32x4 c) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a), __builtin_bit_cast(h4, b), c, 0, 0, 0);
    }
};
template <>
struct Mma16<bf16> {
    static __device__ __forceinline__ f32x4 mma(i16x4 a, i16x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
    }
};

template <bool TR, class T>
__device__ __forceinline__ i16x4 lds_k4(const T* p) {
    if constexpr (TR) {
        typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
    } else {
        return *reinterpret_cast<const i16x4*>(p);
    }
}

// acc[t] += sum_k A(r,k) B(k, 16 t + c) for one 16-row strip of NT 16-column tiles, K a multiple of 16.
// TA = false: A is stored [row][k] (pitch lda) and points at the strip's first row; TA = true: A is
// stored [k][row] and points at the strip's first column.  TB = false: B is stored [column][k] and
// points at the first column's row; TB = true: B is stored [k][column] and points at the first column.
template <int NT, bool TA, bool TB, class T>
__device__ __forceinline__ void strip_mma16_n(f32x4 (&acc)[4], const T* A, int lda, const T* B, int ldb, int K) {
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4, e = r >> 2, c = r & 3;
    const T* a = TA ? A + (4 * q + e) * lda + 4 * c : A + r * lda + 4 * q;
    const T* b = TB ? B + (4 * q + e) * ldb + 4 * c : B + r * ldb + 4 * q;
    const int astep = TA ? 16 * lda : 16, bstep = TB ? 16 * ldb : 16, btile = TB ? 16 : 16 * ldb;
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 16) {
        const i16x4 av = lds_k4<TA>(a);
        i16x4 bv[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) bv[t] = lds_k4<TB>(b + t * btile);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = Mma16<T>::mma(av, bv[t], acc[t]);
        a += astep;
        b += bstep;
    }
}
template <bool TA, bool TB, class T>
__device__ __forceinline__ void strip_mma16(f32x4 (&acc)[4], int nt, const T* A, int lda, const T* B, int ldb, int K) {
    switch (nt) {   // nt is the same for every lane of the wave
        case 1: return strip_mma16_n<1, TA, TB>(acc, A, lda, B, ldb, K);
        case 2: return strip_mma16_n<2, TA, TB>(acc, A, lda, B, ldb, K);
        case 3: return strip_mma16_n<3, TA, TB>(acc, A, lda, B, ldb, K);
        default: return strip_mma16_n<4, TA, TB>(acc, A, lda, B, ldb, K);
    }
}

// LDS of the 16-bit Z / L stage: aL[M16][ldd], W[M16][ldw] (Z: Y_j; L: gaR_j rounded), cl[M16],
// cw[M16], Qt[TL][ldd], dO[TL][ldw] (Z), qok[TL], U[TL][ldm] f32, Gg[TL][ldm] f32, G16[TL][ldp].
// The rounded probabilities U16 are written over U row by row (row pitch 2 ldm elements).
struct LzLayout16 {
    int ldd, ldw, ldm, ldp;
    unsigned aLt, Wt, cl, cw, Qt, dO, qok, U, Gg, G16, total;
};
__host__ __device__ inline LzLayout16 lz_layout16(int M, int D, int W, bool z, int TL) {
    const int M16 = up(M, 16), D16 = up(D, 16), W16 = up(W, 16);
    LzLayout16 L;
    L.ldd = ld16(D16);
    L.ldw = ld16(W16);
    L.ldm = ld_of(M16);
    L.ldp = ld16(M16);
    unsigned off = 0;
    auto take = [&](size_t bytes) { const unsigned at = off; off += static_cast<unsigned>((bytes + 15) / 16 * 16); return at; };
    L.aLt = take(2 * M16 * L.ldd);
    L.Wt = take(2 * M16 * L.ldw);
    L.cl = take(4 * M16);
    L.cw = take(4 * M16);
    L.Qt = take(2 * TL * L.ldd);
    L.dO = take(z ? 2 * TL * L.ldw : 0);
    L.qok = take(4 * TL);
    L.U = take(4 * TL * L.ldm);
    L.Gg = take(4 * TL * L.ldm);
    L.G16 = take(2 * TL * L.ldp);
    L.total = off;
    return L;
}

// S16: the state gradients gaL, gY, gaR are kept in the operand dtype instead of fp32 (the host sets it
// when every stage runs these kernels and no state gradient is accumulated over several tiles: the
// values are rounded to the operand dtype on their way into the next stage's LDS either way)
template <class TQ, bool kZ, int NTH, int GL, bool S16>
__global__ __launch_bounds__(NTH) void lz_bwd_mfma16(Problem P, BwdBuffers G, int TL) {
    using TG = typename std::conditional<S16, TQ, float>::type;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    const int M = P.M, D = P.D, B = P.B, W = kZ ? P.Dv : P.D;
    const int M16 = up(M, 16), D16 = up(D, 16), W16 = up(W, 16);
    const LzLayout16 L = lz_layout16(M, D, W, kZ, TL);
    const int ldd = L.ldd, ldw = L.ldw, ldm = L.ldm, ldp = L.ldp;
    int w = blockIdx.x;
    const int j = w % B; w /= B;
    const int h = w % P.H, e = w / P.H;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long jm = (eh * B + j) * M;
    TQ* aLt = reinterpret_cast<TQ*>(lds_raw + L.aLt);
    TQ* Wt = reinterpret_cast<TQ*>(lds_raw + L.Wt);
    float* cl = reinterpret_cast<float*>(lds_raw + L.cl);
    float* cw = reinterpret_cast<float*>(lds_raw + L.cw);
    TQ* Qt = reinterpret_cast<TQ*>(lds_raw + L.Qt);
    TQ* dO = reinterpret_cast<TQ*>(lds_raw + L.dO);
    float* qok = reinterpret_cast<float*>(lds_raw + L.qok);
    float* U = reinterpret_cast<float*>(lds_raw + L.U);
    float* Gg = reinterpret_cast<float*>(lds_raw + L.Gg);
    typedef TQ __attribute__((may_alias)) TQa;   // 16-bit values stored over fp32 ones that were just read
    TQa* U16 = reinterpret_cast<TQa*>(lds_raw + L.U);
    const int ldu = 2 * ldm;
    TQ* G16 = reinterpret_cast<TQ*>(lds_raw + L.G16);

    const TQ* aL = reinterpret_cast<const TQ*>(P.aL) + jm * D;
    const TQ* Y = reinterpret_cast<const TQ*>(P.Y) + jm * W;
    auto aL_row = [=](int k) { return k < M ? aL + k * D : nullptr; };
    auto y_row = [=](int k) { return k < M ? Y + k * static_cast<long long>(W) : nullptr; };
    const TG* gaR = reinterpret_cast<const TG*>(G.gaR);
    auto gar_row = [=](int k) { return k < M ? gaR + ((eh * M + k) * B + j) * D : nullptr; };
    constexpr bool kJoint = NTH == 64;   // single-wave workgroups stage all their tiles in one go
    if (!kJoint) {
        stage_rows<NTH, TQ, TQ>(aLt, ldd, M16, D16, D, 1.f, aL_row);
        if (kZ) stage_rows<NTH, TQ, TQ>(Wt, ldw, M16, W16, W, 1.f, y_row);
        else stage_rows<NTH, TG, TQ>(Wt, ldw, M16, W16, W, 1.f, gar_row);
    }
    for (int k = threadIdx.x; k < M16; k += NTH) {
        cl[k] = k < M ? P.cL[jm + k] : 0.f;
        cw[k] = (!kZ && k < M) ? G.gcR[(eh * M + k) * B + j] : 0.f;
    }

    for (int l0 = 0; l0 < M; l0 += TL) {
        auto q_row = [=](int ll) {
            return l0 + ll < M ? tok_row<TQ>(P.q, P.qs, e, h, (l0 + ll) * B + j - P.pad_off, P.N) : nullptr;
        };
        auto do_row = [=](int ll) {
            return l0 + ll < M ? tok_row<TQ>(G.dout, G.dos, e, h, (l0 + ll) * B + j - P.pad_off, P.N) : nullptr;
        };
        if (kJoint) {   // the state tiles of the whole problem travel with the first tile of query blocks
            const int state_rows = l0 == 0 ? M16 : 0;
            if (kZ)
                stage_tiles<NTH>(tile_of<TQ>(aLt, ldd, state_rows, D16, D, 1.f, aL_row), tile_of<TQ>(Wt, ldw, state_rows, W16, W, 1.f, y_row),
                                 tile_of<TQ>(Qt, ldd, TL, D16, D, 1.f, q_row), tile_of<TQ>(dO, ldw, TL, W16, W, 1.f, do_row));
            else
                stage_tiles<NTH>(tile_of<TQ>(aLt, ldd, state_rows, D16, D, 1.f, aL_row),
                                 tile_of<TG>(Wt, ldw, state_rows, W16, W, 1.f, gar_row), tile_of<TQ>(Qt, ldd, TL, D16, D, 1.f, q_row));
        } else {
            stage_rows<NTH, TQ, TQ>(Qt, ldd, TL, D16, D, 1.f, q_row);
            if (kZ) stage_rows<NTH, TQ, TQ>(dO, ldw, TL, W16, W, 1.f, do_row);
        }
        for (int ll = threadIdx.x; ll < TL; ll += NTH)
            qok[ll] = (l0 + ll < M && token_ok(P, e, (l0 + ll) * B + j - P.pad_off)) ? 1.f : 0.f;
        __syncthreads();

        // U = round(Qt aL^T) - cL, -inf in the columns beyond M
        for_strips<NTH>(TL, M16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<false, false>(acc, nt, Qt + r0 * ldd, ldd, aLt + c0 * ldd, ldd, D16);
            strip_each(acc, nt, r0, c0, [&](int ll, int k, float x) { U[ll * ldm + k] = k < M ? round_to<TQ>(x) - cl[k] : -INFINITY; });
        });
        // Z: gLz = dO Y^T;  L: gLm = mask_q (Qt gaR^T + gcR)
        for_strips<NTH>(TL, M16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            if (kZ) strip_mma16<false, false>(acc, nt, dO + r0 * ldw, ldw, Wt + c0 * ldw, ldw, W16);
            else strip_mma16<false, false>(acc, nt, Qt + r0 * ldd, ldd, Wt + c0 * ldw, ldw, W16);
            strip_each(acc, nt, r0, c0, [&](int ll, int k, float x) {
                if (!kZ) x = (k < M && qok[ll] != 0.f) ? x + cw[k] : 0.f;
                Gg[ll * ldm + k] = x;
            });
        });
        __syncthreads();
        // per row: softmax, dU = p (g - sum g p); U16 <- rounded (L: query-masked) probabilities, G16 <- rounded dU
        {
            constexpr int RPP = 64 / GL;
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane / GL, cg = lane % GL;
            // rows of up to four entries per lane stay in registers between the reductions
            const bool in_regs = with_entries<GL>(M16, [&](auto etag) {
                constexpr int EPL = decltype(etag)::value;
                for (int l1 = wave * RPP; l1 < TL; l1 += (NTH / 64) * RPP) {
                    const int ll = l1 + sub;
                    float* Ul = U + ll * ldm;
                    float* Gl = Gg + ll * ldm;
                    float u[EPL], g[EPL];
                    float mx = -INFINITY;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int k = cg + GL * e;
                        u[e] = k < M16 ? Ul[k] : -INFINITY;
                        g[e] = k < M16 ? Gl[k] : 0.f;
                        mx = fmaxf(mx, u[e]);
                    }
                    mx = seg_max<GL>(mx);
                    float sum = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        u[e] = __expf(u[e] - mx);
                        sum += u[e];
                    }
                    const float inv = mfma::rcp(seg_sum<GL>(sum));
                    float dot = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        u[e] *= inv;
                        dot = fmaf(g[e], u[e], dot);
                    }
                    dot = seg_sum<GL>(dot);
                    const float keep = kZ ? 1.f : qok[ll];
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int k = cg + GL * e;
                        if (k >= M16) continue;
                        const float du = u[e] * (g[e] - dot);
                        Gl[k] = du;
                        G16[ll * ldp + k] = from_f<TQ>(du);
                        U16[ll * ldu + k] = from_f<TQ>(keep * u[e]);   // over fp32 entries this row's lanes have read
                    }
                }
            });
            if (!in_regs)
            for (int l1 = wave * RPP; l1 < TL; l1 += (NTH / 64) * RPP) {
                const int ll = l1 + sub;
                float* Ul = U + ll * ldm;
                float* Gl = Gg + ll * ldm;
                float mx = -INFINITY;
                for (int k = cg; k < M16; k += GL) mx = fmaxf(mx, Ul[k]);
                mx = seg_max<GL>(mx);
                float sum = 0.f;
                for (int k = cg; k < M16; k += GL) {
                    const float p = __expf(Ul[k] - mx);
                    Ul[k] = p;
                    sum += p;
                }
                const float inv = 1.0f / seg_sum<GL>(sum);
                float dot = 0.f;
                for (int k = cg; k < M16; k += GL) dot = fmaf(Gl[k], Ul[k] * inv, dot);
                dot = seg_sum<GL>(dot);
                const float keep = kZ ? 1.f : qok[ll];
                for (int k = cg; k < M16; k += GL) {
                    const float p = Ul[k] * inv;
                    const float du = p * (Gl[k] - dot);
                    Gl[k] = du;
                    G16[ll * ldp + k] = from_f<TQ>(du);
                    U16[ll * ldu + k] = from_f<TQ>(keep * p);   // lands on fp32 entries these lanes have read already
                }
            }
        }
        __syncthreads();
        if (kZ) {   // gY (+)= round(Lz)^T dO
            for_strips<NTH>(M16, W16, [&](int r0, int c0, int nt) {
                f32x4 acc[4];
                zero_acc(acc);
                strip_mma16<true, true>(acc, nt, reinterpret_cast<const TQ*>(U16) + r0, ldu, dO + c0, ldw, TL);
                if (S16) strip_store16(acc, nt, r0, c0, reinterpret_cast<TQ*>(G.gY) + jm * W, W, M, W);
                else strip_rmw(acc, nt, r0, c0, l0 != 0, G.gY + jm * W, W, M, W);
            });
        }
        // gaL (+)= dU^T Qt
        for_strips<NTH>(M16, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<true, true>(acc, nt, G16 + r0, ldp, Qt + c0, ldd, TL);
            if (S16) strip_store16(acc, nt, r0, c0, reinterpret_cast<TQ*>(G.gaL) + jm * D, D, M, D);
            else strip_rmw(acc, nt, r0, c0, l0 != 0, G.gaL + jm * D, D, M, D);
        });
        for (int k = threadIdx.x; k < M; k += NTH) {   // gcL (+)= -sum_l dU
            float acc = l0 ? G.gcL[jm + k] : 0.f;
#pragma unroll 8
            for (int ll = 0; ll < TL; ++ll) acc -= Gg[ll * ldm + k];
            G.gcL[jm + k] = acc;
        }
        // dq rows (l, j) += dU aL  (L: + round(Lm) gaR)
        for_strips<NTH>(TL, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<false, true>(acc, nt, G16 + r0 * ldp, ldp, aLt + c0, ldd, M16);
            if (!kZ) strip_mma16<false, true>(acc, nt, reinterpret_cast<const TQ*>(U16) + r0 * ldu, ldu, Wt + c0, ldw, M16);
            // the Z stage runs first and every dq row belongs to one tile of one workgroup: it is written, not added to
            strip_rmw(acc, nt, r0, c0, !kZ, G.dq + (eh * M * B + static_cast<long long>(l0) * B + j) * D, static_cast<long long>(B) * D,
                      M - l0, D);
        });
        __syncthreads();
    }
}

// LDS of the 16-bit R stage: Kt[B16][ldd], Vt[B16][ldv], kok[B16], X[TJ][ldd], Ga[TJ][ldd]
// (sm * gaL, rounded), Gy[TJ][ldv], c[TJ], gcl[TJ], S, R, Gg [TJ][ldb] f32.  The rounded
// probabilities and the rounded dDot are written over R and Gg row by row (row pitch 2 ldb elements).
struct RLayout16 {
    int ldd, ldv, ldb;
    unsigned Kt, Vt, kok, X, Ga, Gy, c, gcl, S, R, Gg, total;
};
__host__ __device__ inline RLayout16 r_layout16(int B, int D, int Dv, bool with_v, int TJ) {
    const int B16 = up(B, 16), D16 = up(D, 16), V16 = up(Dv, 16);
    RLayout16 L;
    L.ldd = ld16(D16);
    L.ldv = ld16(V16);
    L.ldb = ld_of(B16);
    unsigned off = 0;
    auto take = [&](size_t bytes) { const unsigned at = off; off += static_cast<unsigned>((bytes + 15) / 16 * 16); return at; };
    L.Kt = take(2 * B16 * L.ldd);
    L.Vt = take(with_v ? 2 * B16 * L.ldv : 0);
    L.kok = take(4 * B16);
    L.X = take(2 * TJ * L.ldd);
    L.Ga = take(2 * TJ * L.ldd);
    L.Gy = take(with_v ? 2 * TJ * L.ldv : 0);
    L.c = take(4 * TJ);
    L.gcl = take(4 * TJ);
    L.S = take(4 * TJ * L.ldb);
    L.R = take(4 * TJ * L.ldb);
    L.Gg = take(4 * TJ * L.ldb);
    L.total = off;
    return L;
}

template <class TQ, int NTH, int GL, bool S16>
__global__ __launch_bounds__(NTH) void r_bwd_mfma16(Problem P, BwdBuffers G, int TJ, int first, int with_v) {
    using TG = typename std::conditional<S16, TQ, float>::type;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    const int B = P.B, M = P.M, D = P.D, Dv = P.Dv;
    const int B16 = up(B, 16), D16 = up(D, 16), V16 = up(Dv, 16);
    const RLayout16 L = r_layout16(B, D, Dv, with_v != 0, TJ);
    const int ldd = L.ldd, ldv = L.ldv, ldb = L.ldb, ldp = 2 * L.ldb;
    // G.jt_split > 0: the tiles of query rows of a block go to different workgroups (few, large blocks);
    // their dk / dv parts then land in per-tile partial buffers that a reduction adds up in a fixed order
    int w = blockIdx.x;
    const int jt = G.jt_split ? w % G.jt_split : 0;
    if (G.jt_split) w /= G.jt_split;
    const int k = w % M; w /= M;
    const int h = w % P.H, e = w / P.H;
    const int j_begin = G.jt_split ? jt * TJ : 0, j_end = G.jt_split ? min(B, j_begin + TJ) : B;
    const long long part = static_cast<long long>(jt) * P.E * P.H * M * B;   // row offset into the partial buffers
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aR = reinterpret_cast<const TQ*>(P.aR) + (eh * M + k) * B * D;
    const float* cR = P.cR + (eh * M + k) * B;
    const float sm = P.sm_scale;
    TQ* Kt = reinterpret_cast<TQ*>(lds_raw + L.Kt);
    TQ* Vt = reinterpret_cast<TQ*>(lds_raw + L.Vt);
    float* kok = reinterpret_cast<float*>(lds_raw + L.kok);
    TQ* X = reinterpret_cast<TQ*>(lds_raw + L.X);
    TQ* Ga = reinterpret_cast<TQ*>(lds_raw + L.Ga);
    TQ* Gy = reinterpret_cast<TQ*>(lds_raw + L.Gy);
    float* c = reinterpret_cast<float*>(lds_raw + L.c);
    float* gcl = reinterpret_cast<float*>(lds_raw + L.gcl);
    float* S = reinterpret_cast<float*>(lds_raw + L.S);
    float* R = reinterpret_cast<float*>(lds_raw + L.R);
    float* Gg = reinterpret_cast<float*>(lds_raw + L.Gg);
    typedef TQ __attribute__((may_alias)) TQa;   // 16-bit values stored over fp32 ones that were just read
    TQa* R16 = reinterpret_cast<TQa*>(lds_raw + L.R);
    TQa* Dd = reinterpret_cast<TQa*>(lds_raw + L.Gg);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    auto k_row = [=](int i) { return i < B ? tok_row<TQ>(P.k, P.ks, e, h, k * B + i - P.pad_off, P.N) : nullptr; };
    auto v_row = [=](int i) { return i < B ? tok_row<TQ>(P.v, P.vs, e, h, k * B + i - P.pad_off, P.N) : nullptr; };
    constexpr bool kJoint = NTH == 64;   // single-wave workgroups stage all their tiles in one go
    if (!kJoint) {
        stage_rows<NTH, TQ, TQ>(Kt, ldd, B16, D16, D, 1.f, k_row);
        if (with_v) stage_rows<NTH, TQ, TQ>(Vt, ldv, B16, V16, Dv, 1.f, v_row);
    }
    for (int i = threadIdx.x; i < B16; i += NTH) kok[i] = (i < B && token_ok(P, e, k * B + i - P.pad_off)) ? 1.f : 0.f;

    for (int j0 = j_begin; j0 < j_end; j0 += TJ) {
        auto x_row = [=](int jj) -> const TQ* {
            if (j0 + jj >= B) return nullptr;
            return first ? tok_row<TQ>(P.q, P.qs, e, h, k * B + j0 + jj - P.pad_off, P.N) : aR + (j0 + jj) * D;
        };
        const TG* gaL = reinterpret_cast<const TG*>(G.gaL);
        const TG* gY = reinterpret_cast<const TG*>(G.gY);
        auto ga_row = [=](int jj) { return j0 + jj < B ? gaL + ((eh * B + j0 + jj) * M + k) * D : nullptr; };
        auto gy_row = [=](int jj) {
            return j0 + jj < B ? gY + ((eh * B + j0 + jj) * M + k) * static_cast<long long>(Dv) : nullptr;
        };
        if (kJoint) {   // the key / value tiles of the block travel with the first tile of query rows
            const int kv_rows = j0 == j_begin ? B16 : 0;
            stage_tiles<NTH>(tile_of<TQ>(Kt, ldd, kv_rows, D16, D, 1.f, k_row),
                             tile_of<TQ>(Vt, ldv, with_v ? kv_rows : 0, V16, Dv, 1.f, v_row), tile_of<TQ>(X, ldd, TJ, D16, D, 1.f, x_row),
                             tile_of<TG>(Ga, ldd, TJ, D16, D, sm, ga_row), tile_of<TG>(Gy, ldv, with_v ? TJ : 0, V16, Dv, 1.f, gy_row));
        } else {
            stage_rows<NTH, TQ, TQ>(X, ldd, TJ, D16, D, 1.f, x_row);
            stage_rows<NTH, TG, TQ>(Ga, ldd, TJ, D16, D, sm, ga_row);
            if (with_v) stage_rows<NTH, TG, TQ>(Gy, ldv, TJ, V16, Dv, 1.f, gy_row);
        }
        for (int jj = threadIdx.x; jj < TJ; jj += NTH) {
            const bool in = j0 + jj < B;
            c[jj] = 1.0f / (((first || !in) ? 1.0f : cR[j0 + jj]) + P.eps);   // c holds 1 / (cR + eps)
            gcl[jj] = in ? G.gcL[(eh * B + j0 + jj) * M + k] : 0.f;
        }
        __syncthreads();

        // S = sm round(X K^T) / (cR + eps), -inf for masked / padded keys
        for_strips<NTH>(TJ, B16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<false, false>(acc, nt, X + r0 * ldd, ldd, Kt + c0 * ldd, ldd, D16);
            strip_each(acc, nt, r0, c0,
                       [&](int jj, int i, float x) { S[jj * ldb + i] = kok[i] != 0.f ? sm * round_to<TQ>(x) * c[jj] : -INFINITY; });
        });
        // sm gaL K^T + gY V^T, the part of g that does not need the probabilities
        for_strips<NTH>(TJ, B16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<false, false>(acc, nt, Ga + r0 * ldd, ldd, Kt + c0 * ldd, ldd, D16);
            if (with_v) strip_mma16<false, false>(acc, nt, Gy + r0 * ldv, ldv, Vt + c0 * ldv, ldv, V16);
            strip_each(acc, nt, r0, c0, [&](int jj, int i, float x) { Gg[jj * ldb + i] = x; });
        });
        __syncthreads();
        {
            constexpr int RPP = 64 / GL;
            const int sub = lane / GL, cg = lane % GL;
            // rows of up to four entries per lane stay in registers between the reductions
            const bool in_regs = with_entries<GL>(B16, [&](auto etag) {
                constexpr int EPL = decltype(etag)::value;
                for (int j1 = wave * RPP; j1 < TJ; j1 += (NTH / 64) * RPP) {
                    const int jj = j1 + sub;
                    const float* Sj = S + jj * ldb;
                    const float* Gj = Gg + jj * ldb;
                    float sv[EPL], g[EPL], r[EPL];
                    // probabilities (ma_torch.py:14-18)
                    float mx = -INFINITY;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int i = cg + GL * e;
                        sv[e] = i < B16 ? Sj[i] : -INFINITY;
                        g[e] = i < B16 ? Gj[i] : 0.f;
                        mx = fmaxf(mx, sv[e]);
                    }
                    mx = fmaxf(seg_max<GL>(mx), P.eps);
                    float sum = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        r[e] = __expf(sv[e] - mx);
                        sum += r[e];
                    }
                    const float inv = mfma::rcp(seg_sum<GL>(sum) + P.eps);
                    // g = gcL (log r + 1) + sm gaL K^T + gY V^T where the clamp did not act, else 0
                    float dot = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int i = cg + GL * e;
                        const float ru = r[e] * inv;
                        r[e] = i < B ? fmaxf(ru, kTiny) : 0.f;
                        g[e] = (i < B && ru >= kTiny) ? fmaf(gcl[jj], __logf(r[e]) + 1.0f, g[e]) : 0.f;
                        dot = fmaf(g[e], r[e], dot);
                    }
                    dot = seg_sum<GL>(dot);
                    // dS, gcR; D16 <- dDot = dS sm / (cR + eps); R16 <- round(r)
                    float gc = 0.f;
                    const float cj = c[jj];
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int i = cg + GL * e;
                        if (i >= B16) continue;
                        const float ds = sv[e] == -INFINITY ? 0.f : r[e] * (g[e] - dot);
                        if (sv[e] != -INFINITY) gc = fmaf(-ds, sv[e] * cj, gc);
                        Dd[jj * ldp + i] = from_f<TQ>(ds * sm * cj);   // both over fp32 entries this row's lanes have read
                        R16[jj * ldp + i] = from_f<TQ>(r[e]);
                    }
                    gc = seg_sum<GL>(gc);
                    if (!first && cg == 0 && j0 + jj < B) G.gcR[(eh * M + k) * B + j0 + jj] = gc;
                }
            });
            if (!in_regs)
            for (int j1 = wave * RPP; j1 < TJ; j1 += (NTH / 64) * RPP) {
                const int jj = j1 + sub;
                float* Sj = S + jj * ldb;
                float* Rj = R + jj * ldb;
                float* Gj = Gg + jj * ldb;
                // probabilities (ma_torch.py:14-18)
                float mx = -INFINITY;
                for (int i = cg; i < B16; i += GL) mx = fmaxf(mx, Sj[i]);
                mx = fmaxf(seg_max<GL>(mx), P.eps);
                float sum = 0.f;
                for (int i = cg; i < B16; i += GL) {
                    const float p = __expf(Sj[i] - mx);
                    Rj[i] = p;
                    sum += p;
                }
                const float inv = 1.0f / (seg_sum<GL>(sum) + P.eps);
                // g = gcL (log r + 1) + sm gaL K^T + gY V^T where the clamp did not act, else 0
                float dot = 0.f;
                for (int i = cg; i < B16; i += GL) {
                    const float r = Rj[i] * inv;
                    const float rc = i < B ? fmaxf(r, kTiny) : 0.f;
                    const float g = (i < B && r >= kTiny) ? fmaf(gcl[jj], __logf(rc) + 1.0f, Gj[i]) : 0.f;
                    Rj[i] = rc;
                    Gj[i] = g;
                    dot = fmaf(g, rc, dot);
                }
                dot = seg_sum<GL>(dot);
                // dS, gcR; D16 <- dDot = dS sm / (cR + eps); R16 <- round(r)
                float gc = 0.f;
                for (int i = cg; i < B16; i += GL) {
                    const float sv = Sj[i], r = Rj[i];
                    const float ds = sv == -INFINITY ? 0.f : r * (Gj[i] - dot);
                    if (sv != -INFINITY) gc = fmaf(-ds, sv * c[jj], gc);
                    Dd[jj * ldp + i] = from_f<TQ>(ds * sm * c[jj]);   // both land on fp32 entries these lanes have read already
                    R16[jj * ldp + i] = from_f<TQ>(r);
                }
                gc = seg_sum<GL>(gc);
                if (!first && cg == 0 && j0 + jj < B) G.gcR[(eh * M + k) * B + j0 + jj] = gc;
            }
        }
        __syncthreads();
        // gaR = dDot K (first step: aR is q, the rows of block k of dq)
        for_strips<NTH>(TJ, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<false, true>(acc, nt, reinterpret_cast<const TQ*>(Dd) + r0 * ldp, ldp, Kt + c0, ldd, B16);
            if (S16 && !first) strip_store16(acc, nt, r0, c0, reinterpret_cast<TQ*>(G.gaR) + ((eh * M + k) * B + j0) * D, D, B - j0, D);
            else strip_rmw(acc, nt, r0, c0, first != 0, (first ? G.dq : G.gaR) + ((eh * M + k) * B + j0) * D, D, B - j0, D);
        });
        // dK += round(r)^T (sm gaL) + dDot^T X
        for_strips<NTH>(B16, D16, [&](int r0, int c0, int nt) {
            f32x4 acc[4];
            zero_acc(acc);
            strip_mma16<true, true>(acc, nt, reinterpret_cast<const TQ*>(R16) + r0, ldp, Ga + c0, ldd, TJ);
            strip_mma16<true, true>(acc, nt, reinterpret_cast<const TQ*>(Dd) + r0, ldp, X + c0, ldd, TJ);
            strip_rmw(acc, nt, r0, c0, !G.jt_split, (G.jt_split ? G.pk + part * D : G.dk) + (eh * M + k) * B * D, D, B, D);
        });
        if (with_v)   // dV += round(r)^T gY
            for_strips<NTH>(B16, V16, [&](int r0, int c0, int nt) {
                f32x4 acc[4];
                zero_acc(acc);
                strip_mma16<true, true>(acc, nt, reinterpret_cast<const TQ*>(R16) + r0, ldp, Gy + c0, ldv, TJ);
                strip_rmw(acc, nt, r0, c0, j0 != j_begin,   // dv has this one writer
                          (G.jt_split ? G.pv + part * Dv : G.dv) + (eh * M + k) * B * static_cast<long long>(Dv), Dv, B, Dv);
            });
        __syncthreads();
    }
}

// dst[i] += sum_t part[t][i], t ascending (n floats per part; four per thread)
__global__ void add_parts_kernel(float* dst, const float* part, long long n, int parts, int assign) {
    for (long long i = 4 * (blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x); i < n;
         i += 4 * static_cast<long long>(gridDim.x) * blockDim.x) {
        f32x4 acc = assign ? f32x4{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const f32x4*>(dst + i);
        for (int t = 0; t < parts; ++t) acc += *reinterpret_cast<const f32x4*>(part + t * n + i);
        *reinterpret_cast<f32x4*>(dst + i) = acc;
    }
}

// threads per workgroup for a stage whose probability matrix has `tiles` 16 x 16 tiles
int threads_for(int tiles) { return tiles <= 2 ? 64 : tiles <= 8 ? 256 : 1024; }

#include "ma_bwd_reg.h"

template <class T>
constexpr int dtype_of() { return sizeof(T) == 4 ? MA_F32 : std::is_same<T, f16>::value ? MA_F16 : MA_BF16; }

// Tile of query rows of the R stage for a problem, 0 if it does not fit the LDS.
inline int r_tile(const Problem& P, int dt_qk, bool with_v) {
    auto bytes = [&](int t) -> size_t {
        return dt_qk == MA_F32 ? r_layout<float>(P.B, P.D, P.Dv, with_v, t).total : r_layout16(P.B, P.D, P.Dv, with_v, t).total;
    };
    return pick_tile(P.B, bytes);
}

// Whether the register kernels (ma_bwd_reg.h) take the L / Z stages resp. the R stage of a problem.
inline bool reg_operands_ok(const Problem& P, int dt_qk, int dt_v) {
    return dt_qk != MA_F32 && dt_qk == dt_v && P.Dv == P.D && P.D % 4 == 0 && P.D <= 128;
}

// Whether a backward pass of this problem can keep its state gradients in the operand dtype: fp16 /
// bf16 operands of one dtype, every stage on a 16-bit matrix-core kernel, and gaL and gY written once,
// not accumulated over tiles of query blocks (the register kernels always do; the LDS kernels when
// the L / Z stages fit in a single tile).  The values are rounded to the operand dtype on their way
// into the next stage's operand tiles either way, so the result is the same bit for bit.
inline bool state16_ok(const Problem& P, int dt_qk, int dt_v) {
    if (dt_qk == MA_F32 || dt_qk != dt_v) return false;
    const bool reg = reg_operands_ok(P, dt_qk, dt_v);
    const int M16 = up(P.M, 16);
    const bool lz_ok = (reg && P.M <= 128) || (lz_layout16(P.M, P.D, P.Dv, true, M16).total <= kLdsBudget &&
                                               lz_layout16(P.M, P.D, P.D, false, M16).total <= kLdsBudget);
    const bool r_ok = r_tile(P, dt_qk, true) > 0 || (reg && P.B <= 128);
    return lz_ok && r_ok;
}

// Number of per-tile partial buffers the R stage wants for dk / dv (0: none).  Splitting a block's
// tiles of query rows over workgroups pays when the blocks alone cannot fill the chip.
inline int r_split_tiles(const Problem& P, int dt_qk, int dt_v) {
    if (dt_qk != dt_v) return 0;
    const int TJ = r_tile(P, dt_qk, true);
    if (TJ == 0) return 0;
    const int tiles = (P.B + TJ - 1) / TJ;
    const long long blocks = static_cast<long long>(P.E) * P.H * P.M;
    const long long np = static_cast<long long>(P.M) * P.B;
    return (tiles > 1 && blocks < 512 && (np * P.D) % 4 == 0 && (np * P.Dv) % 4 == 0) ? tiles : 0;
}

// Whether every stage of a backward pass runs a register kernel.  Those write every row of dq (Z stage)
// and dv, and the first R stage they run starts dk's sums: the accumulators need no zeroing then.
inline bool all_reg(const Problem& P, int dt_qk, int dt_v) {
    return reg_operands_ok(P, dt_qk, dt_v) && P.M <= 128 && P.B <= 128 && r_split_tiles(P, dt_qk, dt_v) <= 1;
}

// The launchers return MA_ERR_UNSUPPORTED when the problem does not fit; the caller then takes the FMA kernel.
template <class TQ>
int launch_lz_t(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s) {
    constexpr bool k32 = sizeof(TQ) == 4;
    const int W = z ? P.Dv : P.D;
    auto bytes = [&](int t) -> size_t {
        return k32 ? lz_layout<TQ>(P.M, P.D, W, z, t).total : lz_layout16(P.M, P.D, W, z, t).total;
    };
    if constexpr (!k32) {   // 16-bit operands: the register kernel where it applies
        const int st = launch_lz_reg<TQ>(P, G, z, s);
        if (st != static_cast<int>(MA_ERR_UNSUPPORTED)) return st;
    }
    const int TL = pick_tile(P.M, bytes);
    if (TL == 0) return static_cast<int>(MA_ERR_UNSUPPORTED);
    const size_t lds = bytes(TL);
    const int nth = threads_for((TL / 16) * (up(P.M, 16) / 16));
    auto launch = [&](auto kernel) {
        const int attr = mfma::set_lds_limit(kernel, kLdsBudget);
        if (attr) return attr;
        hipLaunchKernelGGL(kernel, dim3(P.E * P.H * P.B), dim3(nth), lds, s, P, G, TL);
        return static_cast<int>(hipGetLastError());
    };
    if constexpr (k32) {
        if (nth == 64) return z ? launch(lz_bwd_mfma<TQ, true, 64>) : launch(lz_bwd_mfma<TQ, false, 64>);
        if (nth == 256) return z ? launch(lz_bwd_mfma<TQ, true, 256>) : launch(lz_bwd_mfma<TQ, false, 256>);
        return z ? launch(lz_bwd_mfma<TQ, true, 1024>) : launch(lz_bwd_mfma<TQ, false, 1024>);
    } else {
        // lanes per probability row: short rows go with the small workgroups
        const int gl = group_lanes(up(P.M, 16));
        auto pick = [&](auto s16) {
            constexpr bool S = decltype(s16)::value;
            if (nth == 64 && gl == 4) return z ? launch(lz_bwd_mfma16<TQ, true, 64, 4, S>) : launch(lz_bwd_mfma16<TQ, false, 64, 4, S>);
            if (nth == 64 && gl == 8) return z ? launch(lz_bwd_mfma16<TQ, true, 64, 8, S>) : launch(lz_bwd_mfma16<TQ, false, 64, 8, S>);
            if (nth == 64) return z ? launch(lz_bwd_mfma16<TQ, true, 64, 64, S>) : launch(lz_bwd_mfma16<TQ, false, 64, 64, S>);
            if (nth == 256 && gl == 8) return z ? launch(lz_bwd_mfma16<TQ, true, 256, 8, S>) : launch(lz_bwd_mfma16<TQ, false, 256, 8, S>);
            if (nth == 256) return z ? launch(lz_bwd_mfma16<TQ, true, 256, 64, S>) : launch(lz_bwd_mfma16<TQ, false, 256, 64, S>);
            return z ? launch(lz_bwd_mfma16<TQ, true, 1024, 64, S>) : launch(lz_bwd_mfma16<TQ, false, 1024, 64, S>);
        };
        return G.state16 ? pick(std::true_type{}) : pick(std::false_type{});
    }
}

template <class TQ>
int launch_r_t(const Problem& P, const BwdBuffers& G0, bool first, bool with_v, hipStream_t s) {
    constexpr bool k32 = sizeof(TQ) == 4;
    constexpr int dt_qk = dtype_of<TQ>();
    auto bytes = [&](int t) -> size_t {
        return k32 ? r_layout<TQ>(P.B, P.D, P.Dv, with_v, t).total : r_layout16(P.B, P.D, P.Dv, with_v, t).total;
    };
    // the partial buffers are sized for the tiling of the step that also forms dv (the smallest tile)
    const int parts = G0.pk != nullptr ? r_split_tiles(P, dt_qk, dt_qk) : 0;
    if constexpr (!k32) {   // 16-bit operands: the register kernel where it applies
        if (parts <= 1) {
            const int st = launch_r_reg<TQ>(P, G0, first, with_v, s);
            if (st != static_cast<int>(MA_ERR_UNSUPPORTED)) return st;
        }
    }
    int TJ = pick_tile(P.B, bytes);
    if (TJ == 0) return static_cast<int>(MA_ERR_UNSUPPORTED);
    BwdBuffers G = G0;
    G.jt_split = 0;
    if (parts > 1) {
        TJ = min(TJ, r_tile(P, dt_qk, true));
        G.jt_split = (P.B + TJ - 1) / TJ;
    }
    const size_t lds = bytes(TJ);
    const int nth = threads_for((TJ / 16) * (up(P.B, 16) / 16));
    const long long grid = static_cast<long long>(P.E) * P.H * P.M * (G.jt_split ? G.jt_split : 1);
    auto launch = [&](auto kernel) {
        const int attr = mfma::set_lds_limit(kernel, kLdsBudget);
        if (attr) return attr;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(nth), lds, s, P, G, TJ, first ? 1 : 0, with_v ? 1 : 0);
        return static_cast<int>(hipGetLastError());
    };
    int st;
    if constexpr (k32) {
        if (nth == 64) st = launch(r_bwd_mfma<TQ, 64>);
        else if (nth == 256) st = launch(r_bwd_mfma<TQ, 256>);
        else st = launch(r_bwd_mfma<TQ, 1024>);
    } else {
        const int gl = group_lanes(up(P.B, 16));
        auto pick = [&](auto s16) {
            constexpr bool S = decltype(s16)::value;
            if (nth == 64 && gl == 4) return launch(r_bwd_mfma16<TQ, 64, 4, S>);
            if (nth == 64 && gl == 8) return launch(r_bwd_mfma16<TQ, 64, 8, S>);
            if (nth == 64) return launch(r_bwd_mfma16<TQ, 64, 64, S>);
            if (nth == 256 && gl == 8) return launch(r_bwd_mfma16<TQ, 256, 8, S>);
            if (nth == 256) return launch(r_bwd_mfma16<TQ, 256, 64, S>);
            return launch(r_bwd_mfma16<TQ, 1024, 64, S>);
        };
        st = G.state16 ? pick(std::true_type{}) : pick(std::false_type{});
    }
    if (st || !G.jt_split) return st;
    const long long rows = static_cast<long long>(P.E) * P.H * P.M * P.B;
    hipLaunchKernelGGL(add_parts_kernel, dim3(1024), dim3(256), 0, s, G.dk, G.pk, rows * P.D, G.jt_split, 0);
    if (with_v) hipLaunchKernelGGL(add_parts_kernel, dim3(1024), dim3(256), 0, s, G.dv, G.pv, rows * P.Dv, G.jt_split, 0);
    return static_cast<int>(hipGetLastError());
}

}  // namespace
}  // namespace ma
