// Device and host helpers shared by the FMA kernels (forward stages, dense
// matrix, backward stages).
#pragma once

#include "ma_common.h"

namespace ma {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr float kTiny = 1.17549435e-38f;  // finfo(float32).tiny, ma_torch.py:18

__device__ __forceinline__ float wave_max(float x) {
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

// Row pointer of a padded-sequence token in q / k / v, or nullptr for a pad row.
template <class T>
__device__ __forceinline__ const T* tok_row(const char* base, const long long* st, int e, int h, int t, int N) {
    if (t < 0 || t >= N) return nullptr;
    return reinterpret_cast<const T*>(base) + e * st[0] + h * st[1] + static_cast<long long>(t) * st[2];
}

// dot product of two rows; both operands have the same element type.  Four
// elements per load when the rows allow it (length and addresses multiples of 4
// elements), which shortens the dependent load chain fourfold.
template <class T>
__device__ __forceinline__ float dot_rows(const T* a, const T* b, int D) {
    float acc = 0.f;
    if (a == nullptr || b == nullptr) return acc;
    struct alignas(4 * sizeof(T)) Quad { T v[4]; };
    if (D % 4 == 0 && (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % sizeof(Quad) == 0) {
        const Quad* qa = reinterpret_cast<const Quad*>(a);
        const Quad* qb = reinterpret_cast<const Quad*>(b);
#pragma unroll 4
        for (int d = 0; d < D / 4; ++d) {   // unrolled: the loads of several steps are in flight together
            const Quad x = qa[d], y = qb[d];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = fmaf(to_f(x.v[i]), to_f(y.v[i]), acc);
        }
        return acc;
    }
    for (int d = 0; d < D; ++d) acc = fmaf(to_f(a[d]), to_f(b[d]), acc);
    return acc;
}

// sum_i round(w[i * ws]) * X[t0 + i * ts][d] over `rows` tokens of q / k / v; pad rows
// (t outside [0, N)) count as zero.  The row index is clamped and the weight
// zeroed instead of branching, so that the unrolled loop keeps several
// (independent) loads in flight.
template <class T>
__device__ __forceinline__ float weighted_column(const float* w, int ws, const char* base, const long long* st, int e, int h, int t0,
                                                 int ts, int rows, int N, int d) {
    const T* x = reinterpret_cast<const T*>(base) + e * st[0] + h * st[1] + d;
    float acc = 0.f;
#pragma unroll 4
    for (int i = 0; i < rows; ++i) {
        const int t = t0 + i * ts;
        const bool ok = t >= 0 && t < N;
        const float xv = to_f(x[static_cast<long long>(ok ? t : 0) * st[2]]);
        acc = fmaf(ok ? round_to<T>(w[i * ws]) : 0.f, xv, acc);
    }
    return acc;
}

// ---------------------------------------------------------------- L / Z logits
// U[ll][k] = round(Qt[j,l,:] . aL[j,k,:]) - cL[j,k] for TL query blocks l.
template <class TQ>
__device__ __forceinline__ void lz_logits(const Problem& P, float* U, int e, int h, int j, int l0, int rows) {
    const int M = P.M, D = P.D;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aL = reinterpret_cast<const TQ*>(P.aL) + (eh * P.B + j) * M * D;
    const float* cL = P.cL + (eh * P.B + j) * M;
    for (int idx = threadIdx.x; idx < rows * M; idx += kThreads) {
        const int ll = idx / M, kk = idx % M;
        const TQ* qr = tok_row<TQ>(P.q, P.qs, e, h, (l0 + ll) * P.B + j - P.pad_off, P.N);
        U[ll * M + kk] = round_to<TQ>(dot_rows(qr, aL + kk * D, D)) - cL[kk];
    }
}

__device__ __forceinline__ void decode_bj(const Problem& P, int tiles, int& e, int& h, int& j, int& tile) {
    int w = blockIdx.x;
    tile = w % tiles; w /= tiles;
    j = w % P.B; w /= P.B;
    h = w % P.H;
    e = w / P.H;
}

// rows per workgroup so that rows * width floats fit the LDS budget
inline int tile_rows(int width, int want) {
    const long long budget = 48 * 1024 / 4;
    long long r = budget / (width > 0 ? width : 1);
    if (r < 1) r = 1;
    return static_cast<int>(r < want ? r : want);
}

template <class F>
int dispatch_qk(int dt, F&& f) {
    switch (dt) {
        case MA_F32: return f(float{});
        case MA_F16: return f(f16{});
        default: return f(bf16{});
    }
}

}  // namespace
}  // namespace ma
