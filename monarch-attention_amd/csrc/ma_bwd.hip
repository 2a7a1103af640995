// Backward pass of the forward stages, fp32 FMA arithmetic, every dtype / shape /
// stride / mask the forward accepts.  The reference has no backward code of its
// own: it trains through PyTorch autograd over ma/ma_torch.py:10-108.  These
// kernels are that derivative written out per stage; casts count as identity
// (as autograd treats `.to(dtype)`), the clamp to `tiny` blocks the gradient of
// clamped entries (:18), and the 1e-12-relative gradient through the row
// maximum (:14-16) is dropped.
//
// With S = sm*round(aR K^T)/(cR+eps), r = clamp(softmax-like(S)), cL = sum r log r,
// aL = sm*round(round(r) K), Y = round(r) V            (R step, :10-23 / :38-52)
//   g    = gcL*(log r + 1) + sm*gaL K^T + gY V^T           (0 where r was clamped)
//   dS   = r*(g - sum_i g r),  dDot = dS*sm/(cR+eps)
//   gaR  = dDot K,  gcR = -sum_i dS*S/(cR+eps)
//   dK  += sm*round(r)^T gaL + dDot^T aR,   dV += round(r)^T gY
// With U = round(Q aL^T) - cL, Lp = softmax_k(U), Lm = mask_q*Lp, cR = sum_l Lm,
// aR = round(Lm)^T Q                                         (L step, :26-35)
//   gLm  = gcR + gaR Q^T,  dU = Lp*(mask_q*gLm - sum_k mask_q*gLm*Lp)
//   dQ  += round(Lm) gaR + dU aL,   gaL = dU^T Q,   gcL = -sum_l dU
// With Lz = softmax_k(U), out = round(Lz) Y                   (Z step, :55-62)
//   gLz  = dout Y^T,  dU = Lz*(gLz - sum_k gLz Lz),  gY = round(Lz)^T dout
//   dQ  += dU aL,   gaL = dU^T Q,   gcL = -sum_l dU
// A workgroup owns every row it accumulates into (dQ rows (l,j) for fixed j in
// the L / Z stages, rows of block k in the R stage), so the sums are plain
// read-modify-writes in a fixed order: the result is reproducible bit for bit.
#include "ma_generic_dev.h"

namespace ma {
namespace {

template <class T>
__device__ __forceinline__ float dot_f32_rows(const float* g, const T* x, int D) {
    if (x == nullptr) return 0.f;
    float acc = 0.f;
#pragma unroll 4
    for (int d = 0; d < D; ++d) acc = fmaf(g[d], to_f(x[d]), acc);
    return acc;
}

__device__ __forceinline__ void decode_ehx(int X, int H, int& e, int& h, int& x) {
    int w = blockIdx.x;
    x = w % X; w /= X;
    h = w % H;
    e = w / H;
}

// softmax over the M entries of every row of U[rows][M], in place
__device__ __forceinline__ void softmax_rows(float* U, int rows, int M) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int ll = wave; ll < rows; ll += kWaves) {
        float* Ul = U + ll * M;
        float mx = -INFINITY;
        for (int k = lane; k < M; k += 64) mx = fmaxf(mx, Ul[k]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int k = lane; k < M; k += 64) {
            const float p = expf(Ul[k] - mx);
            Ul[k] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        for (int k = lane; k < M; k += 64) Ul[k] = Ul[k] / sum;
    }
}

// G[ll][k] <- Lp[ll][k] * (G[ll][k] - sum_k' G[ll][k'] Lp[ll][k'])
__device__ __forceinline__ void softmax_rows_bwd(const float* Lp, float* G, int rows, int M) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int ll = wave; ll < rows; ll += kWaves) {
        float dot = 0.f;
        for (int k = lane; k < M; k += 64) dot = fmaf(G[ll * M + k], Lp[ll * M + k], dot);
        dot = wave_sum(dot);
        for (int k = lane; k < M; k += 64) G[ll * M + k] = Lp[ll * M + k] * (G[ll * M + k] - dot);
    }
}

// gaL[j,k,:] (+)= sum_ll dU[ll][k] Q[(l0+ll, j), :],  gcL[j,k] (+)= -sum_ll dU[ll][k],
// dq[(l0+ll, j), :] += sum_k dU[ll][k] aL[j,k,:]          (shared tail of the L and Z stages)
template <class TQ>
__device__ __forceinline__ void logits_bwd(const Problem& P, const BwdBuffers& G, const float* dU, int e, int h, int j, int l0,
                                           int rows, bool accumulate) {
    const int M = P.M, D = P.D, B = P.B;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long jm = (eh * B + j) * M;
    const TQ* aL = reinterpret_cast<const TQ*>(P.aL) + jm * D;
    for (int idx = threadIdx.x; idx < M * (D + 1); idx += kThreads) {
        const int k = idx / (D + 1), d = idx % (D + 1);
        if (d == D) {
            float acc = accumulate ? G.gcL[jm + k] : 0.f;
            for (int ll = 0; ll < rows; ++ll) acc -= dU[ll * M + k];
            G.gcL[jm + k] = acc;
        } else {
            float acc = accumulate ? G.gaL[(jm + k) * D + d] : 0.f;
            for (int ll = 0; ll < rows; ++ll) {
                const TQ* qr = tok_row<TQ>(P.q, P.qs, e, h, (l0 + ll) * B + j - P.pad_off, P.N);
                if (qr != nullptr) acc = fmaf(dU[ll * M + k], to_f(qr[d]), acc);
            }
            G.gaL[(jm + k) * D + d] = acc;
        }
    }
    for (int idx = threadIdx.x; idx < rows * D; idx += kThreads) {
        const int ll = idx / D, d = idx % D;
        float acc = 0.f;
#pragma unroll 4
        for (int k = 0; k < M; ++k) acc = fmaf(dU[ll * M + k], to_f(aL[k * D + d]), acc);
        G.dq[(eh * M * B + (l0 + ll) * B + j) * D + d] += acc;
    }
}

// ---------------------------------------------------------------- Z stage
// One workgroup per (e,h,j), TL query blocks l at a time.  LDS: Lz[TL][M], G2[TL][M].
template <class TQ, class TV>
__global__ __launch_bounds__(kThreads) void z_bwd_kernel(Problem P, BwdBuffers G, int TL) {
    extern __shared__ float lds[];
    const int M = P.M, Dv = P.Dv, B = P.B;
    int e, h, j;
    decode_ehx(B, P.H, e, h, j);
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long jm = (eh * B + j) * M;
    float* Lz = lds;
    float* G2 = lds + TL * M;
    const TV* Y = reinterpret_cast<const TV*>(P.Y) + jm * Dv;
    for (int l0 = 0; l0 < M; l0 += TL) {
        const int rows = min(TL, M - l0);
        lz_logits<TQ>(P, Lz, e, h, j, l0, rows);
        __syncthreads();
        softmax_rows(Lz, rows, M);
        for (int idx = threadIdx.x; idx < rows * M; idx += kThreads) {   // gLz = dout Y^T
            const int ll = idx / M, k = idx % M;
            const TV* go = tok_row<TV>(G.dout, G.dos, e, h, (l0 + ll) * B + j - P.pad_off, P.N);
            float acc = 0.f;
            if (go != nullptr)
                for (int d = 0; d < Dv; ++d) acc = fmaf(to_f(go[d]), to_f(Y[k * static_cast<long long>(Dv) + d]), acc);
            G2[idx] = acc;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < M * Dv; idx += kThreads) {     // gY = round(Lz)^T dout
            const int k = idx / Dv, d = idx % Dv;
            float acc = l0 ? G.gY[(jm + k) * Dv + d] : 0.f;
            for (int ll = 0; ll < rows; ++ll) {
                const TV* go = tok_row<TV>(G.dout, G.dos, e, h, (l0 + ll) * B + j - P.pad_off, P.N);
                if (go != nullptr) acc = fmaf(round_to<TV>(Lz[ll * M + k]), to_f(go[d]), acc);
            }
            G.gY[(jm + k) * Dv + d] = acc;
        }
        softmax_rows_bwd(Lz, G2, rows, M);
        __syncthreads();
        logits_bwd<TQ>(P, G, G2, e, h, j, l0, rows, l0 != 0);
        __syncthreads();
    }
}

// ---------------------------------------------------------------- L stage
// One workgroup per (e,h,j), TL query blocks l at a time.  LDS: Lp[TL][M], G2[TL][M].
template <class TQ>
__global__ __launch_bounds__(kThreads) void l_bwd_kernel(Problem P, BwdBuffers G, int TL) {
    extern __shared__ float lds[];
    const int M = P.M, D = P.D, B = P.B;
    int e, h, j;
    decode_ehx(B, P.H, e, h, j);
    const long long eh = static_cast<long long>(e) * P.H + h;
    float* Lp = lds;
    float* G2 = lds + TL * M;
    for (int l0 = 0; l0 < M; l0 += TL) {
        const int rows = min(TL, M - l0);
        lz_logits<TQ>(P, Lp, e, h, j, l0, rows);
        __syncthreads();
        softmax_rows(Lp, rows, M);
        for (int idx = threadIdx.x; idx < rows * M; idx += kThreads) {   // mask_q * (gcR + gaR Q^T)
            const int ll = idx / M, k = idx % M;
            const int t = (l0 + ll) * B + j - P.pad_off;
            float g = 0.f;
            if (token_ok(P, e, t)) {
                const long long kj = (eh * M + k) * B + j;
                g = G.gcR[kj] + dot_f32_rows(G.gaR + kj * D, tok_row<TQ>(P.q, P.qs, e, h, t, P.N), D);
            }
            G2[idx] = g;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < rows * D; idx += kThreads) {   // dQ += round(Lm) gaR
            const int ll = idx / D, d = idx % D;
            const int t = (l0 + ll) * B + j - P.pad_off;
            if (!token_ok(P, e, t)) continue;
            float acc = 0.f;
            for (int k = 0; k < M; ++k) acc = fmaf(round_to<TQ>(Lp[ll * M + k]), G.gaR[((eh * M + k) * B + j) * D + d], acc);
            G.dq[(eh * M * B + (l0 + ll) * B + j) * D + d] += acc;
        }
        softmax_rows_bwd(Lp, G2, rows, M);
        __syncthreads();
        logits_bwd<TQ>(P, G, G2, e, h, j, l0, rows, l0 != 0);
        __syncthreads();
    }
}

// ---------------------------------------------------------------- R stage
// One workgroup per key block (e,h,k), TJ query rows j at a time.
// LDS: S[TJ][B] logits, R[TJ][B] probabilities, G2[TJ][B].
template <class TQ, class TV>
__global__ __launch_bounds__(kThreads) void r_bwd_kernel(Problem P, BwdBuffers G, int TJ, int first, int with_v) {
    extern __shared__ float lds[];
    const int B = P.B, M = P.M, D = P.D, Dv = P.Dv;
    int e, h, k;
    decode_ehx(M, P.H, e, h, k);
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aR = reinterpret_cast<const TQ*>(P.aR) + (eh * M + k) * B * D;
    const float* cR = P.cR + (eh * M + k) * B;
    float* S = lds;
    float* R = lds + TJ * B;
    float* G2 = lds + 2 * TJ * B;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float sm = P.sm_scale;
    for (int j0 = 0; j0 < B; j0 += TJ) {
        const int rows = min(TJ, B - j0);
        // forward again: logits and probabilities (ma_torch.py:11-18)
        for (int idx = threadIdx.x; idx < rows * B; idx += kThreads) {
            const int jj = idx / B, i = idx % B, j = j0 + jj;
            const TQ* x = first ? tok_row<TQ>(P.q, P.qs, e, h, k * B + j - P.pad_off, P.N) : aR + j * D;
            const int ti = k * B + i - P.pad_off;
            float s = sm * round_to<TQ>(dot_rows(x, tok_row<TQ>(P.k, P.ks, e, h, ti, P.N), D));
            s = s / ((first ? 1.0f : cR[j]) + P.eps);
            if (!token_ok(P, e, ti)) s = -INFINITY;
            S[idx] = s;
        }
        __syncthreads();
        for (int jj = wave; jj < rows; jj += kWaves) {
            float mx = -INFINITY;
            for (int i = lane; i < B; i += 64) mx = fmaxf(mx, S[jj * B + i]);
            mx = fmaxf(wave_max(mx), P.eps);
            float sum = 0.f;
            for (int i = lane; i < B; i += 64) {
                const float p = expf(S[jj * B + i] - mx);
                R[jj * B + i] = p;
                sum += p;
            }
            sum = wave_sum(sum) + P.eps;
            for (int i = lane; i < B; i += 64) {
                const float r = R[jj * B + i] / sum;
                G2[jj * B + i] = r >= kTiny ? 1.f : 0.f;   // the clamp passes the gradient where it did not act
                R[jj * B + i] = fmaxf(r, kTiny);
            }
        }
        __syncthreads();
        // g = gcL (log r + 1) + sm gaL K^T + gY V^T
        for (int idx = threadIdx.x; idx < rows * B; idx += kThreads) {
            const int jj = idx / B, i = idx % B, j = j0 + jj;
            float g = 0.f;
            if (G2[idx] != 0.f) {
                const long long jk = (eh * B + j) * M + k;
                const int ti = k * B + i - P.pad_off;
                g = G.gcL[jk] * (logf(R[idx]) + 1.0f);
                g = fmaf(sm, dot_f32_rows(G.gaL + jk * D, tok_row<TQ>(P.k, P.ks, e, h, ti, P.N), D), g);
                if (with_v) g += dot_f32_rows(G.gY + jk * Dv, tok_row<TV>(P.v, P.vs, e, h, ti, P.N), Dv);
            }
            G2[idx] = g;
        }
        __syncthreads();
        // dS = r (g - sum g r); gcR = -sum dS S / c; G2 <- dDot = dS sm / c
        for (int jj = wave; jj < rows; jj += kWaves) {
            const int j = j0 + jj;
            float dot = 0.f;
            for (int i = lane; i < B; i += 64) dot = fmaf(G2[jj * B + i], R[jj * B + i], dot);
            dot = wave_sum(dot);
            const float c = (first ? 1.0f : cR[j]) + P.eps;
            float gc = 0.f;
            for (int i = lane; i < B; i += 64) {
                const float s = S[jj * B + i];
                const float ds = s == -INFINITY ? 0.f : R[jj * B + i] * (G2[jj * B + i] - dot);
                if (s != -INFINITY) gc = fmaf(-ds, s / c, gc);
                G2[jj * B + i] = ds * sm / c;
            }
            gc = wave_sum(gc);
            if (!first && lane == 0) G.gcR[(eh * M + k) * B + j] = gc;
        }
        __syncthreads();
        // gaR = dDot K (for the first step aR is q itself: the rows of block k of dq)
        for (int idx = threadIdx.x; idx < rows * D; idx += kThreads) {
            const int jj = idx / D, d = idx % D, j = j0 + jj;
            float acc = 0.f;
            for (int i = 0; i < B; ++i) {
                const TQ* kr = tok_row<TQ>(P.k, P.ks, e, h, k * B + i - P.pad_off, P.N);
                if (kr != nullptr) acc = fmaf(G2[jj * B + i], to_f(kr[d]), acc);
            }
            const long long row = (eh * M + k) * B + j;
            if (first) G.dq[row * D + d] += acc;
            else G.gaR[row * D + d] = acc;
        }
        // dK += sm round(r)^T gaL + dDot^T aR
        for (int idx = threadIdx.x; idx < B * D; idx += kThreads) {
            const int i = idx / D, d = idx % D;
            float acc = 0.f;
            for (int jj = 0; jj < rows; ++jj) {
                const int j = j0 + jj;
                const TQ* x = first ? tok_row<TQ>(P.q, P.qs, e, h, k * B + j - P.pad_off, P.N) : aR + j * D;
                acc = fmaf(sm * round_to<TQ>(R[jj * B + i]), G.gaL[((eh * B + j) * M + k) * D + d], acc);
                if (x != nullptr) acc = fmaf(G2[jj * B + i], to_f(x[d]), acc);
            }
            G.dk[((eh * M + k) * B + i) * D + d] += acc;
        }
        if (with_v) {   // dV += round(r)^T gY
            for (int idx = threadIdx.x; idx < B * Dv; idx += kThreads) {
                const int i = idx / Dv, d = idx % Dv;
                float acc = 0.f;
                for (int jj = 0; jj < rows; ++jj)
                    acc = fmaf(round_to<TV>(R[jj * B + i]), G.gY[((eh * B + (j0 + jj)) * M + k) * Dv + d], acc);
                G.dv[((eh * M + k) * B + i) * static_cast<long long>(Dv) + d] += acc;
            }
        }
        __syncthreads();
    }
}

__global__ void fill_zero_kernel(float* p, long long n) {
    for (long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; i < n;
         i += static_cast<long long>(gridDim.x) * blockDim.x)
        p[i] = 0.f;
}

// real rows of padded fp32 gradients (E,H,Np,W) -> the caller's tensors (dtype T, their strides); up to three
// tensors of one width and dtype per launch (blockIdx.y selects).
// VEC = 4: four consecutive columns per thread (W % 4 == 0, rows of dst aligned to four elements).
struct GradOut {
    const float* src[3];
    char* dst[3];
    long long st[3][3];
};
template <class T, int VEC>
__global__ void grad_out_kernel(GradOut g, int E, int H, int N, int Np, int W, int pad_off) {
    const float* src = g.src[blockIdx.y];
    char* dst = g.dst[blockIdx.y];
    const long long s0 = g.st[blockIdx.y][0], s1 = g.st[blockIdx.y][1], s2 = g.st[blockIdx.y][2];
    const int WV = W / VEC;
    const long long total = static_cast<long long>(E) * H * N * WV;
    for (long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; i < total;
         i += static_cast<long long>(gridDim.x) * blockDim.x) {
        const int d = static_cast<int>(i % WV) * VEC;
        long long w = i / WV;
        const int t = static_cast<int>(w % N); w /= N;
        const int h = static_cast<int>(w % H);
        const int e = static_cast<int>(w / H);
        const float* x = src + ((static_cast<long long>(e) * H + h) * Np + (t + pad_off)) * W + d;
        T* y = reinterpret_cast<T*>(dst) + e * s0 + h * s1 + t * s2 + d;
        if constexpr (VEC == 4) {
            struct alignas(4 * sizeof(T)) Quad { T v[4]; };
            const float4 v = *reinterpret_cast<const float4*>(x);
            *reinterpret_cast<Quad*>(y) = Quad{{from_f<T>(v.x), from_f<T>(v.y), from_f<T>(v.z), from_f<T>(v.w)}};
        } else {
            *y = from_f<T>(*x);
        }
    }
}

int blocks_for(long long n) { return static_cast<int>(n / 256 + 1 < 4096 ? n / 256 + 1 : 4096); }

}  // namespace

bool bwd_fits(const Problem& P) {
    return 2ull * P.M * sizeof(float) <= 48 * 1024 && 3ull * P.B * sizeof(float) <= 48 * 1024 &&
           static_cast<long long>(P.E) * P.H * P.B <= 0x7FFFFFFFLL && static_cast<long long>(P.E) * P.H * P.M <= 0x7FFFFFFFLL;
}

int launch_bwd_zero(float* p, long long n, hipStream_t s) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks_for(n)), dim3(256), 0, s, p, n);
    return static_cast<int>(hipGetLastError());
}

int launch_bwd_z(const Problem& P, const BwdBuffers& G, int dt_qk, int dt_v, hipStream_t s) {
    if (!G.fma_only && dt_qk == dt_v) {
        const int st = launch_bwd_lz_mfma(P, G, dt_qk, true, s);
        if (st != MA_ERR_UNSUPPORTED) return st;
    }
    const int TL = tile_rows(2 * P.M, P.M);
    const size_t lds = 2ull * TL * P.M * sizeof(float);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        return dispatch_qk(dt_v, [&](auto tv) {
            using TV = decltype(tv);
            hipLaunchKernelGGL((z_bwd_kernel<TQ, TV>), dim3(P.E * P.H * P.B), dim3(kThreads), lds, s, P, G, TL);
            return static_cast<int>(hipGetLastError());
        });
    });
}

int launch_bwd_l(const Problem& P, const BwdBuffers& G, int dt_qk, hipStream_t s) {
    if (!G.fma_only) {
        const int st = launch_bwd_lz_mfma(P, G, dt_qk, false, s);
        if (st != MA_ERR_UNSUPPORTED) return st;
    }
    const int TL = tile_rows(2 * P.M, P.M);
    const size_t lds = 2ull * TL * P.M * sizeof(float);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        hipLaunchKernelGGL((l_bwd_kernel<TQ>), dim3(P.E * P.H * P.B), dim3(kThreads), lds, s, P, G, TL);
        return static_cast<int>(hipGetLastError());
    });
}

int launch_bwd_r(const Problem& P, const BwdBuffers& G, int dt_qk, int dt_v, bool first, bool with_v, hipStream_t s) {
    if (!G.fma_only && dt_qk == dt_v) {
        const int st = launch_bwd_r_mfma(P, G, dt_qk, first, with_v, s);
        if (st != MA_ERR_UNSUPPORTED) return st;
    }
    const int TJ = tile_rows(3 * P.B, P.B);
    const size_t lds = 3ull * TJ * P.B * sizeof(float);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        return dispatch_qk(dt_v, [&](auto tv) {
            using TV = decltype(tv);
            hipLaunchKernelGGL((r_bwd_kernel<TQ, TV>), dim3(P.E * P.H * P.M), dim3(kThreads), lds, s, P, G, TJ, first ? 1 : 0,
                               with_v ? 1 : 0);
            return static_cast<int>(hipGetLastError());
        });
    });
}

// n (1..3) gradients of width W and dtype dt in one launch
int launch_bwd_out(int n, const float* const* src, void* const* dst, const long long (*st)[3], int dt, const Problem& P, int W,
                   hipStream_t s) {
    return dispatch_qk(dt, [&](auto t) {
        using T = decltype(t);
        GradOut g;
        bool vec = W % 4 == 0;
        for (int i = 0; i < 3; ++i) {
            const int j = i < n ? i : 0;
            g.src[i] = src[j];
            g.dst[i] = static_cast<char*>(dst[j]);
            for (int a = 0; a < 3; ++a) g.st[i][a] = st[j][a];
            vec = vec && reinterpret_cast<uintptr_t>(dst[j]) % (4 * sizeof(T)) == 0 && st[j][0] % 4 == 0 && st[j][1] % 4 == 0 &&
                  st[j][2] % 4 == 0 && reinterpret_cast<uintptr_t>(src[j]) % 16 == 0;
        }
        const long long total = static_cast<long long>(P.E) * P.H * P.N * (vec ? W / 4 : W);
        const dim3 grid(blocks_for(total), n);
        if (vec)
            hipLaunchKernelGGL((grad_out_kernel<T, 4>), grid, dim3(256), 0, s, g, P.E, P.H, P.N, P.M * P.B, W, P.pad_off);
        else
            hipLaunchKernelGGL((grad_out_kernel<T, 1>), grid, dim3(256), 0, s, g, P.E, P.H, P.N, P.M * P.B, W, P.pad_off);
        return static_cast<int>(hipGetLastError());
    });
}

}  // namespace ma
