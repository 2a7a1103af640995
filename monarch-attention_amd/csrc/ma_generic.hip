// Generic stage kernels: plain fp32 FMA arithmetic, every dtype / shape /
// stride / mask the operator accepts.  They are the correctness backbone (the
// fp32 path with its 1e-5 bound, ragged and odd shapes, Dv != D, an fp32 V
// with 16-bit q/k) and the on-device cross-check for the MFMA kernels.
//
// Stage -> reference function:
//   r_step_kernel   al_cl_ref (ma/ma_torch.py:10-23) / al_y_cl_ref (:38-52)
//   l_stats_kernel + l_accum_kernel   ar_cr_ref (:26-35)
//   z_step_kernel   z_ref (:55-62) + the final slice (:106-108)
// The rounding points of the reference are kept: every matmul result is rounded
// to the operand dtype before the fp32 softmax math, probabilities are rounded
// to the operand dtype before the second matmul, and sm_scale is applied to aL
// after that rounding.
#include "ma_generic_dev.h"

namespace ma {
namespace {

// ---------------------------------------------------------------- R step
// One workgroup: TJ query rows j of one key block (e,h,m).  LDS: S[TJ][B].
template <class TQ, class TV>
__global__ __launch_bounds__(kThreads) void r_step_kernel(Problem P, int TJ, int first, int with_v) {
    extern __shared__ float lds[];
    const int B = P.B, M = P.M, D = P.D, Dv = P.Dv;
    const int jt_count = (B + TJ - 1) / TJ;
    int w = blockIdx.x;
    const int jt = w % jt_count; w /= jt_count;
    const int m = w % M; w /= M;
    const int h = w % P.H;
    const int e = w / P.H;
    const int j0 = jt * TJ;
    const int rows = min(TJ, B - j0);
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aR = reinterpret_cast<const TQ*>(P.aR) + (eh * M + m) * B * D;
    const float* cR = P.cR + (eh * M + m) * B;

    // logits (ma_torch.py:11-13)
    for (int idx = threadIdx.x; idx < rows * B; idx += kThreads) {
        const int jj = idx / B, i = idx % B, j = j0 + jj;
        const TQ* x = first ? tok_row<TQ>(P.q, P.qs, e, h, m * B + j - P.pad_off, P.N) : aR + j * D;
        const int ti = m * B + i - P.pad_off;
        const TQ* kr = tok_row<TQ>(P.k, P.ks, e, h, ti, P.N);
        float s = P.sm_scale * round_to<TQ>(dot_rows(x, kr, D));
        const float c = first ? 1.0f : cR[j];
        s = s / (c + P.eps);
        if (!token_ok(P, e, ti)) s = -INFINITY;
        lds[jj * B + i] = s;
    }
    __syncthreads();

    // clamped-max softmax, tiny clamp, cL = sum r log r (ma_torch.py:14-20)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int jj = wave; jj < rows; jj += kWaves) {
        float* S = lds + jj * B;
        float mx = -INFINITY;
        for (int i = lane; i < B; i += 64) mx = fmaxf(mx, S[i]);
        mx = fmaxf(wave_max(mx), P.eps);
        float sum = 0.f;
        for (int i = lane; i < B; i += 64) {
            const float p = expf(S[i] - mx);
            S[i] = p;
            sum += p;
        }
        sum = wave_sum(sum) + P.eps;
        float ent = 0.f;
        for (int i = lane; i < B; i += 64) {
            const float r = fmaxf(S[i] / sum, kTiny);
            S[i] = r;
            ent += r * logf(r);
        }
        ent = wave_sum(ent);
        if (lane == 0) P.cL[(eh * B + (j0 + jj)) * M + m] = ent;
    }
    __syncthreads();

    // aL = sm_scale * round(R) K, Y = round(R) V  (ma_torch.py:21, :49-50)
    TQ* aL = reinterpret_cast<TQ*>(P.aL);
    for (int idx = threadIdx.x; idx < rows * D; idx += kThreads) {
        const int jj = idx / D, d = idx % D;
        const float* S = lds + jj * B;
        const float acc = weighted_column<TQ>(S, 1, P.k, P.ks, e, h, m * B - P.pad_off, 1, B, P.N, d);
        aL[((eh * B + (j0 + jj)) * M + m) * D + d] = from_f<TQ>(P.sm_scale * round_to<TQ>(acc));
    }
    if (with_v) {
        TV* Y = reinterpret_cast<TV*>(P.Y);
        for (int idx = threadIdx.x; idx < rows * Dv; idx += kThreads) {
            const int jj = idx / Dv, d = idx % Dv;
            const float* S = lds + jj * B;
            const float acc = weighted_column<TV>(S, 1, P.v, P.vs, e, h, m * B - P.pad_off, 1, B, P.N, d);
            Y[((eh * B + (j0 + jj)) * M + m) * static_cast<long long>(Dv) + d] = from_f<TV>(acc);
        }
    }
}

// L step, pass 1: softmax statistics over key blocks k for every query block l.
template <class TQ>
__global__ __launch_bounds__(kThreads) void l_stats_kernel(Problem P, int TL) {
    extern __shared__ float lds[];
    const int M = P.M;
    int e, h, j, lt;
    decode_bj(P, (M + TL - 1) / TL, e, h, j, lt);
    const int l0 = lt * TL, rows = min(TL, M - l0);
    lz_logits<TQ>(P, lds, e, h, j, l0, rows);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long eh = static_cast<long long>(e) * P.H + h;
    for (int ll = wave; ll < rows; ll += kWaves) {
        const float* U = lds + ll * M;
        float mx = -INFINITY;
        for (int k = lane; k < M; k += 64) mx = fmaxf(mx, U[k]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int k = lane; k < M; k += 64) sum += expf(U[k] - mx);
        sum = wave_sum(sum);
        if (lane == 0) {
            float* st = P.stats + ((eh * P.B + j) * M + (l0 + ll)) * 2;
            st[0] = mx;
            st[1] = sum;
        }
    }
}

// L step, pass 2: TK key blocks k of one (e,h,j): L[k,l] for all l, then
// cR[k,j] = sum_l L, aR[k,j,:] = round(L) Qt   (ma_torch.py:29-33).  LDS: Pl[M][TK].
template <class TQ>
__global__ __launch_bounds__(kThreads) void l_accum_kernel(Problem P, int TK) {
    extern __shared__ float lds[];
    const int M = P.M, D = P.D, B = P.B;
    int e, h, j, kt;
    decode_bj(P, (M + TK - 1) / TK, e, h, j, kt);
    const int k0 = kt * TK, cols = min(TK, M - k0);
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TQ* aL = reinterpret_cast<const TQ*>(P.aL) + (eh * B + j) * M * D;
    const float* cL = P.cL + (eh * B + j) * M;
    const float* st = P.stats + (eh * B + j) * M * 2;
    for (int idx = threadIdx.x; idx < M * cols; idx += kThreads) {
        const int l = idx / cols, kk = idx % cols;
        const int t = l * B + j - P.pad_off;
        const TQ* qr = tok_row<TQ>(P.q, P.qs, e, h, t, P.N);
        const float u = round_to<TQ>(dot_rows(qr, aL + (k0 + kk) * D, D)) - cL[k0 + kk];
        float p = expf(u - st[2 * l]) / st[2 * l + 1];
        if (!token_ok(P, e, t)) p = 0.f;  // query mask after the softmax (:30)
        lds[l * TK + kk] = p;
    }
    __syncthreads();
    TQ* aR = reinterpret_cast<TQ*>(P.aR);
    for (int idx = threadIdx.x; idx < cols * (D + 1); idx += kThreads) {
        const int kk = idx / (D + 1), d = idx % (D + 1);
        float acc = 0.f;
        if (d == D) {
            for (int l = 0; l < M; ++l) acc += lds[l * TK + kk];
            P.cR[(eh * M + (k0 + kk)) * B + j] = acc;
        } else {
            acc = weighted_column<TQ>(lds + kk, TK, P.q, P.qs, e, h, j - P.pad_off, B, M, P.N, d);
            aR[((eh * M + (k0 + kk)) * B + j) * D + d] = from_f<TQ>(acc);
        }
    }
}

// Z step: TL query blocks l of one (e,h,j); writes the real output rows.
template <class TQ, class TV>
__global__ __launch_bounds__(kThreads) void z_step_kernel(Problem P, int TL) {
    extern __shared__ float lds[];
    const int M = P.M, Dv = P.Dv, B = P.B;
    int e, h, j, lt;
    decode_bj(P, (M + TL - 1) / TL, e, h, j, lt);
    const int l0 = lt * TL, rows = min(TL, M - l0);
    lz_logits<TQ>(P, lds, e, h, j, l0, rows);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int ll = wave; ll < rows; ll += kWaves) {
        float* U = lds + ll * M;
        float mx = -INFINITY;
        for (int k = lane; k < M; k += 64) mx = fmaxf(mx, U[k]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int k = lane; k < M; k += 64) {
            const float p = expf(U[k] - mx);
            U[k] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        for (int k = lane; k < M; k += 64) U[k] = U[k] / sum;
    }
    __syncthreads();
    const long long eh = static_cast<long long>(e) * P.H + h;
    const TV* Y = reinterpret_cast<const TV*>(P.Y) + (eh * B + j) * M * static_cast<long long>(Dv);
    TV* out = reinterpret_cast<TV*>(P.out) + e * P.os[0] + h * P.os[1];
    for (int idx = threadIdx.x; idx < rows * Dv; idx += kThreads) {
        const int ll = idx / Dv, d = idx % Dv;
        const int t = (l0 + ll) * B + j - P.pad_off;
        if (t < 0 || t >= P.N) continue;  // padded query rows are dropped (:108)
        const float* U = lds + ll * M;
        float acc = 0.f;
#pragma unroll 4
        for (int k = 0; k < M; ++k) acc = fmaf(round_to<TV>(U[k]), to_f(Y[k * static_cast<long long>(Dv) + d]), acc);
        out[static_cast<long long>(t) * P.os[2] + d] = from_f<TV>(acc);
    }
}

// Dense attention matrix, written directly: row (l, j) of block-row j is
// A[(l,j), (k,i)] = Lz[j][l,k] * R[k][j,i], which is what the forward pass
// returns for an fp32 identity as v (ma/monarch_attention.py:61-66: Y is then R
// itself and the Z step's sum over k has one non-zero term).  Needs aL, cL of
// the last R step (and aR, cR of the last L step when T > 1) in the workspace.
// One workgroup: TL query blocks l of one (e,h,j).  LDS: R[M][B], then U[TL][M].
template <class TQ>
__global__ __launch_bounds__(kThreads) void matrix_kernel(Problem P, float* A, int TL, int first) {
    extern __shared__ float lds[];
    const int M = P.M, D = P.D, B = P.B;
    int e, h, j, lt;
    decode_bj(P, (M + TL - 1) / TL, e, h, j, lt);
    const int l0 = lt * TL, rows = min(TL, M - l0);
    const long long eh = static_cast<long long>(e) * P.H + h;
    float* R = lds;
    float* U = lds + M * B;

    // logits of query row j against every key block k (ma_torch.py:11-13)
    for (int idx = threadIdx.x; idx < M * B; idx += kThreads) {
        const int k = idx / B;
        const long long row = (eh * M + k) * B + j;
        const TQ* x = first ? tok_row<TQ>(P.q, P.qs, e, h, k * B + j - P.pad_off, P.N)
                            : reinterpret_cast<const TQ*>(P.aR) + row * D;
        const int ti = idx - P.pad_off;
        const TQ* kr = tok_row<TQ>(P.k, P.ks, e, h, ti, P.N);
        float s = P.sm_scale * round_to<TQ>(dot_rows(x, kr, D));
        const float c = first ? 1.0f : P.cR[row];
        s = s / (c + P.eps);
        if (!token_ok(P, e, ti)) s = -INFINITY;
        R[idx] = s;
    }
    lz_logits<TQ>(P, U, e, h, j, l0, rows);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int k = wave; k < M; k += kWaves) {  // ma_torch.py:14-18
        float* S = R + k * B;
        float mx = -INFINITY;
        for (int i = lane; i < B; i += 64) mx = fmaxf(mx, S[i]);
        mx = fmaxf(wave_max(mx), P.eps);
        float sum = 0.f;
        for (int i = lane; i < B; i += 64) {
            const float p = expf(S[i] - mx);
            S[i] = p;
            sum += p;
        }
        sum = wave_sum(sum) + P.eps;
        for (int i = lane; i < B; i += 64) S[i] = fmaxf(S[i] / sum, kTiny);
    }
    for (int ll = wave; ll < rows; ll += kWaves) {  // ma_torch.py:58-59
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
    __syncthreads();

    // A thread keeps its columns (four consecutive ones where rows of A allow 16-byte stores) and walks
    // the query rows: one LDS read and one store per row and chunk.
    typedef float f4 __attribute__((ext_vector_type(4)));
    const bool vec = B % 4 == 0 && P.N % 4 == 0 && P.pad_off % 4 == 0;   // chunks stay inside a block and rows of A are aligned
    if (vec) {
        for (int idx = 4 * threadIdx.x; idx < M * B; idx += 4 * kThreads) {
            const int tk = idx - P.pad_off;
            if (tk < 0 || tk >= P.N) continue;
            const f4 r4 = *reinterpret_cast<const f4*>(R + idx);
            const int k = idx / B;
            for (int ll = 0; ll < rows; ++ll) {
                const int tq = (l0 + ll) * B + j - P.pad_off;
                if (tq < 0 || tq >= P.N) continue;  // padded query rows are dropped
                *reinterpret_cast<f4*>(A + (eh * P.N + tq) * P.N + tk) = U[ll * M + k] * r4;
            }
        }
    } else {
        for (int idx = threadIdx.x; idx < M * B; idx += kThreads) {
            const int tk = idx - P.pad_off;
            if (tk < 0 || tk >= P.N) continue;
            const float r = R[idx];
            const int k = idx / B;
            for (int ll = 0; ll < rows; ++ll) {
                const int tq = (l0 + ll) * B + j - P.pad_off;
                if (tq < 0 || tq >= P.N) continue;
                A[(eh * P.N + tq) * P.N + tk] = U[ll * M + k] * r;
            }
        }
    }
}

}  // namespace

int launch_generic_r(const Problem& P, int dt_qk, int dt_v, bool first, bool with_v, hipStream_t s) {
    const int TJ = tile_rows(P.B, 16);
    const long long grid = static_cast<long long>(P.E) * P.H * P.M * ((P.B + TJ - 1) / TJ);
    const size_t lds = static_cast<size_t>(TJ) * P.B * sizeof(float);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        return dispatch_qk(dt_v, [&](auto tv) {
            using TV = decltype(tv);
            hipLaunchKernelGGL((r_step_kernel<TQ, TV>), dim3(grid), dim3(kThreads), lds, s, P, TJ, first ? 1 : 0,
                               with_v ? 1 : 0);
            return static_cast<int>(hipGetLastError());
        });
    });
}

int launch_generic_l(const Problem& P, int dt_qk, hipStream_t s) {
    const int TL = tile_rows(P.M, 16);
    const int TK = tile_rows(P.M, 16);
    const long long ehb = static_cast<long long>(P.E) * P.H * P.B;
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        hipLaunchKernelGGL((l_stats_kernel<TQ>), dim3(ehb * ((P.M + TL - 1) / TL)), dim3(kThreads),
                           static_cast<size_t>(TL) * P.M * sizeof(float), s, P, TL);
        int err = static_cast<int>(hipGetLastError());
        if (err) return err;
        hipLaunchKernelGGL((l_accum_kernel<TQ>), dim3(ehb * ((P.M + TK - 1) / TK)), dim3(kThreads),
                           static_cast<size_t>(TK) * P.M * sizeof(float), s, P, TK);
        return static_cast<int>(hipGetLastError());
    });
}

int launch_generic_z(const Problem& P, int dt_qk, int dt_v, hipStream_t s) {
    const int TL = tile_rows(P.M, 16);
    const long long grid = static_cast<long long>(P.E) * P.H * P.B * ((P.M + TL - 1) / TL);
    const size_t lds = static_cast<size_t>(TL) * P.M * sizeof(float);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        return dispatch_qk(dt_v, [&](auto tv) {
            using TV = decltype(tv);
            hipLaunchKernelGGL((z_step_kernel<TQ, TV>), dim3(grid), dim3(kThreads), lds, s, P, TL);
            return static_cast<int>(hipGetLastError());
        });
    });
}

bool generic_matrix_fits(const Problem& P) {
    const int TL = tile_rows(P.M, 64);
    const size_t lds = (static_cast<size_t>(P.M) * P.B + static_cast<size_t>(TL) * P.M) * sizeof(float);
    const long long grid = static_cast<long long>(P.E) * P.H * P.B * ((P.M + TL - 1) / TL);
    return lds <= kMatrixLdsBytes && grid <= 0x7FFFFFFFLL;
}

int launch_generic_matrix(const Problem& P, int dt_qk, float* A, bool first, hipStream_t s) {
    if (!generic_matrix_fits(P)) return MA_ERR_UNSUPPORTED;
    const int TL = tile_rows(P.M, 64);
    const size_t lds = (static_cast<size_t>(P.M) * P.B + static_cast<size_t>(TL) * P.M) * sizeof(float);
    const long long grid = static_cast<long long>(P.E) * P.H * P.B * ((P.M + TL - 1) / TL);
    return dispatch_qk(dt_qk, [&](auto tq) {
        using TQ = decltype(tq);
        const int rc = static_cast<int>(hipFuncSetAttribute(reinterpret_cast<const void*>(matrix_kernel<TQ>),
                                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                                            static_cast<int>(kMatrixLdsBytes)));
        if (rc) return rc;
        hipLaunchKernelGGL((matrix_kernel<TQ>), dim3(grid), dim3(kThreads), lds, s, P, A, TL, first ? 1 : 0);
        return static_cast<int>(hipGetLastError());
    });
}

}  // namespace ma
