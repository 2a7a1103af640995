// Backward stages for fp16 / bf16 operands with the probabilities and their
// gradients kept in MFMA accumulator registers, the way the forward stages keep
// theirs (ma_mfma.h): no fp32 matrices in LDS, no LDS round trip between the
// products.  Included by ma_bwd_mfma.h inside namespace ma::{anonymous}; the
// formulas are at the top of ma_bwd.hip, the reference is autograd through
// al_cl_ref / al_y_cl_ref (ma/ma_torch.py:10-23, :38-52).
//
// R stage: one workgroup per block problem (e, h, k), one wave per 16-row strip.  LDS holds
// five 16-bit operand tiles - K, V, X (aR rows, or Q rows in the first step),
// Ga = round(sm * gaL), Gy = round(gY) - and seven floats per row.  The products
// of the stage contract over three different indices, and a lane of the 16x16x32
// instruction can only feed a B operand from accumulators whose ROWS are the
// contraction index.  So the stage runs in two passes over the same logits:
//
//   pass 1, wave = strip of QUERY rows j (accumulator rows = keys i):
//     S = X K^T, Gg = Ga K^T + Gy V^T  ->  r, g, dS, dDot in registers;
//     gaR[j] = sum_i dDot[j,i] K[i]  (dDot straight into the B operand),
//     gcR[j]; the row statistics (max, 1 / sum, sum_i g r, ...) go to LDS.
//   pass 2, wave = strip of KEYS i (accumulator rows = query rows j):
//     the same two products with the operand roles swapped, r and dDot formed
//     again from the row statistics of pass 1;
//     dK[i] (+)= sum_j r[j,i] Ga[j] + dDot[j,i] X[j],  dV[i] = sum_j r[j,i] Gy[j].
//
// The recomputation costs four more small products on matrix pipes that are
// otherwise idle and the softmax arithmetic a second time; it saves three fp32
// B x B matrices in LDS (the tiles of a 64-row block take 46 KB instead of 150 KB,
// so three workgroups share a compute unit) and every pass over them.
// Rounding points are those of the LDS kernels: logits rounded to the operand
// dtype, probabilities, dDot, sm * gaL and gY rounded to it as operands.

template <class T, int DT, int NWT>
struct RBwdReg {
    using Gm = mfma::Geom<DT>;
    static constexpr int ROWS = 16 * NWT, LD = Gm::LD, KS = Gm::KS, COLS = Gm::COLS, TILE = ROWS * LD;
    static constexpr int kStats = 7;   // kok, cj, gcl, mx, inv, lg1, dot
    static constexpr size_t kLds = 5 * static_cast<size_t>(TILE) * sizeof(T) + kStats * ROWS * sizeof(float);
};


// A lane's 4*DT results of one row as 16-bit elements at dst (the row's first element).  Tiles 2p and 2p+1
// hold 8 consecutive columns (mfma::chunk_col): they go out as ONE 16-byte piece where the row allows it (D a
// multiple of 8, the piece 16-byte aligned), so that the four lane groups of a row write 64 contiguous bytes
// with one instruction; else, and for the last tile of an odd DT, as 8-byte pieces.
template <class T, int DT>
__device__ __forceinline__ void store_row16(T* dst, int D, const f32x4 (&O)[DT], int q) {
    typedef typename mfma::Ops<T>::v4 V4;
    const bool wide = D % 8 == 0 && (reinterpret_cast<unsigned long long>(dst) & 15ull) == 0;
#pragma unroll
    for (int p = 0; p < DT / 2; ++p) {
        const int d0 = mfma::chunk_col<DT>(q, 2 * p);   // d0 + 4 == chunk_col(q, 2 * p + 1)
        const V4 a = {from_f<T>(O[2 * p][0]), from_f<T>(O[2 * p][1]), from_f<T>(O[2 * p][2]), from_f<T>(O[2 * p][3])};
        const V4 b = {from_f<T>(O[2 * p + 1][0]), from_f<T>(O[2 * p + 1][1]), from_f<T>(O[2 * p + 1][2]), from_f<T>(O[2 * p + 1][3])};
        if (wide) {
            if (d0 < D) {
                const mfma::u32x2 lo = __builtin_bit_cast(mfma::u32x2, a), hi = __builtin_bit_cast(mfma::u32x2, b);
                *reinterpret_cast<mfma::u32x4*>(dst + d0) = mfma::u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
        } else {
            if (d0 < D) *reinterpret_cast<V4*>(dst + d0) = a;
            if (d0 + 4 < D) *reinterpret_cast<V4*>(dst + d0 + 4) = b;
        }
    }
    if (DT % 2 == 1) {
        const int d0 = mfma::chunk_col<DT>(q, DT - 1);
        const V4 a = {from_f<T>(O[DT - 1][0]), from_f<T>(O[DT - 1][1]), from_f<T>(O[DT - 1][2]), from_f<T>(O[DT - 1][3])};
        if (d0 < D) *reinterpret_cast<V4*>(dst + d0) = a;
    }
}

// O[dt] += sum_w tile[w][4*DT*q + 4*dt + v] * P[w][lane column]   (gemm2 of ma_mfma.h, accumulating)
template <class T, int DT, int NWT>
__device__ __forceinline__ void gemm2_acc(f32x4 (&O)[DT], const T* tile, const typename mfma::Ops<T>::v8 (&pb)[(NWT + 1) / 2], int r, int q) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < (NWT + 1) / 2; ++g)
            O[dt] = mfma::Ops<T>::mma(mfma::lds_tr8<T, DT>(tile, 32 * g + 4 * q, 16, 2 * g + 1 < NWT, dt, r), pb[g], O[dt]);
}

// A ROWS x COLS tile of 16-bit rows in flight: issue() starts this thread's 16-byte loads into
// registers, commit() writes them to the LDS tile (scaled and rounded again where scale != 1).  All
// tiles of a stage are issued before the first is committed, so staging waits for ONE memory round
// trip.  For rows of whole 16-byte pieces at 16-byte aligned addresses (the caller checks).
template <class T, int NTH, int ROWS, int COLS, int LD>
struct Stage16 {
    static constexpr int CH = COLS / 8, CNT = (ROWS * CH + NTH - 1) / NTH;
    mfma::u32x4 v[CNT];
    template <class RowPtr>
    __device__ __forceinline__ void issue(RowPtr&& row_ptr, int D) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = static_cast<int>(threadIdx.x) + i * NTH;
            const int row = c / CH, ch = c % CH;
            const T* p = (ROWS * CH % NTH == 0 || c < ROWS * CH) ? row_ptr(row) : nullptr;
            v[i] = mfma::u32x4{0u, 0u, 0u, 0u};
            if (p != nullptr && 8 * ch < D) v[i] = *reinterpret_cast<const mfma::u32x4*>(p + 8 * ch);
        }
    }
    __device__ __forceinline__ void commit(T* tile, float scale) const {
        using V8 = typename mfma::Ops<T>::v8;
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int c = static_cast<int>(threadIdx.x) + i * NTH;
            if (ROWS * CH % NTH != 0 && c >= ROWS * CH) continue;
            mfma::u32x4 x = v[i];
            if (scale != 1.f) {
                V8 a = __builtin_bit_cast(V8, x);
#pragma unroll
                for (int u = 0; u < 8; ++u) a[u] = from_f<T>(scale * to_f(a[u]));
                x = __builtin_bit_cast(mfma::u32x4, a);
            }
            *reinterpret_cast<mfma::u32x4*>(tile + (c / CH) * LD + (c % CH) * 8) = x;
        }
    }
};
// rows of a (.., t, D) tensor view start on 16-byte boundaries
__device__ __forceinline__ bool rows16(const void* base, const long long* st) {
    return reinterpret_cast<uintptr_t>(base) % 16 == 0 && st[0] % 8 == 0 && st[1] % 8 == 0 && st[2] % 8 == 0;
}

template <class T, int DT, int NWT, bool S16>
__global__ __launch_bounds__(64 * NWT) void r_bwd_reg(Problem P, BwdBuffers G, int first, int with_v) {
    using mfma::lds_row8;
    using mfma::quad_rows_max;
    using mfma::quad_rows_sum;
    using RB = RBwdReg<T, DT, NWT>;
    using TG = typename std::conditional<S16, T, float>::type;
    using V8 = typename mfma::Ops<T>::v8;
    using V4 = typename mfma::Ops<T>::v4;
    using MM = mfma::Ops<T>;
    constexpr int NTH = 64 * NWT, ROWS = RB::ROWS, LD = RB::LD, KS = RB::KS, COLS = RB::COLS, TILE = RB::TILE;
    constexpr float kLog2e = mfma::kLog2e;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    T* Kt = reinterpret_cast<T*>(lds_raw);
    T* Vt = Kt + TILE;
    T* Xt = Vt + TILE;
    T* Gat = Xt + TILE;
    T* Gyt = Gat + TILE;
    float* kok = reinterpret_cast<float*>(Gyt + TILE);
    float* cjs = kok + ROWS;
    float* gcls = cjs + ROWS;
    float* mxs = gcls + ROWS;
    float* invs = mxs + ROWS;
    float* lg1s = invs + ROWS;
    float* dots = lg1s + ROWS;

    const int B = P.B, M = P.M, D = P.D;
    int w = blockIdx.x;
    const int k = w % M; w /= M;
    const int h = w % P.H, e = w / P.H;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long blk = (eh * M + k) * B;   // first row of block k in the (E,H,M,B,.) arrays
    const float sm = P.sm_scale;
    const int wave = mfma::wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;

    // ---- operand tiles, zero-padded to the tile grid
    {
        const T* aR = reinterpret_cast<const T*>(P.aR) + blk * D;
        const TG* gaL = reinterpret_cast<const TG*>(G.gaL);
        const TG* gY = reinterpret_cast<const TG*>(G.gY);
        auto k_row = [=](int i) { return i < B ? tok_row<T>(P.k, P.ks, e, h, k * B + i - P.pad_off, P.N) : nullptr; };
        auto v_row = [=](int i) { return i < B ? tok_row<T>(P.v, P.vs, e, h, k * B + i - P.pad_off, P.N) : nullptr; };
        auto x_row = [=](int j) -> const T* {
            if (j >= B) return nullptr;
            return first ? tok_row<T>(P.q, P.qs, e, h, k * B + j - P.pad_off, P.N) : aR + j * D;
        };
        auto ga_row = [=](int j) { return j < B ? gaL + ((eh * B + j) * M + k) * D : nullptr; };
        auto gy_row = [=](int j) { return j < B ? gY + ((eh * B + j) * M + k) * D : nullptr; };
        // one memory round trip for all tiles where the rows allow 16-byte loads (uniform test)
        const bool fast = std::is_same<TG, T>::value && D % 8 == 0 && rows16(P.k, P.ks) && (!with_v || rows16(P.v, P.vs)) &&
                          (!first || rows16(P.q, P.qs));
        if (fast) {
            using St = Stage16<T, NTH, ROWS, COLS, LD>;
            St sk, sx, sa, sv, sy;
            sk.issue(k_row, D);
            sx.issue(x_row, D);
            sa.issue([=](int j) { return reinterpret_cast<const T*>(ga_row(j)); }, D);
            if (with_v) {
                sv.issue(v_row, D);
                sy.issue([=](int j) { return reinterpret_cast<const T*>(gy_row(j)); }, D);
            }
            sk.commit(Kt, 1.f);
            sx.commit(Xt, 1.f);
            sa.commit(Gat, sm);
            if (with_v) {
                sv.commit(Vt, 1.f);
                sy.commit(Gyt, 1.f);
            }
        } else {
            stage_rows<NTH, T, T>(Kt, LD, ROWS, COLS, D, 1.f, k_row);
            stage_rows<NTH, T, T>(Xt, LD, ROWS, COLS, D, 1.f, x_row);
            stage_rows<NTH, TG, T>(Gat, LD, ROWS, COLS, D, sm, ga_row);
            if (with_v) {
                stage_rows<NTH, T, T>(Vt, LD, ROWS, COLS, D, 1.f, v_row);
                stage_rows<NTH, TG, T>(Gyt, LD, ROWS, COLS, D, 1.f, gy_row);
            }
        }
        const float* cR = P.cR + blk;
        for (int i = threadIdx.x; i < ROWS; i += NTH) {
            const bool in = i < B;
            kok[i] = (in && token_ok(P, e, k * B + i - P.pad_off)) ? 1.f : 0.f;
            cjs[i] = 1.0f / (((first || !in) ? 1.0f : cR[i]) + P.eps);   // 1 / (cR + eps)
            gcls[i] = in ? G.gcL[(eh * B + i) * M + k] : 0.f;
        }
    }
    __syncthreads();

    // Probability r (clamped, ma_torch.py:18) and gradient g of one entry from its logit sv (-inf:
    // masked key), the gradient part gg = (sm gaL K^T + gY V^T) and its row's statistics.  g is 0
    // where the clamp acted; log r = (S - max) + log(1 / (sum + eps)).
    auto prob_grad = [](float sv, float gg, bool key_in, float gcl, float mx, float inv, float lg1, float& rc, float& g) {
        const float d = sv - mx;
        const float ru = __builtin_amdgcn_exp2f(kLog2e * d) * inv;
        rc = key_in ? fmaxf(ru, kTiny) : 0.f;
        g = (key_in && ru >= kTiny) ? fmaf(gcl, d + lg1, gg) : 0.f;
    };

    // a finished gradient row is rounded straight into the caller's tensor `which` (0 dq, 1 dk, 2 dv) at token t;
    // padding positions have no row there
    auto emit = [&](int which, int t, const f32x4 (&val)[DT]) {
        if (t < 0 || t >= P.N) return;
        T* y = reinterpret_cast<T*>(G.out[which]) + e * G.outs[which][0] + h * G.outs[which][1] + t * G.outs[which][2];
        store_row16<T, DT>(y, D, val, q);
    };

    // ---- pass 1: this wave's strip of query rows (accumulator rows = keys)
    {
        const int j = 16 * wave + r;
        const bool jv = j < B;
        V8 xb[KS], ga[KS], gy[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            xb[ks] = lds_row8<T>(Xt + j * LD + 32 * ks + 8 * q);
            ga[ks] = lds_row8<T>(Gat + j * LD + 32 * ks + 8 * q);
            if (with_v) gy[ks] = lds_row8<T>(Gyt + j * LD + 32 * ks + 8 * q);
        }
        const float cj = cjs[j], gcl = gcls[j];
        f32x4 S[NWT], Gg[NWT];
        float mx = -INFINITY;
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const V8 kr = lds_row8<T>(Kt + (16 * wt + r) * LD + 32 * ks + 8 * q);
                a = MM::mma(kr, xb[ks], a);
                g = MM::mma(kr, ga[ks], g);
                if (with_v) g = MM::mma(lds_row8<T>(Vt + (16 * wt + r) * LD + 32 * ks + 8 * q), gy[ks], g);
            }
            const f32x4 ok = *reinterpret_cast<const f32x4*>(kok + 16 * wt + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                a[v] = ok[v] != 0.f ? sm * round_to<T>(a[v]) * cj : -INFINITY;   // S, -inf for masked / padded keys
                mx = fmaxf(mx, a[v]);
            }
            S[wt] = a;
            Gg[wt] = g;
        }
        // row statistics: clamped maximum, 1 / (sum + eps)   (ma_torch.py:14-17)
        mx = fmaxf(quad_rows_max(mx), P.eps);
        float sum = 0.f;
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) sum += __builtin_amdgcn_exp2f(kLog2e * (S[wt][v] - mx));
        const float inv = mfma::rcp(quad_rows_sum(sum) + P.eps);
        const float lg1 = __logf(inv) + 1.0f;
        f32x4 Rc[NWT];
        float dot = 0.f;   // sum_i g r
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float rc, g;
                prob_grad(S[wt][v], Gg[wt][v], 16 * wt + 4 * q + v < B, gcl, mx, inv, lg1, rc, g);
                Rc[wt][v] = rc;
                Gg[wt][v] = g;
                dot = fmaf(g, rc, dot);
            }
        dot = quad_rows_sum(dot);
        // dS = r (g - dot), gcR = -sum_i dS S / (cR + eps), dDot = dS sm / (cR + eps)
        float gc = 0.f;
#pragma unroll
        for (int wt = 0; wt < NWT; ++wt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const bool live = S[wt][v] != -INFINITY;
                const float ds = live ? Rc[wt][v] * (Gg[wt][v] - dot) : 0.f;
                gc = live ? fmaf(-ds, S[wt][v] * cj, gc) : gc;
                Rc[wt][v] = ds * (sm * cj);
            }
        gc = quad_rows_sum(gc);
        if (q == 0) {
            mxs[j] = mx;
            invs[j] = inv;
            lg1s[j] = lg1;
            dots[j] = dot;
            if (!first && jv) G.gcR[blk + j] = gc;
        }
        // gaR[j] = sum_i dDot[j,i] K[i]   (first step: aR is q, the rows of block k of dq)
        V8 pb[(NWT + 1) / 2];
        mfma::pack_p<T, NWT>(pb, Rc);
        f32x4 O[DT];
        mfma::gemm2<T, DT, NWT>(O, Kt, pb, r, q);
        if (jv) {
            if (first) {   // dq is complete with this stage's part
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const int d0 = mfma::chunk_col<DT>(q, dt);
                    if (d0 >= D) continue;   // D is a multiple of 4 (checked by the launcher)
                    f32x4* dst = reinterpret_cast<f32x4*>(G.dq + (blk + j) * D + d0);
                    O[dt] += *dst;
                    if (!G.direct) *dst = O[dt];
                }
                if (G.direct) emit(0, k * B + j - P.pad_off, O);
            } else if (S16) {
                store_row16<T, DT>(reinterpret_cast<T*>(G.gaR) + (blk + j) * D, D, O, q);
            } else {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const int d0 = mfma::chunk_col<DT>(q, dt);
                    if (d0 < D) *reinterpret_cast<f32x4*>(G.gaR + (blk + j) * D + d0) = O[dt];
                }
            }
        }
    }
    __syncthreads();

    // ---- pass 2: this wave's strip of keys (accumulator rows = query rows)
    {
        const int i = 16 * wave + r;
        const bool key_in = i < B, key_ok = kok[i] != 0.f;
        V8 kb[KS], vb[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            kb[ks] = lds_row8<T>(Kt + i * LD + 32 * ks + 8 * q);
            if (with_v) vb[ks] = lds_row8<T>(Vt + i * LD + 32 * ks + 8 * q);
        }
        f32x4 PR[NWT], DD[NWT];
#pragma unroll
        for (int jt = 0; jt < NWT; ++jt) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a = MM::mma(lds_row8<T>(Xt + (16 * jt + r) * LD + 32 * ks + 8 * q), kb[ks], a);
                g = MM::mma(lds_row8<T>(Gat + (16 * jt + r) * LD + 32 * ks + 8 * q), kb[ks], g);
                if (with_v) g = MM::mma(lds_row8<T>(Gyt + (16 * jt + r) * LD + 32 * ks + 8 * q), vb[ks], g);
            }
            const int j0 = 16 * jt + 4 * q;
            const f32x4 cj4 = *reinterpret_cast<const f32x4*>(cjs + j0), gcl4 = *reinterpret_cast<const f32x4*>(gcls + j0);
            const f32x4 mx4 = *reinterpret_cast<const f32x4*>(mxs + j0), inv4 = *reinterpret_cast<const f32x4*>(invs + j0);
            const f32x4 lg4 = *reinterpret_cast<const f32x4*>(lg1s + j0), dot4 = *reinterpret_cast<const f32x4*>(dots + j0);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float sv = key_ok ? sm * round_to<T>(a[v]) * cj4[v] : -INFINITY;
                float rc, gv;
                prob_grad(sv, g[v], key_in, gcl4[v], mx4[v], inv4[v], lg4[v], rc, gv);
                PR[jt][v] = rc;
                DD[jt][v] = key_ok ? rc * (gv - dot4[v]) * (sm * cj4[v]) : 0.f;
            }
        }
        V8 pr[(NWT + 1) / 2], pd[(NWT + 1) / 2];
        mfma::pack_p<T, NWT>(pr, PR);
        mfma::pack_p<T, NWT>(pd, DD);
        // dK[i] += sum_j round(r)[j,i] (sm gaL)[j] + dDot[j,i] X[j]
        f32x4 O[DT];
        mfma::gemm2<T, DT, NWT>(O, Gat, pr, r, q);
        gemm2_acc<T, DT, NWT>(O, Xt, pd, r, q);
        if (key_in) {
            const bool done = first && G.direct;   // dk is complete: it goes to the caller's tensor
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d0 = mfma::chunk_col<DT>(q, dt);
                if (d0 >= D) continue;
                f32x4* dst = reinterpret_cast<f32x4*>(G.dk + (blk + i) * D + d0);
                // the stage that also forms dv is the first R stage of a backward pass: it starts dk's sums
                if (!with_v) O[dt] += *dst;
                if (!done) *dst = O[dt];
            }
            if (done) emit(1, k * B + i - P.pad_off, O);
        }
        if (with_v) {   // dV[i] = sum_j round(r)[j,i] gY[j]: this stage is dv's only writer
            mfma::gemm2<T, DT, NWT>(O, Gyt, pr, r, q);
            if (key_in) {
                if (G.direct) {
                    emit(2, k * B + i - P.pad_off, O);
                } else {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const int d0 = mfma::chunk_col<DT>(q, dt);
                        if (d0 < D) *reinterpret_cast<f32x4*>(G.dv + (blk + i) * D + d0) = O[dt];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- L and Z stages
// The same scheme for one in-block position j (e, h, j): an M x M problem over query blocks l and
// key blocks k (formulas at the top of ma_bwd.hip; reference: autograd through ar_cr_ref and z_ref,
// ma/ma_torch.py:26-35, :55-62).  LDS: aL_j, W (Z: Y_j; L: round(gaR_j)), the Q rows (l, j), in the
// Z stage the dout rows (l, j), and six floats per row.
//   pass 1, wave = strip of query blocks l (accumulator rows = key blocks k): U, g -> p, dU;
//     dq[(l,j)] (+)= sum_k dU[l,k] aL[j,k]  (L: + round(mask_q p)[l,k] gaR[k,j]); row statistics to LDS.
//   pass 2, wave = strip of key blocks k (accumulator rows = query blocks l): p, dU again;
//     gaL[j,k] = sum_l dU[l,k] Q[l],  gcL[j,k] = -sum_l dU[l,k],  Z: gY[j,k] = sum_l round(p)[l,k] dout[l].
template <class T, int DT, int NWT, bool kZ>
struct LzBwdReg {
    using Gm = mfma::Geom<DT>;
    static constexpr int ROWS = 16 * NWT, LD = Gm::LD, TILE = ROWS * LD;
    static constexpr size_t kLds = (kZ ? 4 : 3) * static_cast<size_t>(TILE) * sizeof(T) + 6 * ROWS * sizeof(float);
};

template <class T, int DT, int NWT, bool kZ, bool S16>
__global__ __launch_bounds__(64 * NWT) void lz_bwd_reg(Problem P, BwdBuffers G) {
    using mfma::lds_row8;
    using mfma::quad_rows_max;
    using mfma::quad_rows_sum;
    using LB = LzBwdReg<T, DT, NWT, kZ>;
    using TG = typename std::conditional<S16, T, float>::type;
    using V8 = typename mfma::Ops<T>::v8;
    using V4 = typename mfma::Ops<T>::v4;
    using MM = mfma::Ops<T>;
    constexpr int NTH = 64 * NWT, ROWS = LB::ROWS, LD = LB::LD, KS = mfma::Geom<DT>::KS, COLS = mfma::Geom<DT>::COLS, TILE = LB::TILE;
    constexpr float kLog2e = mfma::kLog2e;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    T* aLt = reinterpret_cast<T*>(lds_raw);
    T* Wt = aLt + TILE;
    T* Qt = Wt + TILE;
    T* dOt = Qt + TILE;   // Z stage only
    float* cl = reinterpret_cast<float*>(Qt + (kZ ? 2 : 1) * TILE);
    float* cw = cl + ROWS;
    float* qok = cw + ROWS;
    float* mxs = qok + ROWS;
    float* invs = mxs + ROWS;
    float* dots = invs + ROWS;

    const int M = P.M, D = P.D, B = P.B;
    int w = blockIdx.x;
    const int j = w % B; w /= B;
    const int h = w % P.H, e = w / P.H;
    const long long eh = static_cast<long long>(e) * P.H + h;
    const long long jm = (eh * B + j) * M;   // first row of position j in the (E,H,B,M,.) arrays
    const int wave = mfma::wave_id(), lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;

    {
        const T* aL = reinterpret_cast<const T*>(P.aL) + jm * D;
        const T* Y = reinterpret_cast<const T*>(P.Y) + jm * D;
        const TG* gaR = reinterpret_cast<const TG*>(G.gaR);
        auto aL_row = [=](int k) { return k < M ? aL + k * D : nullptr; };
        auto y_row = [=](int k) { return k < M ? Y + k * D : nullptr; };
        auto gar_row = [=](int k) { return k < M ? gaR + ((eh * M + k) * B + j) * D : nullptr; };
        auto q_row = [=](int l) { return l < M ? tok_row<T>(P.q, P.qs, e, h, l * B + j - P.pad_off, P.N) : nullptr; };
        auto do_row = [=](int l) { return l < M ? tok_row<T>(G.dout, G.dos, e, h, l * B + j - P.pad_off, P.N) : nullptr; };
        const bool fast = (kZ || std::is_same<TG, T>::value) && D % 8 == 0 && rows16(P.q, P.qs) && (!kZ || rows16(G.dout, G.dos));
        if (fast) {
            using St = Stage16<T, NTH, ROWS, COLS, LD>;
            St sa, sq, sw, so;
            sa.issue(aL_row, D);
            sq.issue(q_row, D);
            if (kZ) {
                sw.issue(y_row, D);
                so.issue(do_row, D);
            } else {
                sw.issue([=](int k) { return reinterpret_cast<const T*>(gar_row(k)); }, D);
            }
            sa.commit(aLt, 1.f);
            sq.commit(Qt, 1.f);
            sw.commit(Wt, 1.f);
            if (kZ) so.commit(dOt, 1.f);
        } else {
            stage_rows<NTH, T, T>(aLt, LD, ROWS, COLS, D, 1.f, aL_row);
            stage_rows<NTH, T, T>(Qt, LD, ROWS, COLS, D, 1.f, q_row);
            if (kZ) {
                stage_rows<NTH, T, T>(Wt, LD, ROWS, COLS, D, 1.f, y_row);
                stage_rows<NTH, T, T>(dOt, LD, ROWS, COLS, D, 1.f, do_row);
            } else {
                stage_rows<NTH, TG, T>(Wt, LD, ROWS, COLS, D, 1.f, gar_row);
            }
        }
        for (int i = threadIdx.x; i < ROWS; i += NTH) {
            cl[i] = i < M ? P.cL[jm + i] : 0.f;
            cw[i] = (!kZ && i < M) ? G.gcR[(eh * M + i) * B + j] : 0.f;
            qok[i] = (i < M && token_ok(P, e, i * B + j - P.pad_off)) ? 1.f : 0.f;
        }
    }
    __syncthreads();

    // ---- pass 1: this wave's strip of query blocks (accumulator rows = key blocks)
    {
        const int l = 16 * wave + r;
        V8 xq[KS], xo[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            xq[ks] = lds_row8<T>(Qt + l * LD + 32 * ks + 8 * q);
            if (kZ) xo[ks] = lds_row8<T>(dOt + l * LD + 32 * ks + 8 * q);
        }
        const float keep = kZ ? 1.f : qok[l];
        f32x4 U[NWT], Gg[NWT];
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a = MM::mma(lds_row8<T>(aLt + (16 * kt + r) * LD + 32 * ks + 8 * q), xq[ks], a);
                g = MM::mma(lds_row8<T>(Wt + (16 * kt + r) * LD + 32 * ks + 8 * q), kZ ? xo[ks] : xq[ks], g);
            }
            const f32x4 cl4 = *reinterpret_cast<const f32x4*>(cl + 16 * kt + 4 * q), cw4 = *reinterpret_cast<const f32x4*>(cw + 16 * kt + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const bool kin = 16 * kt + 4 * q + v < M;
                a[v] = kin ? round_to<T>(a[v]) - cl4[v] : -INFINITY;   // U, -inf beyond the M key blocks
                if (!kZ) g[v] = kin ? keep * (g[v] + cw4[v]) : 0.f;     // gLm = mask_q (Q gaR^T + gcR)
                mx = fmaxf(mx, a[v]);
            }
            U[kt] = a;
            Gg[kt] = g;
        }
        mx = quad_rows_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                U[kt][v] = __builtin_amdgcn_exp2f(kLog2e * (U[kt][v] - mx));
                sum += U[kt][v];
            }
        const float inv = mfma::rcp(quad_rows_sum(sum));
        float dot = 0.f;
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                U[kt][v] *= inv;
                dot = fmaf(Gg[kt][v], U[kt][v], dot);
            }
        dot = quad_rows_sum(dot);
        if (q == 0) {
            mxs[l] = mx;
            invs[l] = inv;
            dots[l] = dot;
        }
#pragma unroll
        for (int kt = 0; kt < NWT; ++kt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                Gg[kt][v] = U[kt][v] * (Gg[kt][v] - dot);   // dU
                if (!kZ) U[kt][v] *= keep;                  // Lm = mask_q Lp
            }
        // dq rows (l, j) (+)= dU aL  (L: + round(Lm) gaR)
        V8 pd[(NWT + 1) / 2];
        mfma::pack_p<T, NWT>(pd, Gg);
        f32x4 O[DT];
        mfma::gemm2<T, DT, NWT>(O, aLt, pd, r, q);
        if (!kZ) {
            V8 pp[(NWT + 1) / 2];
            mfma::pack_p<T, NWT>(pp, U);
            gemm2_acc<T, DT, NWT>(O, Wt, pp, r, q);
        }
        if (l < M) {
            float* row = G.dq + ((eh * M + l) * B + j) * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d0 = mfma::chunk_col<DT>(q, dt);
                if (d0 >= D) continue;
                f32x4* dst = reinterpret_cast<f32x4*>(row + d0);
                // the Z stage runs first and every dq row belongs to one workgroup: it is written, not added to
                *dst = kZ ? O[dt] : *dst + O[dt];
            }
        }
    }
    __syncthreads();

    // ---- pass 2: this wave's strip of key blocks (accumulator rows = query blocks)
    {
        const int k = 16 * wave + r;
        const bool kin = k < M;
        V8 ak[KS], wk[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            ak[ks] = lds_row8<T>(aLt + k * LD + 32 * ks + 8 * q);
            wk[ks] = lds_row8<T>(Wt + k * LD + 32 * ks + 8 * q);
        }
        const float clk = cl[k], cwk = cw[k];
        f32x4 PR[NWT], DU[NWT];
        float gcl = 0.f;
#pragma unroll
        for (int lt = 0; lt < NWT; ++lt) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const V8 qr = lds_row8<T>(Qt + (16 * lt + r) * LD + 32 * ks + 8 * q);
                a = MM::mma(qr, ak[ks], a);
                if (kZ) g = MM::mma(lds_row8<T>(dOt + (16 * lt + r) * LD + 32 * ks + 8 * q), wk[ks], g);
                else g = MM::mma(qr, wk[ks], g);
            }
            const int l0 = 16 * lt + 4 * q;
            const f32x4 mx4 = *reinterpret_cast<const f32x4*>(mxs + l0), inv4 = *reinterpret_cast<const f32x4*>(invs + l0);
            const f32x4 dot4 = *reinterpret_cast<const f32x4*>(dots + l0), keep4 = *reinterpret_cast<const f32x4*>(qok + l0);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float u = kin ? round_to<T>(a[v]) - clk : -INFINITY;
                const float p = __builtin_amdgcn_exp2f(kLog2e * (u - mx4[v])) * inv4[v];
                const float gv = kZ ? g[v] : (kin ? keep4[v] * (g[v] + cwk) : 0.f);
                const float du = p * (gv - dot4[v]);
                PR[lt][v] = kZ ? p : keep4[v] * p;
                DU[lt][v] = du;
                gcl -= du;
            }
        }
        gcl = quad_rows_sum(gcl);
        if (q == 0 && kin) G.gcL[jm + k] = gcl;   // gcL[j,k] = -sum_l dU
        V8 pd[(NWT + 1) / 2];
        mfma::pack_p<T, NWT>(pd, DU);
        f32x4 O[DT];
        auto store_state = [&](float* base32) {   // row (j, k) of gaL / gY, in the operand dtype or fp32
            if (!kin) return;
            if (S16) {
                store_row16<T, DT>(reinterpret_cast<T*>(base32) + (jm + k) * D, D, O, q);
                return;
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d0 = mfma::chunk_col<DT>(q, dt);
                if (d0 < D) *reinterpret_cast<f32x4*>(base32 + (jm + k) * D + d0) = O[dt];
            }
        };
        mfma::gemm2<T, DT, NWT>(O, Qt, pd, r, q);   // gaL[j,k] = sum_l dU[l,k] Q[l]
        store_state(G.gaL);
        if (kZ) {   // gY[j,k] = sum_l round(Lz)[l,k] dout[l]
            V8 pp[(NWT + 1) / 2];
            mfma::pack_p<T, NWT>(pp, PR);
            mfma::gemm2<T, DT, NWT>(O, dOt, pp, r, q);
            store_state(G.gY);
        }
    }
}

template <class T>
int launch_lz_reg(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s) {
    if (P.Dv != P.D || P.D % 4 != 0 || P.D > 128 || P.M > 128) return static_cast<int>(MA_ERR_UNSUPPORTED);
    const long long grid = static_cast<long long>(P.E) * P.H * P.B;
    auto launch = [&](auto dt, auto nt) {
        constexpr int DT = decltype(dt)::value, NWT = decltype(nt)::value;
        auto go = [&](auto kernel, size_t lds) {
            const int attr = mfma::set_lds_limit(kernel, lds);
            if (attr) return attr;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * NWT), lds, s, P, G);
            return static_cast<int>(hipGetLastError());
        };
        constexpr size_t lz = LzBwdReg<T, DT, NWT, true>::kLds, ll = LzBwdReg<T, DT, NWT, false>::kLds;
        if (z) return G.state16 ? go(lz_bwd_reg<T, DT, NWT, true, true>, lz) : go(lz_bwd_reg<T, DT, NWT, true, false>, lz);
        return G.state16 ? go(lz_bwd_reg<T, DT, NWT, false, true>, ll) : go(lz_bwd_reg<T, DT, NWT, false, false>, ll);
    };
    auto by_rows = [&](auto dt) {
        if (P.M <= 16) return launch(dt, std::integral_constant<int, 1>{});
        if (P.M <= 32) return launch(dt, std::integral_constant<int, 2>{});
        if (P.M <= 64) return launch(dt, std::integral_constant<int, 4>{});
        return launch(dt, std::integral_constant<int, 8>{});
    };
    if (P.D <= 64) return by_rows(std::integral_constant<int, 4>{});
    if (P.D <= 80) return by_rows(std::integral_constant<int, 5>{});
    return by_rows(std::integral_constant<int, 8>{});
}

// The register kernel takes problems with Dv = D, D a multiple of 4 and at most 128, blocks of at
// most 128 rows, whose blocks are not split over workgroups; MA_ERR_UNSUPPORTED sends the caller on
// to the LDS kernels.
template <class T>
int launch_r_reg(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s) {
    if (P.Dv != P.D || P.D % 4 != 0 || P.D > 128 || P.B > 128) return static_cast<int>(MA_ERR_UNSUPPORTED);
    const long long grid = static_cast<long long>(P.E) * P.H * P.M;
    auto launch = [&](auto dt, auto nt) {
        constexpr int DT = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr size_t lds = RBwdReg<T, DT, NWT>::kLds;
        auto go = [&](auto kernel) {
            const int attr = mfma::set_lds_limit(kernel, lds);
            if (attr) return attr;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * NWT), lds, s, P, G, first ? 1 : 0, with_v ? 1 : 0);
            return static_cast<int>(hipGetLastError());
        };
        return G.state16 ? go(r_bwd_reg<T, DT, NWT, true>) : go(r_bwd_reg<T, DT, NWT, false>);
    };
    auto by_rows = [&](auto dt) {
        if (P.B <= 16) return launch(dt, std::integral_constant<int, 1>{});
        if (P.B <= 32) return launch(dt, std::integral_constant<int, 2>{});
        if (P.B <= 64) return launch(dt, std::integral_constant<int, 4>{});
        return launch(dt, std::integral_constant<int, 8>{});
    };
    if (P.D <= 64) return by_rows(std::integral_constant<int, 4>{});
    if (P.D <= 80) return by_rows(std::integral_constant<int, 5>{});
    return by_rows(std::integral_constant<int, 8>{});
}
