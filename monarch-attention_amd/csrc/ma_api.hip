// C-ABI layer of libma_hip.so: argument validation, workspace layout, variant
// selection and the launch sequence of one forward call.  The sequence mirrors
// the driver of the reference, monarch_attention_torch (ma/ma_torch.py:100-108):
// (T-1) x [R step, L step], the R step that also forms Y, then the Z step.
#include "ma_common.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

// Scratch of ma_fwd_static: the per-call state (aR, cR, aL, cL, Y, stats, sync area) of callers that
// cannot bring a workspace of their own.  One copy per GPU, at that GPU's own address, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress: kernels get the
// address that call returns, never the name itself.
static __device__ __align__(256) unsigned char scratch[MA_STATIC_WORKSPACE_BYTES];

namespace ma {
namespace {

constexpr uint64_t kAlign = 256;

uint64_t align_up(uint64_t x) { return (x + kAlign - 1) / kAlign * kAlign; }
int elt_size(int dt) { return dt == MA_F32 ? 4 : 2; }
bool dtype_ok(int dt) { return dt == MA_F32 || dt == MA_F16 || dt == MA_BF16; }

// Shape-level validation: everything that can be checked without touching the
// device.  Pointers are checked separately (layout queries pass NULLs).
int check_shape(const ma_fwd_params* p) {
    if (p == nullptr) return MA_ERR_NULL;
    if (p->E < 1 || p->H < 1 || p->N < 1 || p->D < 1 || p->Dv < 1 || p->B < 1 || p->T < 1) return MA_ERR_SHAPE;
    if (!dtype_ok(p->dtype_qk) || !dtype_ok(p->dtype_v)) return MA_ERR_DTYPE;
    if (p->variant < MA_VARIANT_AUTO || p->variant > MA_VARIANT_CHAINED) return MA_ERR_VARIANT;
    if (p->flags & ~(MA_FLAG_SYNC_READY | MA_FLAG_TEST_NO_SPIN | MA_FLAG_DEVICE_EXCLUSIVE)) return MA_ERR_SHAPE;
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    const long long Np = M * p->B;
    // every launch grid and every in-kernel int index must stay inside int32
    const long long eh = static_cast<long long>(p->E) * p->H;
    if (Np > (1LL << 30) || eh > (1LL << 30)) return MA_ERR_SHAPE;
    if (eh * Np > (1LL << 31) - 1) return MA_ERR_SHAPE;
    if (M > 16384) return MA_ERR_UNSUPPORTED;  // LDS tile of the generic L step
    if (p->B > 12288) return MA_ERR_UNSUPPORTED;
    for (int i = 0; i < 3; ++i)
        if (p->q_stride[i] < 0 || p->k_stride[i] < 0 || p->v_stride[i] < 0 || p->out_stride[i] < 0) return MA_ERR_STRIDE;
    if (p->q_stride[2] < p->D || p->k_stride[2] < p->D) {
        if (p->N > 1) return MA_ERR_STRIDE;  // rows of q / k overlap
    }
    if (p->N > 1 && (p->v_stride[2] < p->Dv || p->out_stride[2] < p->Dv)) return MA_ERR_STRIDE;
    // inputs may be broadcast over batch / heads (stride 0); output slices must not coincide
    if ((p->E > 1 && p->out_stride[0] == 0) || (p->H > 1 && p->out_stride[1] == 0)) return MA_ERR_STRIDE;
    if (p->mask_stride[0] < 0 || p->mask_stride[1] < 0) return MA_ERR_STRIDE;
    if (p->mask_dtype < MA_MASK_U8 || p->mask_dtype > MA_MASK_F64) return MA_ERR_DTYPE;
    if (!(p->eps >= 0.0f)) return MA_ERR_SHAPE;
    return MA_OK;
}

int layout_of(const ma_fwd_params* p, ma_ws_layout* L) {
    const int st = check_shape(p);
    if (st != MA_OK) return st;
    const uint64_t M = (static_cast<uint64_t>(p->N) + p->B - 1) / p->B;
    const uint64_t rows = static_cast<uint64_t>(p->E) * p->H * M * p->B;  // E*H*Np
    const uint64_t sq = elt_size(p->dtype_qk), sv = elt_size(p->dtype_v);
    // the sync area comes first so that it stays put (and stays zero) when one
    // workspace serves calls of different shapes
    uint64_t off = 0;
    L->sync = off; off = align_up(off + kSyncAreaBytes);
    L->aR = off; off = align_up(off + rows * p->D * sq);
    L->cR = off; off = align_up(off + rows * 4);
    L->aL = off; off = align_up(off + rows * p->D * sq);
    L->cL = off; off = align_up(off + rows * 4);
    L->Y = off; off = align_up(off + rows * p->Dv * sv);
    L->stats = off; off = align_up(off + rows * 8);
    L->total = off;
    return MA_OK;
}

int check_buffers(const ma_fwd_params* p, const ma_ws_layout& L) {
    if (!p->q || !p->k || !p->v || !p->out) return MA_ERR_NULL;
    if (!p->workspace) return MA_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(p->workspace) % kAlign) return MA_ERR_WORKSPACE;
    if (p->workspace_bytes < L.total) return MA_ERR_WORKSPACE;
    const uintptr_t aq = elt_size(p->dtype_qk), av = elt_size(p->dtype_v);
    if (reinterpret_cast<uintptr_t>(p->q) % aq || reinterpret_cast<uintptr_t>(p->k) % aq ||
        reinterpret_cast<uintptr_t>(p->v) % av || reinterpret_cast<uintptr_t>(p->out) % av)
        return MA_ERR_STRIDE;
    if (reinterpret_cast<uintptr_t>(p->error_word) % 4) return MA_ERR_STRIDE;
    return MA_OK;
}

Problem make_problem(const ma_fwd_params* p, const ma_ws_layout& L) {
    Problem P;
    std::memset(&P, 0, sizeof(P));
    char* ws = static_cast<char*>(p->workspace);
    P.q = static_cast<const char*>(p->q);
    P.k = static_cast<const char*>(p->k);
    P.v = static_cast<const char*>(p->v);
    P.mask = static_cast<const uint8_t*>(p->mask);
    {
        static const int shift[8] = {0, 1, 2, 3, 1, 1, 2, 3};
        P.mask_shift = shift[p->mask_dtype];
        P.mask_float = p->mask_dtype >= MA_MASK_F16 ? 1 : 0;
    }
    P.out = static_cast<char*>(p->out);
    P.aR = ws + L.aR;
    P.cR = reinterpret_cast<float*>(ws + L.cR);
    P.aL = ws + L.aL;
    P.cL = reinterpret_cast<float*>(ws + L.cL);
    P.Y = ws + L.Y;
    P.stats = reinterpret_cast<float*>(ws + L.stats);
    P.sync = reinterpret_cast<unsigned*>(ws + L.sync);
    P.E = p->E; P.H = p->H; P.N = p->N; P.D = p->D; P.Dv = p->Dv; P.B = p->B; P.T = p->T;
    P.M = (p->N + p->B - 1) / p->B;
    P.pad_off = p->pre_pad ? P.M * p->B - p->N : 0;  // ma_torch.py:92
    for (int i = 0; i < 3; ++i) {
        P.qs[i] = p->q_stride[i]; P.ks[i] = p->k_stride[i];
        P.vs[i] = p->v_stride[i]; P.os[i] = p->out_stride[i];
    }
    P.ms[0] = p->mask_stride[0]; P.ms[1] = p->mask_stride[1];
    // sm_scale = 1/sqrt(D) as a Python float, used as an fp32 scalar (ma_torch.py:79)
    P.sm_scale = static_cast<float>(1.0 / std::sqrt(static_cast<double>(p->D)));
    P.eps = p->eps;
    P.test_no_spin = (p->flags & MA_FLAG_TEST_NO_SPIN) ? 1 : 0;
    P.host_error = p->error_word;
    P.pack_shift = 4;
    return P;
}

// What the MFMA kernels need: 16-bit operands of one dtype, Dv == D, 16-byte
// row chunks (D % 8 == 0 and every row start 16-byte aligned), and block
// problems that fit the register / LDS tiles (B, M <= 256, D <= 128: heads of up
// to 65536 tokens; the one-launch kernels stop at 128, see one_launch_tiles).
// Pointers may be NULL in a layout query; they are then not checked.
bool mfma_supported(const ma_fwd_params* p) {
    if (p->dtype_qk == MA_F32 || p->dtype_v != p->dtype_qk) return false;
    if (p->Dv != p->D || p->D % 8 != 0 || p->D > 128) return false;
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    if (p->B > 256 || M > 256) return false;
    for (int i = 0; i < 3; ++i)
        if (p->q_stride[i] % 8 || p->k_stride[i] % 8 || p->v_stride[i] % 8 || p->out_stride[i] % 8) return false;
    if (reinterpret_cast<uintptr_t>(p->q) % 16 || reinterpret_cast<uintptr_t>(p->k) % 16 ||
        reinterpret_cast<uintptr_t>(p->v) % 16 || reinterpret_cast<uintptr_t>(p->out) % 16)
        return false;
    // one (e, h) slice of every tensor and one head of state must fit a 32-bit byte offset
    const unsigned long long lim = 0xFFFF0000ull;
    const unsigned long long n1 = static_cast<unsigned long long>(p->N - 1), db = 2ull * p->D;
    if (n1 * p->q_stride[2] * 2 + db >= lim || n1 * p->k_stride[2] * 2 + db >= lim || n1 * p->v_stride[2] * 2 + db >= lim ||
        n1 * p->out_stride[2] * 2 + db >= lim || static_cast<unsigned long long>(M) * p->B * db >= lim ||
        n1 * static_cast<unsigned long long>(p->mask_stride[1]) * 8 >= lim)
        return false;
    return true;
}

// What the fp32 MFMA stage kernels need: fp32 q, k, v, Dv == D, 16-byte row chunks (D % 4 == 0,
// every row start 16-byte aligned), block problems within the tiles and the LDS.
bool mfma32_supported(const ma_fwd_params* p) {
    if (p->dtype_qk != MA_F32 || p->dtype_v != MA_F32) return false;
    if (p->Dv != p->D || p->D % 4 != 0 || p->D > 128) return false;
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    if (p->B > 128 || M > 128) return false;
    for (int i = 0; i < 3; ++i)
        if (p->q_stride[i] % 4 || p->k_stride[i] % 4 || p->v_stride[i] % 4 || p->out_stride[i] % 4) return false;
    if (reinterpret_cast<uintptr_t>(p->q) % 16 || reinterpret_cast<uintptr_t>(p->k) % 16 ||
        reinterpret_cast<uintptr_t>(p->v) % 16 || reinterpret_cast<uintptr_t>(p->out) % 16)
        return false;
    const unsigned long long lim = 0xFFFF0000ull;
    const unsigned long long n1 = static_cast<unsigned long long>(p->N - 1), db = 4ull * p->D;
    if (n1 * p->q_stride[2] * 4 + db >= lim || n1 * p->k_stride[2] * 4 + db >= lim || n1 * p->v_stride[2] * 4 + db >= lim ||
        n1 * p->out_stride[2] * 4 + db >= lim || static_cast<unsigned long long>(M) * p->B * db >= lim ||
        n1 * static_cast<unsigned long long>(p->mask_stride[1]) * 8 >= lim)
        return false;
    return mfma32_lds_needed(p->D, p->B, static_cast<int>(M)) <= 160 * 1024;
}

int run_resident(const Problem& P, int dtype_qk, bool dry_run, hipStream_t s) {
    if (dtype_qk == MA_F32) return launch_head32(P, dry_run, s);
    const bool h = dtype_qk == MA_F16;
    const int D = P.D;
    if (D <= 32) return h ? launch_resident_f16_d2(P, dry_run, s) : launch_resident_bf16_d2(P, dry_run, s);
    if (D <= 64) return h ? launch_resident_f16_d4(P, dry_run, s) : launch_resident_bf16_d4(P, dry_run, s);
    if (D <= 80) return h ? launch_resident_f16_d5(P, dry_run, s) : launch_resident_bf16_d5(P, dry_run, s);
    return h ? launch_resident_f16_d8(P, dry_run, s) : launch_resident_bf16_d8(P, dry_run, s);
}

// Does a head's state fit in LDS (the resident kernel's condition)?  one_tile: also count the form that
// keeps aL and aR in one tile and passes Y through the workspace.
bool resident_fits(const ma_fwd_params* p, bool one_tile) {
    Problem P;
    std::memset(&P, 0, sizeof(P));
    P.E = p->E; P.H = p->H; P.N = p->N; P.D = p->D; P.Dv = p->Dv; P.B = p->B; P.T = p->T;
    P.M = (p->N + p->B - 1) / p->B;
    P.one_tile_ok = one_tile ? 1 : 0;
    return run_resident(P, p->dtype_qk, true, nullptr) == MA_OK;
}

// Does the head fit in LDS whole (the head-resident forms of the resident kernel)?  forms = 1: Q, K, V and the
// state in four tiles; 2: that, or the state and one input tile at a time.  forms = 3, 4 ask something else: would a
// launch run a head-resident form (4: the four-tile one) in workgroups of 4 or 8 waves, several of them per compute
// unit (more short heads than compute units)?
bool resident_head_fits(const ma_fwd_params* p, int forms = 1) {
    Problem P;
    std::memset(&P, 0, sizeof(P));
    P.E = p->E; P.H = p->H; P.N = p->N; P.D = p->D; P.Dv = p->Dv; P.B = p->B; P.T = p->T;
    P.M = (p->N + p->B - 1) / p->B;
    P.resident_head_only = forms;
    return p->dtype_qk != MA_F32 && run_resident(P, p->dtype_qk, true, nullptr) == MA_OK;
}

// The fused, chained and resident kernels are built for block problems of at most 128 rows.
bool one_launch_tiles(const ma_fwd_params* p) {
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    return p->B <= 128 && M <= 128;
}

// Tasks (workgroups) of one phase of one head in the one-launch kernels: four waves per workgroup; a
// block problem of n rows takes min(ceil(n / 16), 4) waves, rounded up to a power of two.
long long phase_tasks(long long count, long long rows) {
    const long long strips = (rows + 15) / 16;
    const long long waves = strips <= 1 ? 1 : strips <= 2 ? 2 : 4;
    const long long per_wg = 4 / waves;
    return (count + per_wg - 1) / per_wg;
}

// Can the chained kernel take the problem?  Mirrors the launcher's limits: at most 128 tasks per
// head and phase, the heads' sync words (64-bit counters and release words of the 2T - 1 publishing
// phases, in whole 128-byte lines) fit their part of the sync area, the grid is a 31-bit count.
bool chain_fits(const ma_fwd_params* p) {
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    const long long tR = phase_tasks(M, p->B), tL = phase_tasks(p->B, M);
    const long long heads = static_cast<long long>(p->E) * p->H;
    const long long nph1 = 2ll * p->T - 1;
    const long long stride = (2 * nph1 + 2 + 31) / 32 * 32 + (nph1 + 31) / 32 * 32;
    if (!one_launch_tiles(p) || tR > 128 || tL > 128) return false;
    if (heads * stride > static_cast<long long>(kChainSyncBytes / 4)) return false;
    return 8 * ((heads + 7) / 8) * p->T * (tR + tL) <= 0x7fffffffLL;
}

// Few heads whose phases fill the device: every head gets a team with one workgroup per task (64
// or 128 of them per phase), the teams sit on one XCD each and all of them are on the device at
// once (256 CUs x 4 workgroups) - the fused kernel then runs each phase like a per-stage launch
// would, without the launch boundaries.  With a single step that pays for 16 heads of 64-row
// problems only (~4096 tokens: the metric workload); with more steps - the later exchanges of a team stay in its XCD's L2 -
// also for 128 blocks or 128-row blocks (8 heads of ~8192 tokens, 16 of ~4096 in 32- or 128-row
// blocks: 3 - 17 % ahead of the chained kernel), and for 8 heads also with head dims up to 80.
// Blocks or block counts of 65 .. 96 rows stay away: the team kernel runs them as 128-row problems.
bool fused_full_width(const ma_fwd_params* p) {
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    const long long heads = static_cast<long long>(p->E) * p->H;
    const bool steps = p->T > 1;
    const int rows = steps ? 128 : 64;
    if (p->B > rows || M > rows) return false;
    if ((M > 64 && M <= 96) || (p->B > 64 && p->B <= 96)) return false;
    if (p->D > (steps && heads == 8 ? 80 : 64)) return false;   // (head dims of 128: 4 - 50 % behind the chained kernel)
    const long long tR = phase_tasks(M, p->B), tL = phase_tasks(p->B, M);
    const long long widest = tR > tL ? tR : tL;
    if (!steps && heads * widest != 1024) return false;   // a single step: only with every workgroup slot of the device taken
    if (!steps && (tR < 60 || tL < 60)) return false;     // ... in both phases (16 heads of 3000 tokens: 47 R tasks, 12 % behind the chained kernel)
    return heads < 32 && heads % 8 == 0 && widest >= 64 && heads * widest <= 1024;
}

// The variant a problem resolves to.  AUTO: the MFMA kernels when the problem qualifies; among
// them what a sweep on MI355X says (fp16, E*H = 1 .. 384 heads, N = 256 .. 8192, blocks of 16 .. 128
// rows, T = 1, 2, 3, head dims 32, 64, 128; every variant that takes a shape timed: the choice
// below is within 0.0 - 0.7 % of the fastest variant in the geometric mean of each sweep and 18 %
// at worst):
//  * the resident kernel for heads that fit in LDS with their inputs (up to ~256 tokens at d = 64) in
//    blocks of at most 32 rows: from 128 heads on, and with more than one step for any number of
//    heads in 16-row blocks; with two or three state tiles for blocks of at most 16 rows from 128
//    heads on; in its one-tile form
//    (up to ~512 tokens) for problems of one or two strips when the head count fills the
//    device's 256 one-per-CU workgroups to three quarters or more in its last pass (192 heads:
//    0.95 of the chained kernel's time with 0.6 of its traffic, 768: 0.84; 128 or 384 heads:
//    1.05 - 1.3);
//  * the fused kernel (one team of workgroups per head, counter barriers) for 8 or 16 heads whose
//    phases fill the device (fused_full_width; the metric workload: 17.7 us against 20.0 chained
//    and 22.4 as two launches) - only for callers that own the device (device_exclusive): its
//    workgroups wait for each other, and beside a kernel of somebody else they may not all be
//    running; everybody else continues down this list;
//  * one launch per half step where the one-launch kernels are at a disadvantage: 128-row
//    problems both ways on a head count that does not divide by the 8 XCDs the chained kernel
//    pins heads to; head dims above 80 with more than 64 blocks of 64
//    rows and more; fewer than 8 heads of thousands of tokens (a head's tasks all run on one
//    XCD); a single step on an uneven head count from 4096 tokens on, or on 8 heads from ~7000
//    on (two launches against an unbalanced one); few problems of 65 .. 128 rows (a single step:
//    up to ~160 R problems, or 512 on at most 8 heads; more steps, 97 .. 128 rows only: up to 48,
//    or at most 4 heads of up to 4096 tokens), which the stage kernels split in halves when a launch would leave the
//    device mostly empty (10 - 30 % ahead there); blocks or block counts of 129 .. 256 rows
//    (heads of up to 65536 tokens), which only the stage kernels have tile classes for;
//  * else the chained kernel (one launch, tasks in dispatch order): 10 - 25 % ahead of the stage
//    launches over most of the sweep, heads of 2 .. 8 blocks included (their L / Z problems share
//    tiles, see pack_shift_of).
// Does the caller own the device while its calls run (MA_FLAG_DEVICE_EXCLUSIVE, or the environment
// variable MA_HIP_DEVICE_EXCLUSIVE set to something other than 0 / empty)?  Only then may AUTO choose
// the fused kernel, whose workgroups wait for each other and so must all be on the device together.
bool device_exclusive(const ma_fwd_params* p) {
    static const bool env = [] {
        const char* v = std::getenv("MA_HIP_DEVICE_EXCLUSIVE");
        return v != nullptr && v[0] != '\0' && !(v[0] == '0' && v[1] == '\0');
    }();
    return env || (p->flags & MA_FLAG_DEVICE_EXCLUSIVE) != 0;
}

// ---- AUTO: which variant is the fastest for a problem.  Every threshold below is read off the sweeps of
// bench.py --sweep-variants (each variant that takes a shape timed through this ABI); the figures in the comments are
// time ratios against the next best variant.

// fp32: heads of up to 16 blocks of up to 16 rows can run whole in one workgroup each (one launch, no state in
// memory).  A head then has one compute unit to itself, which pays from 64 heads on (256 tokens x 64: 0.93 of the
// stage launches' time at 96 heads, 0.5 - 0.7 from 192 on, also beyond one pass over the compute units) and for any
// head count when the head is small (128 tokens x 32: 0.45 - 0.8); few large heads are faster spread over many
// compute units by the stage launches (one head of 256 x 64, two steps: 16.6 us against 20.4) - unless there is a
// single step: then a workgroup per (head, position) needs nothing from any other (one head of 256 x 64: 5.3 us
// against 7.9 as two launches; 16 heads: 6.7 against 10.3).
int auto_fp32(const ma_fwd_params* p, long long heads, long long M) {
    const bool single_step = p->T == 1 && heads * p->B <= kHead32T1MaxGroups;
    const bool pays = heads >= 64 || M * p->B * p->D <= 4096 || single_step;
    return pays && resident_fits(p, true) ? MA_VARIANT_RESIDENT : MA_VARIANT_STAGED;
}

// 16-bit: does one of the forms of the resident kernel (a whole head per workgroup) win?
bool auto_resident(const ma_fwd_params* p, long long heads, long long M) {
    const long long Np = M * p->B;
    // Heads that fit in LDS whole - Q, K, V and the state in four tiles -, in blocks and block counts of at most two
    // strips (16 waves): every input is read once and no state leaves the compute unit.  From 96 heads on (0.63 - 0.93
    // at T = 1, 2, 3), and with more than one step also for any number of heads of at most 256 tokens in 16-row
    // blocks (0.85 - 0.95 at 256 tokens, 0.55 - 0.8 for shorter heads and three steps; longer heads at D = 32: 1.2 - 1.4
    // below 64 heads; a single step of few heads: 1.03 - 1.23, they stay away).  Head dims up to 64: in the 128-column
    // class the kernel holds heads of ~128 tokens and takes 1.0 - 1.35 of the chained kernel's time on them.
    // (64 heads in longer blocks, more than one step: 0.84 - 0.96; D = 48 at 256 tokens: 1.02)
    if (p->D <= 64 && p->B <= 32 && M <= 32 &&
        (heads >= 96 || (p->T >= 2 && p->B <= 16 && Np <= 256) || (p->T >= 2 && heads >= 64 && Np <= 256) ||
         (heads >= 64 && Np <= 128 && p->B <= 16 && p->D > 32)) &&   // (a single step of 64 short heads: 0.88 - 0.91; D = 32: 1.0)
        resident_head_fits(p))
        return true;
    // Head dims of 65 .. 80 (measured at 72), heads of at most 256 tokens that fit in four tiles or two: 0.48 - 0.95 from
    // 192 heads on for any number of steps (one and a half heads per compute unit: up to 1.05), 0.8 - 1.0 for 128 heads
    // (224 tokens in 32-row blocks: 1.04 - 1.15), and 0.6 - 0.78 for 64 heads of up to 128 tokens in 16-row blocks with
    // more than one step
    if (p->D > 64 && p->D <= 80 && p->B <= 32 && M <= 32 && Np <= 256 && resident_head_fits(p, 2) &&
        (heads >= 192 || (heads >= 128 && (p->B <= 16 || Np <= 192)) || (heads >= 64 && p->B <= 16 && Np <= (p->T >= 2 ? 128 : 64))))
        return true;
    // Head dims above 80 (measured at 96 and 128), more short heads than compute units, in narrow workgroups that share
    // a compute unit, more than one step: 16-row blocks from 512 heads of 96 tokens and more (0.63 - 0.94) and from 1024
    // shorter heads (0.69 - 1.04); longer blocks from 1536 heads (0.78 - 1.04).  A single step: 0.84 - 1.3, they stay away.
    // (D = 128: from 384 heads of 96 tokens and more, 0.87 - 0.93)
    if (p->D > 80 && p->T >= 2 && resident_head_fits(p, 3) &&
        (p->B <= 16 ? (heads >= (p->D > 96 ? 768 : 1024) || (heads >= (p->D > 96 ? 384 : 512) && Np >= 96)) : heads >= (p->D > 96 ? 1024 : 1536)))
        return true;
    // ... D = 128 beyond that: a single step of 1024 heads and more of 96 tokens and more in 16-row blocks (0.84 - 0.97), and
    // with more than one step 192 .. 256 heads of 96 .. 128 tokens (four tiles, one workgroup each: 0.87 - 0.94)
    if (p->D > 96 && p->T == 1 && p->B <= 16 && Np >= 96 && heads >= 1024 && resident_head_fits(p, 3)) return true;
    if (p->D > 96 && p->T >= 2 && p->B <= 16 && Np >= 96 && Np <= 128 && heads >= 192 && heads <= 256 && resident_head_fits(p)) return true;
    // ... and with three steps and more any 64 .. 256 heads of at most 128 tokens in 16-row blocks (four tiles, 0.79 - 0.87)
    if (p->D > 80 && p->T >= 3 && p->B <= 16 && Np <= 128 && heads >= 64 && heads <= 256 && resident_head_fits(p)) return true;
    // Heads of about twice that length (257 .. ~540 tokens at D = 64) keep the state and ONE input tile at a time in
    // LDS.  A head has a compute unit to itself for its 2T phases, so the device has to be full of heads: from 192
    // heads on (0.63 - 0.92 at 192 .. 768 heads with T = 2, 3; 0.71 - 1.02 with a single step), and with more than one
    // step from 128 heads on for heads of 448 tokens and more that are a single strip one way (0.86 - 0.95; others
    // 0.97 - 1.17; D = 48: 1.11 - 1.16).  Blocks and block counts of at most 32 (16 waves per workgroup).
    const bool two_tiles = !resident_head_fits(p, 1) && resident_head_fits(p, 2);
    if (two_tiles && p->B <= 32 && M <= 32) {
        bool enough = heads >= 192 || (p->T >= 2 && heads >= 128 && Np >= 448 && (M <= 16 || p->B <= 16) && p->D > 48);
        // ... in 16-row blocks from 384 tokens on for any number of steps (0.83 - 0.95)
        if (heads >= 128 && p->B <= 16 && Np >= 384 && p->D > 48 && p->D <= 64) enough = true;
        // head dims of 65 .. 80 (measured at 72): a single step 1.24 - 1.35, one and a half passes over the compute units 1.06 - 1.12
        if (p->D > 64 && p->D <= 80 && (p->T == 1 || (heads > 256 && heads < 448))) enough = false;
        // head dims above 80 (256 .. 288 tokens at D = 128): 256 tokens in 16-row blocks 0.79 - 0.87 for 192 .. 256 heads, else
        // only where the heads come in whole passes over the compute units (0.82 - 0.97; 192 or 384 heads: 1.03 - 1.24)
        if (p->D > 80)
            enough = (heads >= 192 && heads <= 256 && Np <= 256 && p->B <= 16) || (heads >= 224 && heads <= 256) || heads >= 448 ||
                     (heads >= 384 && p->T >= 2 && Np <= 256 && p->B <= 16);   // (narrow workgroups: 0.84 - 0.97)
        // ... a single step of such heads in longer blocks (160 / 224 tokens, 32-row blocks): 1.04 - 1.21
        if (p->D > 80 && p->T == 1 && p->B > 16) enough = false;
        // ... and at D = 96 any number of steps of 160 tokens in 32-row blocks: 1.05 - 1.38
        if (p->D > 80 && p->D <= 96 && p->B > 16 && Np < 224) enough = false;
        if (enough) return true;
    }
    // ... in blocks of 33 .. 64 rows (eight waves per workgroup: 0.84 - 1.22): whole passes over the compute units only - one
    // pass of 256 heads 0.84 - 0.91 at T = 2, 3 and (D <= 64) 0.87 - 0.96 with a single step, two or three passes 0.90 - 0.97
    // with more than one step (one and a half: 1.09 - 1.22)
    if (two_tiles && p->D <= 80 && p->B <= 64 && M <= 64 && heads >= 224 && heads <= 256 && (p->T >= 2 || p->D <= 64)) return true;
    if (two_tiles && p->D <= 64 && p->B <= 64 && M <= 64 && p->T >= 2 && heads >= 448 && heads <= 768 && (heads % 256 == 0 || heads % 256 >= 224))
        return true;
    // Many short heads in 16-row blocks, whichever form takes them (D = 128: 1.07 - 1.37; D = 72: a single step
    // 1.2 - 1.35, 128 heads 1.03 - 1.16)
    if (p->D <= 80 && p->B <= 16 && M <= 32 && Np <= 288 && heads >= (p->D > 64 ? 192 : 128) && !(p->D > 64 && p->T == 1) &&
        resident_fits(p, false))
        return true;
    // The one-tile form (aL and aR in one tile, inputs streamed, Y through the workspace) where the heads fill its
    // one-workgroup-per-CU passes (D = 48: 1.12 - 1.19 of the chained kernel's time)
    return heads >= 128 && (heads % 256 == 0 || heads % 256 >= 192) && p->D > 48 && p->D <= 64 &&
           ((p->B <= 32 && M <= 16) || (p->B <= 16 && M <= 32)) && !resident_fits(p, false) && resident_fits(p, true);
}

// 16-bit: the team kernel - only for callers that own the device (its workgroups wait for each other).
bool auto_fused(const ma_fwd_params* p, long long heads, long long M) {
    if (!device_exclusive(p)) return false;
    if (fused_full_width(p)) return true;
    // Head dims of 65 .. 80 (the 80-column tile class; measured at 72) with 128-row problems - blocks or block counts of
    // 97 .. 128 - and more than one step: 8 - 21 % ahead of the chained kernel for 6 .. 128 heads of thousands of tokens
    // (from 2048 tokens on with 32 heads and more, 4096 below that)
    const bool wide5 = p->D > 64 && p->D <= 80, class128 = (M > 96 || p->B > 96) && one_launch_tiles(p);
    return wide5 && class128 && p->T >= 2 && heads >= 6 && heads <= 128 && p->N >= (heads >= 32 ? 2048 : 4096);
}

// 16-bit: do the per-stage launches beat the chained kernel?
bool auto_staged(const ma_fwd_params* p, long long heads, long long M) {
    // head dims of 65 .. 80 with 128-row blocks on 192 heads and more, T >= 2: 4 - 15 % ahead
    if (p->D > 64 && p->D <= 80 && (M > 96 || p->B > 96) && one_launch_tiles(p) && p->T >= 2 && heads >= 192 && p->B > 96 && M >= 4) return true;
    const bool uneven_128 = p->B > 96 && M > 96 && heads % 8 != 0;
    // 128-row blocks in 33 .. 48 blocks (three-strip L / Z problems beside eight-strip R problems) on a head count that
    // does not divide by 8, or on very many heads: 12 / 192 heads of 5000 tokens are 7 - 21 % behind the stage launches
    // in the chained kernel (16 .. 96 heads: 9 - 23 % ahead)
    const bool odd_mix = p->B > 96 && M > 32 && M <= 48 && (heads % 8 != 0 || heads >= 192);
    // head dims above 80 (the 128-column class; measured at 96 and 128): many blocks of 64 rows and more, or 128-row
    // problems on many tokens in total (4 - 16 % behind the stage launches there)
    const bool wide_dim = p->D > 80 && ((M > 64 && p->B >= 64) || ((p->B > 96 || M > 96) && heads * p->N >= 393216));
    // fewer than 8 long heads: a head is pinned to one XCD by the chained kernel
    const bool few_heads = heads < 8 && p->N > (heads <= 2 ? 2048 : 4096);
    // a single step: head counts that do not sit evenly on the XCDs, few very long heads, and at most 4 heads from 1024
    // tokens on (two launches, 3 - 19 % ahead)
    const bool one_step = p->T == 1 && ((heads % 8 != 0 && p->N >= 4096) || (heads < 16 && p->N >= 7168) || (heads <= 4 && p->N >= 1024));
    // launches that leave most of the device empty: the stage kernels run their 6- and 8-strip R and Z problems as two
    // workgroups each then (halves_pay), which the one-launch kernels do not
    const bool rows_halve = p->B > 64 && p->B <= 128, blocks_halve = M > 64 && M <= 128;
    const long long r_problems = heads * M;
    const bool underfilled = (rows_halve && (p->T == 1 ? (r_problems <= 160 || (heads <= 8 && r_problems <= 512))
                                                       : p->B > 96 && (r_problems <= 48 || (heads <= 4 && p->N <= 4096)))) ||
                             (blocks_halve && p->T == 1 && heads * p->B <= 128);
    return uneven_128 || odd_mix || wide_dim || few_heads || one_step || underfilled || !chain_fits(p);
}

int select_variant(const ma_fwd_params* p) {
    const bool fast = mfma_supported(p);
    const bool fast32 = mfma32_supported(p);   // fp32 operands: per-stage launches and the one-launch head kernels
    const long long heads = static_cast<long long>(p->E) * p->H;
    const long long M = (static_cast<long long>(p->N) + p->B - 1) / p->B;
    switch (p->variant) {
        case MA_VARIANT_GENERIC: return MA_VARIANT_GENERIC;
        case MA_VARIANT_STAGED: return fast || fast32 ? MA_VARIANT_STAGED : MA_ERR_UNSUPPORTED;
        case MA_VARIANT_FUSED: return fast && one_launch_tiles(p) ? MA_VARIANT_FUSED : MA_ERR_UNSUPPORTED;
        case MA_VARIANT_CHAINED: return fast && chain_fits(p) ? MA_VARIANT_CHAINED : MA_ERR_UNSUPPORTED;
        case MA_VARIANT_RESIDENT: return (fast || fast32) && resident_fits(p, true) ? MA_VARIANT_RESIDENT : MA_ERR_UNSUPPORTED;
        default:
            if (fast32) return auto_fp32(p, heads, M);
            if (!fast) return MA_VARIANT_GENERIC;
            if (auto_resident(p, heads, M)) return MA_VARIANT_RESIDENT;
            if (auto_fused(p, heads, M)) return MA_VARIANT_FUSED;
            return auto_staged(p, heads, M) ? MA_VARIANT_STAGED : MA_VARIANT_CHAINED;
    }
}

// 16 bytes per lane and store, one workgroup per compute unit or so: the 2 MiB area is gone in two passes
__global__ void zero_sync_kernel(uint4* sync, int chunks) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < chunks; i += gridDim.x * blockDim.x) sync[i] = make_uint4(0u, 0u, 0u, 0u);
}

struct Prepared {
    Problem P;
    int variant;
};

int run_fused(const Prepared& pr, const ma_fwd_params* p, hipStream_t s) {
    const bool ready = (p->flags & MA_FLAG_SYNC_READY) != 0;
    const bool h = p->dtype_qk == MA_F16;
    const int D = p->D;
    if (D <= 32) return h ? launch_fused_f16_d2(pr.P, ready, s) : launch_fused_bf16_d2(pr.P, ready, s);
    if (D <= 64) return h ? launch_fused_f16_d4(pr.P, ready, s) : launch_fused_bf16_d4(pr.P, ready, s);
    if (D <= 80) return h ? launch_fused_f16_d5(pr.P, ready, s) : launch_fused_bf16_d5(pr.P, ready, s);
    return h ? launch_fused_f16_d8(pr.P, ready, s) : launch_fused_bf16_d8(pr.P, ready, s);
}

int run_chain(const Prepared& pr, const ma_fwd_params* p, hipStream_t s) {
    const bool ready = (p->flags & MA_FLAG_SYNC_READY) != 0;
    const bool h = p->dtype_qk == MA_F16;
    const int D = p->D;
    if (D <= 32) return h ? launch_chain_f16_d2(pr.P, ready, s) : launch_chain_bf16_d2(pr.P, ready, s);
    if (D <= 64) return h ? launch_chain_f16_d4(pr.P, ready, s) : launch_chain_bf16_d4(pr.P, ready, s);
    if (D <= 80) return h ? launch_chain_f16_d5(pr.P, ready, s) : launch_chain_bf16_d5(pr.P, ready, s);
    return h ? launch_chain_f16_d8(pr.P, ready, s) : launch_chain_bf16_d8(pr.P, ready, s);
}

int run_r(const Prepared& pr, const ma_fwd_params* p, bool first, bool with_v, hipStream_t s) {
    if (pr.variant == MA_VARIANT_GENERIC) return launch_generic_r(pr.P, p->dtype_qk, p->dtype_v, first, with_v, s);
    if (p->dtype_qk == MA_F32) return launch_mfma32_r(pr.P, first, with_v, s);
    return p->dtype_qk == MA_F16 ? launch_mfma_r_f16(pr.P, first, with_v, s) : launch_mfma_r_bf16(pr.P, first, with_v, s);
}
int run_l(const Prepared& pr, const ma_fwd_params* p, hipStream_t s) {
    if (pr.variant == MA_VARIANT_GENERIC) return launch_generic_l(pr.P, p->dtype_qk, s);
    if (p->dtype_qk == MA_F32) return launch_mfma32_l(pr.P, s);
    return p->dtype_qk == MA_F16 ? launch_mfma_l_f16(pr.P, s) : launch_mfma_l_bf16(pr.P, s);
}
int run_z(const Prepared& pr, const ma_fwd_params* p, hipStream_t s) {
    if (pr.variant == MA_VARIANT_GENERIC) return launch_generic_z(pr.P, p->dtype_qk, p->dtype_v, s);
    if (p->dtype_qk == MA_F32) return launch_mfma32_z(pr.P, s);
    return p->dtype_qk == MA_F16 ? launch_mfma_z_f16(pr.P, s) : launch_mfma_z_bf16(pr.P, s);
}

// Heads of at most 8 blocks: the 16-bit per-stage and chained L and Z problems put 16 >> pack_shift in-block
// positions into one 16-row tile (2^pack_shift >= M rows each) instead of leaving most of the tile empty.
int pack_shift_of(int variant, const ma_fwd_params* p, int M) {
    if ((variant != MA_VARIANT_STAGED && variant != MA_VARIANT_CHAINED) || p->dtype_qk == MA_F32 || M > 8) return 4;
    int sh = 0;
    while ((1 << sh) < M) ++sh;
    return sh;
}

int prepare(const ma_fwd_params* p, Prepared* out) {
    ma_ws_layout L;
    int st = layout_of(p, &L);
    if (st != MA_OK) return st;
    st = check_buffers(p, L);
    if (st != MA_OK) return st;
    const int v = select_variant(p);
    if (v < 0) return v;
    out->P = make_problem(p, L);
    out->variant = v;
    // Streaming stores pay where a launch writes a state that fits the L2 caches and ends right
    // after (few long heads with 64-row blocks: the metric workload gains 1.5 us per forward);
    // with more, smaller problems or a state beyond the caches they cost 5-10 %.
    out->P.stream_stores = v == MA_VARIANT_STAGED && p->dtype_qk != MA_F32 && p->B > 32 && out->P.M > 32 &&
                           static_cast<long long>(p->E) * p->H * out->P.M * p->B <= 128 * 1024;
    out->P.pack_shift = pack_shift_of(v, p, out->P.M);
    // Agent-scope state loads keep the state's lines in the L2 (streaming loads give them up first).  Measured over
    // heads x tokens grids at T = 1, 2, 3, by the size of one state array (heads x tokens x D at 16 bits): the chained
    // kernel gains 2 - 3 % at 6 .. 24 MB, nothing below, 1 % up to 64 MB and loses 3 - 4 % from 128 MB on; the per-stage
    // launches gain 2 - 5 % up to 1.5 MB and lose up to 8 % at 3 .. 12 MB (a single step most); the team kernel is
    // faster with streaming loads (17.2 against 18.0 us on the metric workload).
    {
        const long long state_bytes = static_cast<long long>(p->E) * p->H * out->P.M * p->B * p->D * 2;
        out->P.state_agent = p->dtype_qk != MA_F32 && ((v == MA_VARIANT_CHAINED && state_bytes >= (6ll << 20) && state_bytes <= (64ll << 20)) ||
                                                       (v == MA_VARIANT_STAGED && state_bytes <= (3ll << 19)));
    }
    out->P.one_tile_ok = 1;   // a problem that resolves to the resident kernel may use any of its forms
    return MA_OK;
}


// Workspace of the backward pass: every step's forward state, the state gradients, and padded
// fp32 accumulators of the input gradients.
struct BwdLayout {
    uint64_t aL, cL, aR, cR, Y, stats;      // aL / cL: T slots; aR / cR: T - 1 slots (steps 1..T-1)
    uint64_t gaR, gcR, gaL, gcL, gY, dq, dk, dv, pk, pv;
    int parts;                              // per-tile partial buffers of dk / dv (R stage split over workgroups)
    uint64_t slot_a, slot_c;                // bytes of one aL / aR slot and of one cL / cR slot
    uint64_t total;
};

int bwd_prepare(const ma_bwd_params* b, ma_fwd_params* pp, BwdLayout* L) {
    if (b == nullptr) return MA_ERR_NULL;
    *pp = b->fwd;
    // the forward output is not needed: a stand-in that passes the checks and is never written
    pp->out = b->dv;
    for (int i = 0; i < 3; ++i) pp->out_stride[i] = b->dv_stride[i];
    int st = check_shape(pp);
    if (st != MA_OK) return st;
    if (pp->variant != MA_VARIANT_AUTO && pp->variant != MA_VARIANT_GENERIC && pp->variant != MA_VARIANT_STAGED) return MA_ERR_UNSUPPORTED;
    for (int i = 0; i < 3; ++i)
        if (b->dout_stride[i] < 0 || b->dq_stride[i] < 0 || b->dk_stride[i] < 0 || b->dv_stride[i] < 0) return MA_ERR_STRIDE;
    if (pp->N > 1 && (b->dout_stride[2] < pp->Dv || b->dv_stride[2] < pp->Dv || b->dq_stride[2] < pp->D || b->dk_stride[2] < pp->D))
        return MA_ERR_STRIDE;
    if ((pp->E > 1 && (b->dq_stride[0] == 0 || b->dk_stride[0] == 0 || b->dv_stride[0] == 0)) ||
        (pp->H > 1 && (b->dq_stride[1] == 0 || b->dk_stride[1] == 0 || b->dv_stride[1] == 0)))
        return MA_ERR_STRIDE;
    const uint64_t M = (static_cast<uint64_t>(pp->N) + pp->B - 1) / pp->B;
    const uint64_t rows = static_cast<uint64_t>(pp->E) * pp->H * M * pp->B;
    const uint64_t sq = elt_size(pp->dtype_qk), sv = elt_size(pp->dtype_v), T = pp->T;
    L->slot_a = align_up(rows * pp->D * sq);
    L->slot_c = align_up(rows * 4);
    uint64_t off = 0;
    L->aL = off; off += T * L->slot_a;
    L->cL = off; off += T * L->slot_c;
    L->aR = off; off += (T - 1) * L->slot_a;
    L->cR = off; off += (T - 1) * L->slot_c;
    L->Y = off; off = align_up(off + rows * pp->Dv * sv);
    L->stats = off; off = align_up(off + rows * 8);
    L->gaR = off; off = align_up(off + rows * pp->D * 4);
    L->gcR = off; off = align_up(off + rows * 4);
    L->gaL = off; off = align_up(off + rows * pp->D * 4);
    L->gcL = off; off = align_up(off + rows * 4);
    L->gY = off; off = align_up(off + rows * pp->Dv * 4);
    // dq, dk, dv are contiguous: one fill kernel zeroes the three
    L->dq = off; off += rows * pp->D * 4;
    L->dk = off; off += rows * pp->D * 4;
    L->dv = off; off = align_up(off + rows * pp->Dv * 4);
    {
        ma_ws_layout none;
        std::memset(&none, 0, sizeof(none));
        const Problem P = make_problem(pp, none);
        L->parts = pp->variant == MA_VARIANT_GENERIC ? 0 : bwd_r_split_tiles(P, pp->dtype_qk, pp->dtype_v);
    }
    L->pk = off; off = align_up(off + static_cast<uint64_t>(L->parts) * rows * pp->D * 4);
    L->pv = off; off = align_up(off + static_cast<uint64_t>(L->parts) * rows * pp->Dv * 4);
    L->total = off;
    return MA_OK;
}

// Device address of `scratch` on the current device, resolved once per device.
constexpr int kMaxDevices = 64;
// Per device: the scratch array's address, and what the in-use guard of ma_fwd_static needs - an
// event recorded behind the last call's work and the stream that call was made on.
struct StaticScratch {
    void* ptr = nullptr;
    hipEvent_t done = nullptr;
    hipStream_t last_stream = nullptr;
    bool in_flight = false;
};
std::mutex g_scratch_mutex;
StaticScratch g_scratch[kMaxDevices];

// Looks up (first call on a device: sets up) the current device's entry; the caller holds g_scratch_mutex.
int static_scratch(StaticScratch** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return MA_ERR_DEVICE;
    StaticScratch& sc = g_scratch[dev];
    if (sc.ptr == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (ptr == nullptr) return MA_ERR_DEVICE;
        hipEvent_t ev = nullptr;
        e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
        if (e != hipSuccess) return static_cast<int>(e);
        sc.done = ev;
        sc.ptr = ptr;
    }
    *out = &sc;
    return MA_OK;
}

}  // namespace

int launch_zero_sync(unsigned* sync, hipStream_t s) {
    static_assert(kSyncAreaBytes % 16 == 0, "the sync area is cleared in 16-byte chunks");
    const int chunks = static_cast<int>(kSyncAreaBytes / 16);   // the area starts the workspace: 256-byte aligned
    hipLaunchKernelGGL(zero_sync_kernel, dim3(256), dim3(256), 0, s, reinterpret_cast<uint4*>(sync), chunks);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ma

using namespace ma;

extern "C" {

int ma_abi_version(void) { return MA_ABI_VERSION; }

const char* ma_strerror(int status) {
    switch (status) {
        case MA_OK: return "ok";
        case MA_ERR_NULL: return "a required pointer is NULL";
        case MA_ERR_SHAPE: return "invalid shape: every dimension, B and T must be >= 1 and E*H*Np must fit int32";
        case MA_ERR_DTYPE: return "unknown dtype (expected MA_F32, MA_F16 or MA_BF16)";
        case MA_ERR_STRIDE: return "invalid stride or misaligned tensor pointer";
        case MA_ERR_WORKSPACE: return "workspace missing, not 256-byte aligned or smaller than ma_fwd_workspace_bytes()";
        case MA_ERR_UNSUPPORTED: return "the requested variant does not support this problem";
        case MA_ERR_VARIANT: return "unknown variant";
        case MA_ERR_DEVICE: return "no usable gfx950 device";
        case MA_ERR_BUSY: return "the built-in scratch of ma_fwd_static is still in use by a call on another stream: order the calls on one stream, wait for the earlier one, or call ma_fwd with a workspace per stream";
        case MA_ERR_STATIC_LIMIT: return "the problem's state exceeds MA_STATIC_WORKSPACE_BYTES, the built-in scratch of ma_fwd_static: call ma_fwd with a workspace";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

int ma_fwd_workspace_layout(const ma_fwd_params* p, ma_ws_layout* layout) {
    if (layout == nullptr) return MA_ERR_NULL;
    return layout_of(p, layout);
}

uint64_t ma_fwd_workspace_bytes(const ma_fwd_params* p) {
    ma_ws_layout L;
    return layout_of(p, &L) == MA_OK ? L.total : 0;
}

int ma_workspace_init(const ma_fwd_params* p, void* stream) {
    ma_ws_layout L;
    const int st = layout_of(p, &L);
    if (st != MA_OK) return st;
    if (!p->workspace || reinterpret_cast<uintptr_t>(p->workspace) % kAlign || p->workspace_bytes < L.total) return MA_ERR_WORKSPACE;
    return launch_zero_sync(reinterpret_cast<unsigned*>(static_cast<char*>(p->workspace) + L.sync), static_cast<hipStream_t>(stream));
}

int ma_fwd_select_variant(const ma_fwd_params* p) {
    const int st = check_shape(p);
    if (st != MA_OK) return st;
    return select_variant(p);
}

const char* ma_fwd_kernel_name(const ma_fwd_params* p) {
    if (check_shape(p) != MA_OK) return nullptr;
    const bool f32 = p->dtype_qk == MA_F32;
    switch (select_variant(p)) {
        case MA_VARIANT_GENERIC: return "r_step_kernel";
        case MA_VARIANT_STAGED: return f32 ? "r_step_f32" : "r_step_mfma";
        case MA_VARIANT_FUSED: return "fused_fwd_mfma";
        case MA_VARIANT_CHAINED: return "chain_fwd_mfma";
        case MA_VARIANT_RESIDENT: {
            if (!f32)
                return resident_head_fits(p, 4) ? "resident_head_mfma" : resident_head_fits(p, 3) ? "resident_head2_mfma"
                       : resident_head_fits(p, 1) ? "resident_head_mfma" : resident_head_fits(p, 2) ? "resident_head2_mfma" : "resident_fwd_mfma";
            Problem P;
            std::memset(&P, 0, sizeof(P));
            P.E = p->E; P.H = p->H; P.N = p->N; P.D = p->D; P.Dv = p->Dv; P.B = p->B; P.T = p->T;
            P.M = (p->N + p->B - 1) / p->B;
            return head32_single_step(P) ? "head_t1_f32" : "head_fwd_f32";
        }
        default: return nullptr;
    }
}

int ma_r_step(const ma_fwd_params* p, int first, int with_v, void* stream) {
    Prepared pr;
    const int st = prepare(p, &pr);
    if (st != MA_OK) return st;
    if (pr.variant != MA_VARIANT_GENERIC && pr.variant != MA_VARIANT_STAGED) return MA_ERR_UNSUPPORTED;
    return run_r(pr, p, first != 0, with_v != 0, static_cast<hipStream_t>(stream));
}

int ma_l_step(const ma_fwd_params* p, void* stream) {
    Prepared pr;
    const int st = prepare(p, &pr);
    if (st != MA_OK) return st;
    if (pr.variant != MA_VARIANT_GENERIC && pr.variant != MA_VARIANT_STAGED) return MA_ERR_UNSUPPORTED;
    return run_l(pr, p, static_cast<hipStream_t>(stream));
}

int ma_z_step(const ma_fwd_params* p, void* stream) {
    Prepared pr;
    const int st = prepare(p, &pr);
    if (st != MA_OK) return st;
    if (pr.variant != MA_VARIANT_GENERIC && pr.variant != MA_VARIANT_STAGED) return MA_ERR_UNSUPPORTED;
    return run_z(pr, p, static_cast<hipStream_t>(stream));
}

int ma_fwd(const ma_fwd_params* p, void* stream) {
    Prepared pr;
    int st = prepare(p, &pr);
    if (st != MA_OK) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pr.variant == MA_VARIANT_FUSED) return run_fused(pr, p, s);
    if (pr.variant == MA_VARIANT_CHAINED) return run_chain(pr, p, s);
    if (pr.variant == MA_VARIANT_RESIDENT) return run_resident(pr.P, p->dtype_qk, false, s);
    for (int t = 0; t < p->T - 1; ++t) {
        st = run_r(pr, p, t == 0, false, s);
        if (st) return st;
        st = run_l(pr, p, s);
        if (st) return st;
    }
    st = run_r(pr, p, p->T == 1, true, s);
    if (st) return st;
    return run_z(pr, p, s);
}

int ma_fwd_static(const ma_fwd_params* p, void* stream) {
    if (p == nullptr) return MA_ERR_NULL;
    ma_ws_layout L;
    int st = layout_of(p, &L);
    if (st != MA_OK) return st;
    if (L.total > MA_STATIC_WORKSPACE_BYTES) return MA_ERR_STATIC_LIMIT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusNone;
    }
    const bool capturing = capture != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);   // the guard's bookkeeping; launches are short
    StaticScratch* sc = nullptr;
    st = static_scratch(&sc);
    if (st != MA_OK) return st;
    // In-use guard: the array belongs to the last call until that call's work is complete.  A call on
    // the same stream is ordered behind it; one on another stream is turned away while the event
    // recorded behind the last call has not completed.  (Captured calls are neither checked nor
    // recorded: an event recorded during capture belongs to the graph.)
    if (!capturing && sc->in_flight && sc->last_stream != s) {
        const hipError_t q = hipEventQuery(sc->done);
        if (q == hipErrorNotReady) {
            (void)hipGetLastError();
            return MA_ERR_BUSY;
        }
        if (q != hipSuccess) return static_cast<int>(q);
        sc->in_flight = false;
    }
    ma_fwd_params pp = *p;
    pp.workspace = sc->ptr;
    pp.workspace_bytes = MA_STATIC_WORKSPACE_BYTES;
    // the array keeps what the last call left: nothing may be assumed about its sync area, so the
    // one-launch variants clear it with their fill kernel in front of the forward kernel
    pp.flags &= ~MA_FLAG_SYNC_READY;
    st = ma_fwd(&pp, stream);
    if (!capturing) {
        // also after a failed launch sequence: some of its kernels may have been queued
        const hipError_t r = hipEventRecord(sc->done, s);
        if (r != hipSuccess) return st != MA_OK ? st : static_cast<int>(r);
        sc->last_stream = s;
        sc->in_flight = true;
    }
    return st;
}

int ma_matrix(const ma_fwd_params* p, float* A, void* stream) {
    if (p == nullptr || A == nullptr) return MA_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(A) % 4) return MA_ERR_STRIDE;
    // the T steps on q and k alone: v and out are stand-ins that no stage of this call touches
    ma_fwd_params pp = *p;
    pp.v = pp.q;
    pp.out = A;
    pp.Dv = pp.D;
    pp.dtype_v = pp.dtype_qk;
    for (int i = 0; i < 3; ++i) pp.v_stride[i] = pp.out_stride[i] = pp.q_stride[i];
    if (pp.E > 1 && pp.out_stride[0] == 0) pp.out_stride[0] = 1;   // q may be broadcast; the stand-in
    if (pp.H > 1 && pp.out_stride[1] == 0) pp.out_stride[1] = 1;   // output must pass the overlap check
    if (pp.variant != MA_VARIANT_AUTO && pp.variant != MA_VARIANT_GENERIC && pp.variant != MA_VARIANT_STAGED)
        return pp.variant < MA_VARIANT_AUTO || pp.variant > MA_VARIANT_CHAINED ? MA_ERR_VARIANT : MA_ERR_UNSUPPORTED;
    if (pp.variant == MA_VARIANT_AUTO) {
        const int st = check_shape(&pp);
        if (st != MA_OK) return st;
        pp.variant = mfma_supported(&pp) || mfma32_supported(&pp) ? MA_VARIANT_STAGED : MA_VARIANT_GENERIC;
    }
    Prepared pr;
    int st = prepare(&pp, &pr);
    if (st != MA_OK) return st;
    if (!generic_matrix_fits(pr.P)) return MA_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (int t = 0; t < pp.T - 1; ++t) {
        st = run_r(pr, &pp, t == 0, false, s);
        if (st) return st;
        st = run_l(pr, &pp, s);
        if (st) return st;
    }
    st = run_r(pr, &pp, pp.T == 1, false, s);
    if (st) return st;
    return launch_generic_matrix(pr.P, pp.dtype_qk, A, pp.T == 1, s);
}

uint64_t ma_bwd_workspace_bytes(const ma_bwd_params* b) {
    ma_fwd_params pp;
    BwdLayout L;
    return bwd_prepare(b, &pp, &L) == MA_OK ? L.total : 0;
}

int ma_bwd(const ma_bwd_params* b, void* stream) {
    ma_fwd_params pp;
    BwdLayout L;
    int st = bwd_prepare(b, &pp, &L);
    if (st != MA_OK) return st;
    if (!pp.q || !pp.k || !pp.v || !b->dout || !b->dq || !b->dk || !b->dv) return MA_ERR_NULL;
    if (!pp.workspace || reinterpret_cast<uintptr_t>(pp.workspace) % kAlign || pp.workspace_bytes < L.total) return MA_ERR_WORKSPACE;
    const uintptr_t aq = elt_size(pp.dtype_qk), av = elt_size(pp.dtype_v);
    if (reinterpret_cast<uintptr_t>(pp.q) % aq || reinterpret_cast<uintptr_t>(pp.k) % aq || reinterpret_cast<uintptr_t>(b->dq) % aq ||
        reinterpret_cast<uintptr_t>(b->dk) % aq || reinterpret_cast<uintptr_t>(pp.v) % av || reinterpret_cast<uintptr_t>(b->dout) % av ||
        reinterpret_cast<uintptr_t>(b->dv) % av)
        return MA_ERR_STRIDE;
    const bool fma_only = pp.variant == MA_VARIANT_GENERIC;
    if (pp.variant == MA_VARIANT_AUTO) pp.variant = mfma_supported(&pp) || mfma32_supported(&pp) ? MA_VARIANT_STAGED : MA_VARIANT_GENERIC;
    const int v = select_variant(&pp);
    if (v < 0) return v;

    char* ws = static_cast<char*>(pp.workspace);
    ma_ws_layout none;
    std::memset(&none, 0, sizeof(none));
    Prepared pr;
    pr.P = make_problem(&pp, none);
    pr.variant = v;
    Problem& P = pr.P;
    P.pack_shift = pack_shift_of(v, &pp, P.M);   // the forward steps run again as per-stage launches
    if (!bwd_fits(P)) return MA_ERR_UNSUPPORTED;
    P.Y = ws + L.Y;
    P.stats = reinterpret_cast<float*>(ws + L.stats);
    P.sync = nullptr;
    const int T = pp.T;
    auto at_step = [&](int t) {   // state pointers of step t: aR_t, cR_t in, aL_t, cL_t out
        P.aL = ws + L.aL + t * L.slot_a;
        P.cL = reinterpret_cast<float*>(ws + L.cL + t * L.slot_c);
        // step 0 takes aR = q, cR = 1 from the inputs: its state pointers only have to be valid
        P.aR = ws + (t > 0 ? L.aR + (t - 1) * L.slot_a : L.aL);
        P.cR = reinterpret_cast<float*>(ws + (t > 0 ? L.cR + (t - 1) * L.slot_c : L.cL));
    };
    hipStream_t s = static_cast<hipStream_t>(stream);

    // forward again, every step's state kept
    for (int t = 0; t < T; ++t) {
        at_step(t);
        st = run_r(pr, &pp, t == 0, t == T - 1, s);
        if (st) return st;
        if (t < T - 1) {   // the L step reads aL_t, cL_t and writes aR_{t+1}, cR_{t+1}
            P.aR = ws + L.aR + t * L.slot_a;
            P.cR = reinterpret_cast<float*>(ws + L.cR + t * L.slot_c);
            st = run_l(pr, &pp, s);
            if (st) return st;
        }
    }

    BwdBuffers G;
    G.gaR = reinterpret_cast<float*>(ws + L.gaR); G.gcR = reinterpret_cast<float*>(ws + L.gcR);
    G.gaL = reinterpret_cast<float*>(ws + L.gaL); G.gcL = reinterpret_cast<float*>(ws + L.gcL);
    G.gY = reinterpret_cast<float*>(ws + L.gY);
    G.dq = reinterpret_cast<float*>(ws + L.dq); G.dk = reinterpret_cast<float*>(ws + L.dk); G.dv = reinterpret_cast<float*>(ws + L.dv);
    G.fma_only = fma_only ? 1 : 0;
    G.pk = L.parts ? reinterpret_cast<float*>(ws + L.pk) : nullptr;
    G.pv = L.parts ? reinterpret_cast<float*>(ws + L.pv) : nullptr;
    G.jt_split = 0;
    G.state16 = (!fma_only && bwd_state16_ok(P, pp.dtype_qk, pp.dtype_v)) ? 1 : 0;
    // register kernels in every stage, rows of the caller's gradients aligned for 4-element stores: the stages
    // write dq, dk, dv themselves
    G.direct = 0;
    {
        void* outp[3] = {b->dq, b->dk, b->dv};
        const int64_t* outst[3] = {b->dq_stride, b->dk_stride, b->dv_stride};
        bool ok = !fma_only && bwd_all_reg(P, pp.dtype_qk, pp.dtype_v);
        for (int i = 0; i < 3; ++i) {
            G.out[i] = static_cast<char*>(outp[i]);
            for (int a = 0; a < 3; ++a) G.outs[i][a] = outst[i][a];
            ok = ok && reinterpret_cast<uintptr_t>(outp[i]) % (4 * elt_size(pp.dtype_qk)) == 0 && outst[i][0] % 4 == 0 &&
                 outst[i][1] % 4 == 0 && outst[i][2] % 4 == 0;
        }
        G.direct = ok ? 1 : 0;
    }
    G.dout = static_cast<const char*>(b->dout);
    for (int i = 0; i < 3; ++i) G.dos[i] = b->dout_stride[i];
    const long long rows = static_cast<long long>(P.E) * P.H * P.M * P.B;
    if (fma_only || !bwd_all_reg(P, pp.dtype_qk, pp.dtype_v)) {
        st = launch_bwd_zero(G.dq, rows * (2LL * P.D + P.Dv), s);
        if (st) return st;
    }

    at_step(T - 1);
    st = launch_bwd_z(P, G, pp.dtype_qk, pp.dtype_v, s);
    if (st) return st;
    for (int t = T - 1; t >= 0; --t) {
        at_step(t);
        st = launch_bwd_r(P, G, pp.dtype_qk, pp.dtype_v, t == 0, t == T - 1, s);
        if (st) return st;
        if (t > 0) {   // L step t-1: state aL_{t-1}, cL_{t-1}; gradients gaR, gcR of its outputs
            at_step(t - 1);
            st = launch_bwd_l(P, G, pp.dtype_qk, s);
            if (st) return st;
        }
    }
    if (G.direct) return MA_OK;
    // fp32 accumulators -> the caller's tensors: one launch when dv has the shape and dtype of dq / dk
    long long st3[3][3];
    for (int i = 0; i < 3; ++i) { st3[0][i] = b->dq_stride[i]; st3[1][i] = b->dk_stride[i]; st3[2][i] = b->dv_stride[i]; }
    const float* src[3] = {G.dq, G.dk, G.dv};
    void* dst[3] = {b->dq, b->dk, b->dv};
    const bool same = pp.Dv == pp.D && pp.dtype_v == pp.dtype_qk;
    st = launch_bwd_out(same ? 3 : 2, src, dst, st3, pp.dtype_qk, P, P.D, s);
    if (st || same) return st;
    return launch_bwd_out(1, src + 2, dst + 2, st3 + 2, pp.dtype_v, P, P.Dv, s);
}

}  // extern "C"
