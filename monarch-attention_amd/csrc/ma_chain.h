// Chained forward: all T alternating steps, the product with V and the output
// stage in ONE launch (the whole of monarch_attention_torch,
// ma/ma_torch.py:65-108), as a dataflow over the block problems of all phases.
//
// Every block problem of every phase (p even = R step, p odd = L step, p = 2T-1
// = Z step) is one task of one workgroup.  The grid holds the tasks phase by
// phase - all tasks of phase 0, then all of phase 1, ... - and the hardware
// dispatches workgroups in id order, so when a task starts, every task of the
// phase before it has been dispatched already: it cannot be starved by the task
// that waits for it.  A task of phase p > 0 waits until all tasks of phase p - 1
// of ITS head have finished (their stores acknowledged).  There is no barrier across heads and no co-residency
// requirement: the device is oversubscribed with workgroups, tasks of the next
// phase start as soon as their head is ready, and the tail of one phase overlaps
// the start of the next.  Loads that depend only on the inputs (K / V tiles, Q
// rows, mask bytes) are issued BEFORE the wait.
//
// Hand-over: every phase of a head has an arrival counter and a release word on
// DIFFERENT cache lines of the workspace's sync area.  A task that has finished
// (its stores acknowledged) adds itself to the counter with one 64-bit atomic;
// the task whose add completes the count stores the release word, and that word -
// written once - is the only thing waiting tasks poll.  (Polling words that
// producers are still writing slows the whole memory channel of that line down.)
//
// Coherence: workgroup ids are dealt round-robin to the 8 XCDs, and head h only
// uses ids with id % 8 == h % 8, so producers and consumers of a head share one
// L2: publishing needs only "my stores are acknowledged" (vmcnt(0)), reading uses
// streaming loads that never hit in L1 - no L2 write-back, no invalidate.  The
// arrivals carry the XCC id of their workgroup (sum and sum of squares, which
// agree with a common id only if all ids are equal); the release word tells the
// consumers that id, or that the producers were spread over several XCDs.  A
// consumer on another XCD than its producers cannot rely on what it reads: it
// raises the sync area's error word (2) and treats the phase as failed.
//
// The state arrays are the per-head ones of the staged variant.  Every task
// counts itself as finished once its arrival (and release) has been performed;
// the task of a head that finishes last - normally a Z task, but tasks whose wait
// ran out do not run in phase order - clears the head's words, so the area is
// zero again when the launch is over, also after a failed one.  Every wait is bounded (spin_limit
// polls).  A task that gives up - or whose producers failed - raises the error
// word, computes nothing, still counts itself in (marked as failed, which its
// consumers inherit), and as a Z task writes NaN into the output rows it owns: a
// failure is visible in the output and the grid always drains.
#pragma once

#include "ma_fused.h"

namespace ma {
namespace mfma {

struct ChainPlan {
    int hx;        // heads per XCD (heads xcd, xcd + 8, ...)
    int tR, tL;    // tasks per head in an R phase / an L or Z phase
    int stride;    // sync words per head (see chain_stride)
    int go_off;    // offset of the release words inside a head's words
    unsigned spin_limit;
};

constexpr int kChainWords = 256 * 1024;   // sync words of the chained kernel, behind the team sectors
static_assert(static_cast<uint64_t>(kSyncWords + kChainWords) * 4 == kSyncAreaBytes, "sync area size mismatch");

// A head's sync words: 64-bit arrival counters of the 2T-1 publishing phases and the 64-bit counter
// of finished tasks, rounded up to whole 128-byte lines; then one release word per publishing
// phase, rounded up likewise.
__host__ __device__ inline int chain_go_offset(int T) { return (2 * (2 * T - 1) + 2 + 31) / 32 * 32; }
__host__ __device__ inline int chain_stride(int T) { return chain_go_offset(T) + ((2 * T - 1) + 31) / 32 * 32; }

// fields of an arrival (one 64-bit add): tasks | sum of XCC ids | sum of squared ids | failed tasks
constexpr unsigned long long kArriveOne = 1ull, kArriveFailed = 1ull << 48;
__device__ __forceinline__ unsigned long long arrival_of(unsigned xcc, bool failed) {
    return kArriveOne | (static_cast<unsigned long long>(xcc) << 16) | (static_cast<unsigned long long>(xcc * xcc) << 32) |
           (failed ? kArriveFailed : 0ull);
}
// release word: bit 0 ready, bits 1-4 the producers' common XCC id, bit 8 producers on several XCDs, bit 9 a producer failed
constexpr unsigned kGoReady = 1u, kGoSplit = 1u << 8, kGoFailed = 1u << 9;
__device__ __forceinline__ unsigned release_of(unsigned long long total, unsigned tasks) {
    const unsigned sx = static_cast<unsigned>(total >> 16) & 0xffffu, sxx = static_cast<unsigned>(total >> 32) & 0xffffu;
    const unsigned failed = static_cast<unsigned>(total >> 48);
    const bool same = sxx * tasks == sx * sx;   // zero variance of the ids
    return kGoReady | (same ? (sx / tasks) << 1 : kGoSplit) | (failed ? kGoFailed : 0u);
}

// one thread: poll the release word of the previous phase; returns it, or 0 if the wait ran out
__device__ __forceinline__ unsigned chain_wait(const unsigned* go, unsigned spin_limit, unsigned* error, unsigned* host_error) {
    unsigned spins = 0;
    if (spin_limit == 0u) {   // failure-path tests: give up without looking, whatever the word holds
        raise_error(error, host_error, 1u);
        return 0u;
    }
    for (;;) {
        const unsigned w = __hip_atomic_load(go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (w != 0u) return w;
        if (++spins > spin_limit) {
            raise_error(error, host_error, 1u);
            return 0u;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

template <class T, int DT, int NTB, int NTM, int W>
__global__ __launch_bounds__(64 * W) void chain_fwd_mfma(Problem P, ChainPlan plan) {
    using RP = RProb<T, DT, NTB>;
    using LP = LProb<T, DT, NTM>;
    using ZP = ZProb<T, DT, NTM>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ unsigned wg_word;   // thread 0's verdict on the wait / on being the head's last Z task
    const int wave = wave_id(), lane = threadIdx.x & 63;
    const int nph = 2 * P.T;
    const int heads = P.E * P.H;   // E * H * Np fits int32 (validated by the host)

    // task of this workgroup: phases in grid order, heads of this XCD, tasks of the head
    const unsigned xcd = blockIdx.x & 7, ix = blockIdx.x >> 3;
    const unsigned perR = plan.hx * plan.tR, perL = plan.hx * plan.tL;
    const unsigned step = ix / (perR + perL), rem = ix % (perR + perL);
    const bool odd = rem >= perR;
    const int p = 2 * step + (odd ? 1 : 0);
    const unsigned tasks = odd ? plan.tL : plan.tR;
    const unsigned idx = odd ? rem - perR : rem;
    const int head = xcd + 8 * (idx / tasks);
    const int task = idx % tasks;
    if (p >= nph || head >= heads) return;
    const int e = static_cast<unsigned>(head) / static_cast<unsigned>(P.H), h = static_cast<unsigned>(head) % static_cast<unsigned>(P.H);

    unsigned* words = P.sync + kSyncWords + static_cast<size_t>(head) * plan.stride;   // this head's sync words
    unsigned long long* count = reinterpret_cast<unsigned long long*>(words);        // [phase] arrivals, [2T-1] finished tasks of all phases
    unsigned* go = words + plan.go_off;                                               // [phase] release word
    unsigned* error = P.sync + 1;
    const unsigned prev_count = odd ? plan.tR : plan.tL;   // tasks of the previous phase (p > 0)
    const unsigned my_xcc = xcc_id();
    bool failed = false;

    // waits for the head's previous phase (p > 0); every wave of the workgroup takes part
    auto wait_prev = [&] {
        if (p == 0) return;
        if (threadIdx.x == 0) {
            const unsigned w = chain_wait(go + (p - 1), plan.spin_limit, error, P.host_error);
            bool bad = w == 0u || (w & kGoFailed) != 0u;
            if (w != 0u && ((w & kGoSplit) != 0u || ((w >> 1) & 0xfu) != my_xcc)) {
                // not the id -> XCD dealing this kernel is built on: what this task would read is not reliable
                raise_error(error, P.host_error, 2u);
                bad = true;
            }
            wg_word = bad ? 1u : 0u;
        }
        __syncthreads();
        failed = wg_word != 0u;
    };
    (void)prev_count;

    const Slices S = make_slices<T>(P, e, h, head);
    if (p == nph - 1) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int j = (task * PPW + sub) * (NTM == 1 ? 16 >> P.pack_shift : 1);   // heads of few blocks: several positions per tile (TileIndex)
        const bool active = sub < PPW && j < P.B;
        char* sm = smem + sub * Lds<T, DT, NTM>::Z;
        typename ZP::Pre pre;
        typename ZP::St st;
        ZP::issue(P, S, pre, active, active ? j : 0, wig, lane);
        wait_prev();
        if (failed) {
            if (active) z_poison<T, DT, NTM>(P, S, j, wig, lane);   // the failure shows in the output
        } else {
            ZP::state(P, S, st, active, active ? j : 0, wig, lane);
            ZP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
        }
    } else if (odd) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int j = (task * PPW + sub) * (NTM == 1 ? 16 >> P.pack_shift : 1);
        const bool active = sub < PPW && j < P.B;
        char* sm = smem + sub * Lds<T, DT, NTM>::L;
        typename LP::Pre pre;
        typename LP::St st;
        LP::issue(P, S, pre, active, e, active ? j : 0, wig, lane);
        wait_prev();
        if (!failed) {
            LP::state(P, S, st, active, active ? j : 0, wig, lane);
            LP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
        }
    } else {
        constexpr int WPP = Split<NTB, W>::WPP, PPW = Split<NTB, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int m = task * PPW + sub;
        const bool active = sub < PPW && m < P.M;
        const bool first = p == 0, with_v = p == nph - 2;
        char* sm = smem + sub * Lds<T, DT, NTB>::R;
        typename RP::Pre pre;
        typename RP::St st;
        RP::issue(P, S, pre, active, e, active ? m : 0, first, with_v, wig, lane);
        wait_prev();
        if (!failed) {
            RP::state(P, S, st, active, active ? m : 0, first, wig, lane);
            RP::run(P, S, sm, pre, st, active, active ? m : 0, first, with_v, wig, lane);
        }
    }

    // every wave's stores have reached L2 before the task is published
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        if (p < nph - 1) {
            const unsigned long long mine = arrival_of(my_xcc, failed);
            const unsigned long long before = __hip_atomic_fetch_add(count + p, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (((before + mine) & 0xffffull) == tasks)   // this add completes the phase: release its consumers
                __hip_atomic_store(go + p, release_of(before + mine, tasks), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the arrival and the release have been performed before this task counts as finished
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        // The task of the head that finishes LAST - of any phase: tasks whose wait ran out do not run in
        // phase order - clears the head's words; nothing of this head touches them after that.
        const unsigned long long all = static_cast<unsigned long long>(P.T) * (plan.tR + plan.tL);
        const unsigned long long done = __hip_atomic_fetch_add(count + (nph - 1), 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        wg_word = done + 1ull == all ? 2u : 0u;
    }
    __syncthreads();
    if (wg_word == 2u)
        for (int i = threadIdx.x; i < plan.stride; i += 64 * W) __hip_atomic_store(words + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace mfma
}  // namespace ma
