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
// of ITS head have raised their flags (one word per task in the workspace's sync
// area; one wave polls them), and raises its own flag when its stores have been
// acknowledged.  There is no barrier across heads and no co-residency
// requirement: the device is oversubscribed with workgroups, tasks of the next
// phase start as soon as their head is ready, and the tail of one phase overlaps
// the start of the next.  Loads that depend only on the inputs (K / V tiles, Q
// rows, mask bytes) are issued BEFORE the wait.
//
// Coherence: workgroup ids are dealt round-robin to the 8 XCDs, and head h only
// uses ids with id % 8 == h % 8, so producers and consumers of a head share one
// L2: publishing needs only "my stores are acknowledged" (vmcnt(0)), reading uses
// streaming loads that never hit in L1 - no L2 write-back, no invalidate.  Each
// flag carries the XCC id of its producer; a consumer that finds a producer on
// another XCD (a device that does not deal ids this way) raises the sync area's
// error word, and falls back to an agent-scope acquire.
//
// The state arrays are the per-head ones of the staged variant.  The last Z task
// of a head to finish (a counter per head) clears the head's flags, so the area
// is zero again when the launch is over.  Every wait is bounded (spin_limit
// polls): a task that gives up raises the error word and runs on, so the grid
// always drains.
#pragma once

#include "ma_fused.h"

namespace ma {
namespace mfma {

struct ChainPlan {
    int hx;        // heads per XCD (heads xcd, xcd + 8, ...)
    int tR, tL;    // tasks per head in an R phase / an L or Z phase
    int stride;    // flag words per head: T * (tR + tL) flags + 1 counter
    unsigned spin_limit;
};

constexpr int kChainWords = 256 * 1024;   // flag words of the chained kernel, behind the team sectors
static_assert(static_cast<uint64_t>(kSyncWords + kChainWords) * 4 == kSyncAreaBytes, "sync area size mismatch");

// wave 0: poll until the `count` (<= 128) flags at `f` are all raised; returns false if
// some producer ran on another XCD than `my_xcc`
__device__ __forceinline__ bool chain_wait(const unsigned* f, int count, unsigned my_xcc, unsigned spin_limit, unsigned* error,
                                           int lane) {
    unsigned spins = 0;
    unsigned a = 1u + my_xcc, b = 1u + my_xcc;
    for (;;) {
        a = lane < count ? __hip_atomic_load(f + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1u + my_xcc;
        b = lane + 64 < count ? __hip_atomic_load(f + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1u + my_xcc;
        if (__builtin_amdgcn_ballot_w64(a == 0u || b == 0u) == 0) break;
        __builtin_amdgcn_s_sleep(2);
        if (++spins > spin_limit) {
            if (lane == 0) __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
    }
    return __builtin_amdgcn_ballot_w64((a != 0u && a != 1u + my_xcc) || (b != 0u && b != 1u + my_xcc)) == 0;
}

template <class T, int DT, int NTB, int NTM, int W>
__global__ __launch_bounds__(64 * W) void chain_fwd_mfma(Problem P, ChainPlan plan) {
    using RP = RProb<T, DT, NTB>;
    using LP = LProb<T, DT, NTM>;
    using ZP = ZProb<T, DT, NTM>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int same_xcd;
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

    unsigned* flags = P.sync + kSyncWords + static_cast<size_t>(head) * plan.stride;   // this head's flag words, phase after phase
    unsigned* error = P.sync + 1;
    const int per_step = plan.tR + plan.tL, st = static_cast<int>(step);
    const int off = st * per_step + (odd ? plan.tR : 0);                    // this phase's flags
    const int prev_off = odd ? st * per_step : (st - 1) * per_step + plan.tR;   // only used for p > 0
    const int prev_count = odd ? plan.tR : plan.tL;
    const unsigned my_xcc = xcc_id();

    // waits for the head's previous phase (p > 0); every wave of the workgroup takes part
    auto wait_prev = [&] {
        if (p == 0) return;
        if (threadIdx.x < 64) {
            const bool same = chain_wait(flags + prev_off, prev_count, my_xcc, plan.spin_limit, error, lane);
            if (!same) {   // not the id -> XCD dealing this kernel is built on: say so, and at least drop stale lines
                if (lane == 0) __hip_atomic_store(error, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (lane == 0) same_xcd = same ? 1 : 0;
        }
        __syncthreads();
        if (!same_xcd) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    };

    const Slices S = make_slices<T>(P, e, h, head);
    if (p == nph - 1) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int j = task * PPW + sub;
        const bool active = j < P.B;
        char* sm = smem + sub * Lds<T, DT, NTM>::Z;
        typename ZP::Pre pre;
        typename ZP::St st;
        ZP::issue(P, S, pre, active, active ? j : 0, wig, lane);
        wait_prev();
        ZP::state(P, S, st, active, active ? j : 0, wig, lane);
        ZP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
    } else if (odd) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int j = task * PPW + sub;
        const bool active = j < P.B;
        char* sm = smem + sub * Lds<T, DT, NTM>::L;
        typename LP::Pre pre;
        typename LP::St st;
        LP::issue(P, S, pre, active, e, active ? j : 0, wig, lane);
        wait_prev();
        LP::state(P, S, st, active, active ? j : 0, wig, lane);
        LP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
    } else {
        constexpr int WPP = Split<NTB, W>::WPP, PPW = Split<NTB, W>::PPW;
        const int sub = wave / WPP, wig = wave % WPP;
        const int m = task * PPW + sub;
        const bool active = m < P.M;
        const bool first = p == 0, with_v = p == nph - 2;
        char* sm = smem + sub * Lds<T, DT, NTB>::R;
        typename RP::Pre pre;
        typename RP::St st;
        RP::issue(P, S, pre, active, e, active ? m : 0, first, with_v, wig, lane);
        wait_prev();
        RP::state(P, S, st, active, active ? m : 0, first, wig, lane);
        RP::run(P, S, sm, pre, st, active, active ? m : 0, first, with_v, wig, lane);
    }

    // every wave's stores have reached L2 before the task is published
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (p < nph - 1) {
        if (threadIdx.x == 0) __hip_atomic_store(flags + off + task, 1u + my_xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        // Z tasks: the last one of the head to finish clears the head's flags and the counter
        unsigned* done = flags + plan.stride - 1;
        if (threadIdx.x == 0) {
            const unsigned before = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            same_xcd = before + 1u == static_cast<unsigned>(plan.tL) ? 2 : 0;
        }
        __syncthreads();
        if (same_xcd == 2)
            for (int i = threadIdx.x; i < plan.stride; i += 64 * W) __hip_atomic_store(flags + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace mfma
}  // namespace ma
