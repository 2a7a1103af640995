// Fused forward: all T alternating steps, the product with V and the output
// stage in ONE launch (the whole of monarch_attention_torch,
// ma/ma_torch.py:65-108).
//
// A team of G workgroups works on one head at a time.  Each half step of the
// head is a phase: the team's workgroups split the phase's block problems (R:
// key blocks m, L / Z: in-block positions j) and hand the result over to the
// next phase through a team barrier, because the next phase reads it transposed
// (aL, Y are written per key block and read per position; aR the other way
// round).  Where the device holds a full-width team for every head at once (the
// metric workload: 16 heads x 64 workgroups) every workgroup runs exactly one
// block problem per phase, like the per-stage launches do - without their launch
// boundaries, which cost 2-5 us each.  Workgroup ids are mapped so that a team's
// members share an XCD (ids are dealt round-robin to the 8 XCDs).
//
// The barrier keeps two words per team on DIFFERENT cache lines of the
// workspace's sync area: an arrival counter and a release word.  A member
// arrives with one atomic add on the counter; the member whose add completes the
// count stores the barrier's epoch into the release word, and that word - written
// once per barrier - is the only thing anybody polls.  (Polling words that other
// members are still writing makes the memory channel of that line crawl for
// everybody: a forward of the metric workload took 31 us with per-member flags
// polled by every waiter and 16 us with this scheme.)  Epochs and counts only
// grow: a launch continues from what the previous launch on the same workspace
// recorded, so the sync area needs zeroing once, never between calls.  Every wait
// is bounded (spin_limit polls).  A workgroup that gives up raises the sync area's
// error word, computes nothing more, writes NaN into the output rows it owns and
// still arrives at every barrier, so the grid always drains and the counters stay
// consistent for the next launch.  The grid never exceeds what is co-resident on
// the device (checked by the launcher), which is what makes waiting on other
// workgroups safe.
#pragma once

#include "ma_mfma.h"

namespace ma {
namespace mfma {

struct FusedPlan {
    int G;            // workgroups per team
    int nteams;       // teams (each loops over heads team, team + nteams, ...)
    int xcd_map;      // 1: members of a team share an XCD (nteams % 8 == 0)
    unsigned spin_limit;
};

constexpr int kSyncHeader = 32;    // words: [1] error
constexpr int kMaxTeamSize = 128;  // members per team
// words of a team sector, one 128-byte line each: recorded epoch and count | counter | release word |
// (unused) | XCC ids (four lines)
constexpr int kSyncLine = 32;
constexpr int kSyncCount = 1 * kSyncLine, kSyncGo = 2 * kSyncLine, kSyncXcc = 4 * kSyncLine;
constexpr int kSyncStride = 8 * kSyncLine;
constexpr int kMaxTeams = 1024;    // teams of more than one workgroup
constexpr int kSyncWords = kSyncHeader + kSyncStride * kMaxTeams;
static_assert(static_cast<uint64_t>(kSyncWords) * 4 == kTeamSyncBytes, "sync area size mismatch");
static_assert(kSyncXcc + kMaxTeamSize <= kSyncStride, "XCC ids must fit the team sector");

template <class T, int DT, int NTB, int NTM, int W>
struct FusedLds {
    static constexpr size_t r = Split<NTB, W>::PPW * Lds<T, DT, NTB>::R;
    static constexpr size_t l = Split<NTM, W>::PPW * Lds<T, DT, NTM>::L;
    static constexpr size_t z = Split<NTM, W>::PPW * Lds<T, DT, NTM>::Z;
    static constexpr size_t bytes = r > l ? (r > z ? r : z) : (l > z ? l : z);
};

// Barrier state of one team; every thread keeps a copy, all copies agree.
struct TeamSync {
    unsigned* base;        // team sector: [0] epoch, [1] arrival count the previous launch reached
    unsigned* count;       // arrivals so far
    unsigned* go;          // epoch of the latest complete barrier
    unsigned* xcc;         // [member] XCC (XCD) id the member runs on
    unsigned* error;
    unsigned* host_error;
    unsigned* word;        // LDS word through which wave 0 tells the workgroup how a wait ended
    unsigned epoch;        // epoch of this member's latest arrival
    unsigned target;       // value of the counter when that barrier is complete
    unsigned spin_limit;
    int G, member;
    int mode;              // 0 not decided yet, 1 members share an XCD, 2 they do not
    bool failed;           // a wait of this workgroup ran out: no more arithmetic, NaN output
};

__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

// Phase hand-over inside a team.  Data is written with ordinary stores
// (write-through L1 -> the XCD's L2) and read with streaming loads that never
// hit in L1.
//  * One workgroup per team: a workgroup barrier is all it takes.
//  * Members on ONE XCD (the normal case, checked at run time through the XCC
//    ids the members publish before they first arrive): they share the L2, so
//    publishing needs only "my stores are acknowledged" (vmcnt(0)).
//  * Members on several XCDs: agent-scope release / acquire fences (L2
//    write-back and invalidate) as well, which is correct anywhere but slow.
// The first wait decides: up to then everybody arrives the cheap way; the wait
// compares the (by then complete) XCC ids, and if the team turns out to be split
// all members - they all see the same ids - arrive again with the strong release
// and wait for that second round before they read anything.

// one thread: count this member in; whoever completes the count releases the barrier
__device__ __forceinline__ void publish_arrival(const TeamSync& ts) {
    const unsigned old = __hip_atomic_fetch_add(ts.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old + 1u == ts.target) __hip_atomic_store(ts.go, ts.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void team_arrive(TeamSync& ts) {
    if (ts.G == 1) return;
    // every wave's own stores have reached L2 before thread 0 publishes the arrival
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    ts.epoch += 1;
    ts.target += static_cast<unsigned>(ts.G);
    if (threadIdx.x == 0) {
        if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        publish_arrival(ts);
    }
}

// one thread: poll the release word until the barrier of ts.epoch is complete; false if the wait ran out
__device__ __forceinline__ bool poll_release(const TeamSync& ts) {
    unsigned spins = 0;
    if (ts.spin_limit == 0u) {   // failure-path tests: give up without looking, whatever the word holds
        raise_error(ts.error, ts.host_error, 1u);
        return false;
    }
    for (;;) {
        const unsigned f = __hip_atomic_load(ts.go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (static_cast<int>(f - ts.epoch) >= 0) return true;
        if (++spins > ts.spin_limit) {
            raise_error(ts.error, ts.host_error, 1u);
            return false;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

// All threads call it; every thread leaves with the same ts.
__device__ __forceinline__ void team_wait(TeamSync& ts) {
    if (ts.G == 1) {
        // producer and consumer waves share the CU: the stores only have to be
        // acknowledged by L2 before the (L1-bypassing) loads behind the barrier
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        return;
    }
    // LDS word: bit 0 = a wait ran out, bits 1.. = mode
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        bool bad = ts.failed;   // after a wait that ran out the workgroup only keeps the counters going
        if (lane == 0 && !bad) bad = !poll_release(ts);
        int mode = ts.mode;
        if (mode == 0) {   // the arrivals are complete, and so are the ids
            const unsigned mine = __hip_atomic_load(ts.xcc + ts.member, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned a = lane < ts.G ? __hip_atomic_load(ts.xcc + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : mine;
            const unsigned b = lane + 64 < ts.G ? __hip_atomic_load(ts.xcc + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : mine;
            mode = __builtin_amdgcn_ballot_w64(a != mine || b != mine) == 0 ? 1 : 2;
        }
        if (lane == 0) *ts.word = (bad ? 1u : 0u) | (static_cast<unsigned>(mode) << 1);
    }
    __syncthreads();
    const unsigned w = *ts.word;
    const int mode = static_cast<int>(w >> 1);
    ts.failed = (w & 1u) != 0u;
    if (ts.mode == 0 && mode == 2) {
        // split team: hand everything over again, the strong way (all members do: they read the same ids)
        ts.mode = 2;
        ts.epoch += 1;
        ts.target += static_cast<unsigned>(ts.G);
        __syncthreads();   // everybody has read the LDS word
        if (threadIdx.x == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            publish_arrival(ts);
            const bool bad = ts.failed || !poll_release(ts);
            *ts.word = (bad ? 1u : 0u) | (2u << 1);
        }
        __syncthreads();
        ts.failed = (*ts.word & 1u) != 0u;
    }
    ts.mode = mode;
    if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// One phase of one head: p even = R step (p = 0 reads Q, the last one forms Y), p odd = L step,
// p = 2T-1 = Z step.  The loads that depend only on the inputs (K / V tiles, Q rows, mask bytes) of
// the workgroup's first task are issued BEFORE it waits for the previous phase.  Every member
// takes part in the wait, also one without a task in this phase (the split-team hand-over counts
// on all of them).
template <class T, int DT, int NTB, int NTM, int W>
__device__ __forceinline__ void run_phase(const Problem& P, char* smem, int p, int head, TeamSync& ts, bool wait, int wave, int lane) {
    using RP = RProb<T, DT, NTB>;
    using LP = LProb<T, DT, NTM>;
    using ZP = ZProb<T, DT, NTM>;
    const int e = static_cast<unsigned>(head) / static_cast<unsigned>(P.H), h = static_cast<unsigned>(head) % static_cast<unsigned>(P.H);
    const int nph = 2 * P.T;
    const int G = ts.G, member = ts.member;
    // the tensor slices are made inside each branch: a phase only keeps the resources it uses
    if (p == nph - 1) {
        const Slices S = make_slices<T>(P, e, h, head);
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.B + PPW - 1) / PPW;
        char* sm = smem + slot * Lds<T, DT, NTM>::Z;
        bool first = true;
        for (int task = member; task < tasks || first; task += G) {
            const int j = task * PPW + slot;
            const bool active = task < tasks && slot < PPW && j < P.B;
            typename ZP::Pre pre;
            typename ZP::St st;
            if (!ts.failed) ZP::template issue<true>(P, S, pre, active, active ? j : 0, wig, lane);
            if (first && wait) team_wait(ts);
            first = false;
            if (ts.failed) {
                // this workgroup gave up on a wait: the state it would read is not known to be complete.
                // Nothing is computed; the output rows it owns are filled with NaN so that the failure shows.
                if (active) z_poison<T, DT, NTM>(P, S, j, wig, lane);
                continue;
            }
            ZP::state(P, S, st, active, active ? j : 0, wig, lane);
            ZP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
            __syncthreads();  // the LDS tiles are reused by the next task
        }
    } else if (p & 1) {
        const Slices S = make_slices<T>(P, e, h, head);
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.B + PPW - 1) / PPW;
        char* sm = smem + slot * Lds<T, DT, NTM>::L;
        bool first = true;
        for (int task = member; task < tasks || first; task += G) {
            const int j = task * PPW + slot;
            const bool active = task < tasks && slot < PPW && j < P.B;
            typename LP::Pre pre;
            typename LP::St st;
            if (!ts.failed) LP::template issue<true>(P, S, pre, active, e, active ? j : 0, wig, lane);
            if (first && wait) team_wait(ts);
            first = false;
            if (ts.failed) continue;
            LP::state(P, S, st, active, active ? j : 0, wig, lane);
            LP::run(P, S, sm, pre, st, active, active ? j : 0, wig, lane);
            __syncthreads();
        }
    } else {
        const Slices S = make_slices<T>(P, e, h, head);
        constexpr int WPP = Split<NTB, W>::WPP, PPW = Split<NTB, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.M + PPW - 1) / PPW;
        const bool first_step = p == 0, with_v = p == nph - 2;
        char* sm = smem + slot * Lds<T, DT, NTB>::R;
        bool first = true;
        for (int task = member; task < tasks || first; task += G) {
            const int m = task * PPW + slot;
            const bool active = task < tasks && slot < PPW && m < P.M;
            typename RP::Pre pre;
            typename RP::St st;
            if (!ts.failed) RP::template issue<true>(P, S, pre, active, e, active ? m : 0, first_step, with_v, wig, lane);
            if (first && wait) team_wait(ts);
            first = false;
            if (ts.failed) continue;
            RP::state(P, S, st, active, active ? m : 0, first_step, wig, lane);
            RP::run(P, S, sm, pre, st, active, active ? m : 0, first_step, with_v, wig, lane);
            __syncthreads();
        }
    }
}

template <class T, int DT, int NTB, int NTM, int W>
__global__ __launch_bounds__(64 * W) void fused_fwd_mfma(Problem P, FusedPlan plan) {
    warm_args(P);
    warm_args(plan);
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ unsigned team_word;   // how wave 0's wait ended, for the whole workgroup
    const int wave = wave_id(), lane = threadIdx.x & 63;
    const int G = plan.G;
    int team, member;
    if (plan.xcd_map) {
        const int xcd = blockIdx.x & 7, ix = blockIdx.x >> 3;
        team = (ix / G) * 8 + xcd;
        member = ix % G;
    } else {
        team = blockIdx.x / G;
        member = blockIdx.x % G;
    }
    const int heads = P.E * P.H;   // E * H * Np fits int32 (validated by the host)
    if (team >= heads) return;     // the grid is rounded up to whole teams per XCD; nobody waits for a team without heads
    TeamSync ts;
    ts.base = P.sync + kSyncHeader + kSyncStride * team;
    ts.count = ts.base + kSyncCount;
    ts.go = ts.base + kSyncGo;
    ts.xcc = ts.base + kSyncXcc;
    ts.error = P.sync + 1;
    ts.host_error = P.host_error;
    ts.word = &team_word;
    ts.spin_limit = plan.spin_limit;
    ts.G = G;
    ts.member = member;
    ts.mode = 0;
    ts.epoch = 0;
    ts.target = 0;
    ts.failed = false;
    if (G > 1) {
        // epochs and counts continue where the previous launch on this workspace stopped (the team
        // size may differ from that launch's, so the count is recorded, not derived from the epoch)
        ts.epoch = __hip_atomic_load(ts.base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ts.target = __hip_atomic_load(ts.base + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) __hip_atomic_store(ts.xcc + member, xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const int nph = 2 * P.T;

    // heads of this team: team, team + nteams, ...; every head has state arrays of its own in the
    // workspace, so only the phases of one head wait for each other
    for (int head = team; head < heads; head += plan.nteams) {
#pragma nounroll
        for (int p = 0; p < nph; ++p) {
            // The problem description is re-read from the kernel arguments in every phase (through an
            // offset the compiler cannot see through): otherwise all of it, and everything derived
            // from the head alone (ten buffer resources), is loaded once in front of the loops and
            // kept in scalar registers across all phases - over a hundred of them spill.
            int zero = 0;
            asm volatile("" : "+s"(zero));
            const Problem& Q = *reinterpret_cast<const Problem*>(reinterpret_cast<const char*>(&P) + zero);
            // Likewise the lane and wave indices: every per-lane address of all three kinds of block
            // problems is invariant across phases and would be kept in vector registers side by side.
            int ln = lane, wv = wave;
            asm volatile("" : "+v"(ln));
            asm volatile("" : "+s"(wv));
            run_phase<T, DT, NTB, NTM, W>(Q, smem, p, head, ts, p != 0, wv, ln);
            if (p < nph - 1) team_arrive(ts);
        }
    }
    // Every member has read the team's recorded epoch and count before it first arrived, and all
    // waits of this launch are behind member 0 here: record where the next launch on this
    // workspace continues.
    if (G > 1 && member == 0 && threadIdx.x == 0) {
        __hip_atomic_store(ts.base, ts.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ts.base + 1, ts.target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace mfma
}  // namespace ma
