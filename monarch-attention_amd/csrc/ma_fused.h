// Fused forward: all T alternating steps, the product with V and the output
// stage in ONE launch (the whole of monarch_attention_torch,
// ma/ma_torch.py:65-108).
//
// A team of G workgroups works on its heads two at a time.  Each half step of a
// head is a phase: the team's workgroups split the phase's block problems (R:
// key blocks m, L / Z: in-block positions j) and hand the result over to the
// next phase through a team barrier, because the next phase reads it transposed
// (aL, Y are written per key block and read per position; aR the other way
// round).  The barrier is split into arrive and wait, and the team alternates
// between its two heads, so the wait for one head is covered by a phase of the
// other.  The state lives in two per-TEAM slots of the workspace which are
// reused head after head, so it stays resident in the L2 of the XCD the team
// runs on instead of streaming to HBM.  Workgroup ids are mapped so that a team's members share an XCD (ids are
// dealt round-robin to the 8 XCDs).
//
// The barrier uses one flag word per member in the workspace's sync area: a
// member arrives by storing the barrier's epoch into its flag, and waits by
// polling all G flags with one wave (see team_barrier for the fences).  Epochs
// only grow: a launch continues from the epoch the previous launch on the same
// workspace recorded, so the sync area needs zeroing once, never between calls.
// Every wait is bounded (spin_limit polls); a workgroup that gives up raises
// the sync area's error word and still runs to the end, so the grid always
// drains.  The grid never exceeds what is co-resident on the device (checked by
// the launcher), which is what makes waiting on other workgroups safe.
#pragma once

#include "ma_mfma.h"

namespace ma {
namespace mfma {

struct FusedPlan {
    int G;            // workgroups per team
    int nteams;       // teams (each loops over heads team, team + nteams, ...)
    int xcd_map;      // 1: members of a team share an XCD (grid % (8 G) == 0)
    unsigned spin_limit;
};

constexpr int kSyncHeader = 16;    // words: [1] error
constexpr int kMaxTeamSize = 64;   // members per team (one polling lane each)
constexpr int kSyncFlags = 16;     // offset of the flag words inside a team sector
constexpr int kSyncStride = kSyncFlags + 3 * kMaxTeamSize;  // words per team: base epochs, flags of slot 0 / 1, XCC ids
constexpr int kMaxTeams = 1024;    // teams of more than one workgroup
constexpr int kSyncWords = kSyncHeader + kSyncStride * kMaxTeams;
static_assert(static_cast<uint64_t>(kSyncWords) * 4 == kTeamSyncBytes, "sync area size mismatch");

template <class T, int DT, int NTB, int NTM, int W>
struct FusedLds {
    static constexpr size_t r = Split<NTB, W>::PPW * Lds<T, DT, NTB>::R;
    static constexpr size_t l = Split<NTM, W>::PPW * Lds<T, DT, NTM>::L;
    static constexpr size_t z = Split<NTM, W>::PPW * Lds<T, DT, NTM>::Z;
    static constexpr size_t bytes = r > l ? (r > z ? r : z) : (l > z ? l : z);
};

// Barrier state of one team.  A team keeps TWO heads in flight (slots 0 and 1),
// each with its own flag array and epoch, and alternates between them phase by
// phase: while the arrival flags of one head travel through a loaded memory
// system (several microseconds), the members work on the other head.
struct TeamSync {
    unsigned* base;        // team sector: [0], [1] epochs reached by the previous launch (slot 0, 1)
    unsigned* flags[2];    // [slot][member] epoch of the member's latest arrival
    unsigned* xcc;         // [member] XCC (XCD) id the member runs on
    unsigned* error;
    unsigned epoch[2];     // epoch of the latest arrival per slot
    bool pending[2];       // arrived on the slot, not yet waited for it
    unsigned spin_limit;
    int G, member;
    int mode;              // 0 not decided yet, 1 members share an XCD, 2 they do not
};

__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

// Phase hand-over inside a team.  Data is written with ordinary stores
// (write-through L1 -> the XCD's L2) and read with streaming loads that never
// hit in L1.  Arrival is one relaxed store per member into its own flag word -
// nobody performs a read-modify-write, so arrivals never queue behind each
// other - and waiting is one wave polling all G flags (lane i watches member i).
//  * One workgroup per team: a workgroup barrier is all it takes.
//  * Members on ONE XCD (the normal case, checked at run time through the XCC
//    ids the members publish before they first arrive): they share the L2, so
//    publishing needs only "my stores are acknowledged" (vmcnt(0)).  No L2
//    write-back, no invalidate: the state stays in L2.
//  * Members on several XCDs: agent-scope release / acquire fences (L2
//    write-back and invalidate) as well, which is correct anywhere but slow.
// The first wait decides: up to then everybody arrives the cheap way; the wait
// compares the (by then complete) XCC ids, and if the team turns out to be split
// all members - they all see the same ids - publish again with the strong
// release (for both slots, if the other one has an arrival outstanding) and wait
// for that second round before they read anything.
__device__ __forceinline__ void team_arrive(TeamSync& ts, int slot) {
    if (ts.G == 1) return;
    // every wave's own stores have reached L2 before wave 0 publishes the arrival
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x < 64) {   // wave 0 keeps the barrier state (uniform across its lanes)
        if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        ts.epoch[slot] += 1;
        ts.pending[slot] = true;
        if (threadIdx.x == 0)
            __hip_atomic_store(ts.flags[slot] + ts.member, ts.epoch[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// wave 0: poll until every member's flag of `slot` has reached ts.epoch[slot]
__device__ __forceinline__ void poll_flags(TeamSync& ts, int slot, int lane) {
    const unsigned want = ts.epoch[slot];
    unsigned spins = 0;
    for (;;) {
        const unsigned f = lane < ts.G ? __hip_atomic_load(ts.flags[slot] + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : want;
        if (__builtin_amdgcn_ballot_w64(static_cast<int>(f - want) < 0) == 0) break;
        __builtin_amdgcn_s_sleep(2);
        if (++spins > ts.spin_limit) {
            if (lane == 0) __hip_atomic_store(ts.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
    }
}

__device__ __forceinline__ void team_wait(TeamSync& ts, int slot) {
    if (ts.G == 1) {
        // producer and consumer waves share the CU: the stores only have to be
        // acknowledged by L2 before the (L1-bypassing) loads behind the barrier
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        return;
    }
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        poll_flags(ts, slot, lane);
        if (ts.mode == 0) {
            const unsigned mine = __hip_atomic_load(ts.xcc + ts.member, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned x = lane < ts.G ? __hip_atomic_load(ts.xcc + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : mine;
            ts.mode = (__builtin_amdgcn_ballot_w64(x != mine) == 0) ? 1 : 2;
            if (ts.mode == 2) {  // split team: hand everything outstanding over again, the strong way
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
                const int other = slot ^ 1;
                ts.epoch[slot] += 1;
                if (ts.pending[other]) ts.epoch[other] += 1;
                if (lane == 0) {
                    __hip_atomic_store(ts.flags[slot] + ts.member, ts.epoch[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (ts.pending[other])
                        __hip_atomic_store(ts.flags[other] + ts.member, ts.epoch[other], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                poll_flags(ts, slot, lane);
            }
        }
        if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        ts.pending[slot] = false;
    }
    __syncthreads();
}

// One phase of one head: p even = R step (p = 0 reads Q, the last one forms Y),
// p odd = L step, p = 2T-1 = Z step.
template <class T, int DT, int NTB, int NTM, int W>
__device__ __forceinline__ void run_phase(const Problem& P, char* smem, int p, long long head, long long slot_ws, int member,
                                          int G, int wave, int lane) {
    const int e = head / P.H, h = head % P.H;
    const int nph = 2 * P.T;
    if (p == nph - 1) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.B + PPW - 1) / PPW;
        for (int task = member; task < tasks; task += G) {
            const int j = task * PPW + slot;
            const bool active = j < P.B;
            z_problem<T, DT, NTM>(P, smem + slot * Lds<T, DT, NTM>::Z, active, e, h, slot_ws, active ? j : 0, wig, lane);
            __syncthreads();  // the LDS tiles are reused by the next task
        }
    } else if (p & 1) {
        constexpr int WPP = Split<NTM, W>::WPP, PPW = Split<NTM, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.B + PPW - 1) / PPW;
        for (int task = member; task < tasks; task += G) {
            const int j = task * PPW + slot;
            const bool active = j < P.B;
            l_problem<T, DT, NTM>(P, smem + slot * Lds<T, DT, NTM>::L, active, e, h, slot_ws, active ? j : 0, wig, lane);
            __syncthreads();
        }
    } else {
        constexpr int WPP = Split<NTB, W>::WPP, PPW = Split<NTB, W>::PPW;
        const int slot = wave / WPP, wig = wave % WPP;
        const int tasks = (P.M + PPW - 1) / PPW;
        for (int task = member; task < tasks; task += G) {
            const int m = task * PPW + slot;
            const bool active = m < P.M;
            r_problem<T, DT, NTB>(P, smem + slot * Lds<T, DT, NTB>::R, active, e, h, slot_ws, active ? m : 0, p == 0,
                                  p == nph - 2, wig, lane);
            __syncthreads();
        }
    }
}

template <class T, int DT, int NTB, int NTM, int W>
__global__ __launch_bounds__(64 * W) void fused_fwd_mfma(Problem P, FusedPlan plan) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
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
    TeamSync ts;
    ts.base = P.sync + kSyncHeader + kSyncStride * team;
    ts.flags[0] = ts.base + kSyncFlags;
    ts.flags[1] = ts.flags[0] + kMaxTeamSize;
    ts.xcc = ts.flags[1] + kMaxTeamSize;
    ts.error = P.sync + 1;
    ts.spin_limit = plan.spin_limit;
    ts.G = G;
    ts.member = member;
    ts.mode = 0;
    ts.epoch[0] = ts.epoch[1] = 0;
    ts.pending[0] = ts.pending[1] = false;
    if (G > 1) {
        // epochs continue where the previous launch on this workspace stopped
        ts.epoch[0] = __hip_atomic_load(ts.base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ts.epoch[1] = __hip_atomic_load(ts.base + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) __hip_atomic_store(ts.xcc + member, xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const long long heads = static_cast<long long>(P.E) * P.H;
    const int nph = 2 * P.T;

    // heads of this team: team, team + nteams, ...; a multi-workgroup team pairs consecutive
    // ones on slots 0 / 1, a single workgroup (nothing to wait for) takes them one by one
    const long long stride = (G > 1 ? 2ll : 1ll) * plan.nteams;
    const long long ws_a = G > 1 ? 2ll * team : team, ws_b = ws_a + 1;  // state slots in the workspace
    for (long long hA = team; hA < heads; hA += stride) {
        const long long hB = hA + plan.nteams;
        const bool has_b = G > 1 && hB < heads;
        const bool first_pair = hA == team;
        const bool more_a = hA + stride < heads, more_b = hB + stride < heads;
        for (int p = 0; p < nph; ++p) {
            // a phase may start once every member has finished the previous phase on the same slot
            // (it reads what they wrote, or overwrites what they were reading)
            if (!(first_pair && p == 0)) team_wait(ts, 0);
            run_phase<T, DT, NTB, NTM, W>(P, smem, p, hA, ws_a, member, G, wave, lane);
            if (p < nph - 1 || more_a) team_arrive(ts, 0);
            if (has_b) {
                if (!(first_pair && p == 0)) team_wait(ts, 1);
                run_phase<T, DT, NTB, NTM, W>(P, smem, p, hB, ws_b, member, G, wave, lane);
                if (p < nph - 1 || more_b) team_arrive(ts, 1);
            }
        }
    }
    // Every member has read the team's base epochs before it first arrived, and all
    // waits of this launch are behind member 0 here: record where the next launch on
    // this workspace continues.
    if (G > 1 && member == 0 && threadIdx.x == 0) {   // thread 0 is in wave 0, which keeps the epochs
        __hip_atomic_store(ts.base, ts.epoch[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ts.base + 1, ts.epoch[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace mfma
}  // namespace ma
