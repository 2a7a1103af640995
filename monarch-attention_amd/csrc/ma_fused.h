// Fused forward: all T alternating steps, the product with V and the output
// stage in ONE launch (the whole of monarch_attention_torch,
// ma/ma_torch.py:65-108).
//
// A team of G workgroups owns one (e, h) head at a time.  Each half step is a
// phase: the team's workgroups split the phase's block problems (R: key blocks
// m, L / Z: in-block positions j), then meet at a team barrier, because the
// next phase reads the previous one's results transposed (aL, Y are written per
// key block and read per position; aR the other way round).  That state lives
// in a per-TEAM slot of the workspace which is reused head after head, so it
// stays resident in the L2 of the XCD the team runs on instead of streaming to
// HBM.  Workgroup ids are mapped so that a team's members share an XCD (ids are
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
    int debug;        // development knob: 1 = no waiting, 2 = no invalidate, 4 = sleep longer between polls
};

constexpr int kSyncHeader = 16;    // words: [1] error
constexpr int kMaxTeamSize = 64;   // members per team (one polling lane each)
constexpr int kSyncFlags = 16;     // offset of the flag words inside a team sector
constexpr int kSyncStride = kSyncFlags + 2 * kMaxTeamSize;  // words per team: base epoch, flags, XCC ids
constexpr int kMaxTeams = 1024;    // teams of more than one workgroup
constexpr int kSyncWords = kSyncHeader + kSyncStride * kMaxTeams;
static_assert(static_cast<uint64_t>(kSyncWords) * 4 == kSyncAreaBytes, "sync area size mismatch");

template <class T, int DT, int NTB, int NTM>
struct FusedLds {
    static constexpr size_t r = Split<NTB>::PPW * Lds<T, DT, NTB>::R;
    static constexpr size_t l = Split<NTM>::PPW * Lds<T, DT, NTM>::L;
    static constexpr size_t z = Split<NTM>::PPW * Lds<T, DT, NTM>::Z;
    static constexpr size_t bytes = r > l ? (r > z ? r : z) : (l > z ? l : z);
};

// Barrier state; wave 0 of the workgroup runs the protocol.
struct TeamSync {
    unsigned* base;      // team sector: [0] epoch reached by the previous launch
    unsigned* flags;     // [member] epoch of the member's latest arrival
    unsigned* xcc;       // [member] XCC (XCD) id the member runs on
    unsigned* error;
    unsigned epoch;      // epoch of the latest barrier
    unsigned spin_limit;
    int G, member;
    int mode;            // 0 not decided yet, 1 members share an XCD, 2 they do not
    int debug;
    unsigned long long* stamp;
};

__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

// wave 0: publish this member's arrival at ts.epoch and poll until every member's
// flag has reached it (lane i watches member i; G <= 64)
__device__ __forceinline__ void arrive_and_wait(TeamSync& ts, int lane) {
    if (lane == 0) __hip_atomic_store(ts.flags + ts.member, ts.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (ts.debug & 1) return;
    unsigned spins = 0;
    for (;;) {
        const unsigned f = lane < ts.G ? __hip_atomic_load(ts.flags + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : ts.epoch;
        const bool here = static_cast<int>(f - ts.epoch) >= 0;
        if (__builtin_amdgcn_ballot_w64(!here) == 0) break;
        __builtin_amdgcn_s_sleep(1);
        if (++spins > ts.spin_limit) {
            if (lane == 0) __hip_atomic_store(ts.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
    }
}

// Team barrier.  Data handed over at a barrier is written with ordinary stores
// (write-through L1 -> the XCD's L2) and read with ordinary loads.  Arrival is
// one plain (atomic, relaxed) store per member into its own flag word; nobody
// performs a read-modify-write, so arrivals never queue behind each other.
//  * One workgroup per team: a workgroup barrier is all it takes.
//  * Members on ONE XCD (the normal case, checked at run time through the XCC
//    ids the members publish before they first arrive): they share the L2, so
//    publishing needs only "my stores are acknowledged" (vmcnt(0)); consumers
//    read the shared state with L1-bypassing loads.  No L2 write-back, no
//    invalidate: the state stays in L2.
//  * Members on several XCDs: agent-scope release / acquire fences (L2
//    write-back and invalidate) as well, which is correct anywhere but slow.
// The first barrier decides: everybody arrives the cheap way, compares the (by
// then complete) XCC ids, and if the team turns out to be split all members -
// they all see the same ids - repeat the hand-over with the strong fence.
__device__ __forceinline__ void team_barrier(TeamSync& ts) {
    if (ts.G == 1) {
        __syncthreads();
        return;
    }
    // every wave's own stores have reached L2 before wave 0 publishes the arrival
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if ((ts.debug & 8) && threadIdx.x == 0 && ts.stamp) *ts.stamp++ = wall_clock64();
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        ts.epoch += 1;
        arrive_and_wait(ts, lane);
        if (ts.mode == 0) {
            const unsigned mine = __hip_atomic_load(ts.xcc + ts.member, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned x = lane < ts.G ? __hip_atomic_load(ts.xcc + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : mine;
            ts.mode = (__builtin_amdgcn_ballot_w64(x != mine) == 0) ? 1 : 2;
            if (ts.mode == 2) {  // split team: hand the data over again, the strong way
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
                ts.epoch += 1;
                arrive_and_wait(ts, lane);
            }
        }
        // Shared state is read with streaming loads that never hit in L1, so the
        // same-XCD case needs no invalidate (which would also empty the L2).
        if (ts.mode == 2) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
}

template <class T, int DT, int NTB, int NTM>
__global__ __launch_bounds__(kThreads) void fused_fwd_mfma(Problem P, FusedPlan plan) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
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
    ts.flags = ts.base + kSyncFlags;
    ts.xcc = ts.flags + kMaxTeamSize;
    ts.error = P.sync + 1;
    ts.spin_limit = plan.spin_limit;
    ts.G = G;
    ts.member = member;
    ts.mode = 0;
    ts.debug = plan.debug;
    ts.epoch = 0;
    if (G > 1) {
        // epochs continue where the previous launch on this workspace stopped
        ts.epoch = __hip_atomic_load(ts.base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) __hip_atomic_store(ts.xcc + member, xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long slot_ws = team;  // this team's workspace slot
    unsigned long long* tstamp = reinterpret_cast<unsigned long long*>(P.stats) + 8ull * blockIdx.x;
    int tsi = 0;
    ts.stamp = nullptr;
#define MA_STAMP() do { if ((plan.debug & 8) && threadIdx.x == 0 && tsi < 8) { tstamp[tsi++] = wall_clock64(); ts.stamp = tstamp + tsi; tsi++; } } while (0)
    MA_STAMP();

    for (long long head = team; head < heads; head += plan.nteams) {
        const int e = head / P.H, h = head % P.H;
        for (int t = 0; t < P.T; ++t) {
            {   // R phase: key blocks m
                constexpr int WPP = Split<NTB>::WPP, PPW = Split<NTB>::PPW;
                const int slot = wave / WPP, wig = wave % WPP;
                const int tasks = (P.M + PPW - 1) / PPW;
                for (int task = member; task < tasks; task += G) {
                    const int m = task * PPW + slot;
                    const bool active = m < P.M;
                    r_problem<T, DT, NTB>(P, smem + slot * Lds<T, DT, NTB>::R, active, e, h, slot_ws, active ? m : 0,
                                          t == 0, t == P.T - 1, wig, lane);
                    __syncthreads();  // the LDS tiles are reused by the next task
                }
            }
            MA_STAMP();
            team_barrier(ts);
            MA_STAMP();
            if (t == P.T - 1) break;
            {   // L phase: in-block positions j
                constexpr int WPP = Split<NTM>::WPP, PPW = Split<NTM>::PPW;
                const int slot = wave / WPP, wig = wave % WPP;
                const int tasks = (P.B + PPW - 1) / PPW;
                for (int task = member; task < tasks; task += G) {
                    const int j = task * PPW + slot;
                    const bool active = j < P.B;
                    l_problem<T, DT, NTM>(P, smem + slot * Lds<T, DT, NTM>::L, active, e, h, slot_ws, active ? j : 0, wig, lane);
                    __syncthreads();
                }
            }
            team_barrier(ts);
        }
        {   // Z phase
            constexpr int WPP = Split<NTM>::WPP, PPW = Split<NTM>::PPW;
            const int slot = wave / WPP, wig = wave % WPP;
            const int tasks = (P.B + PPW - 1) / PPW;
            for (int task = member; task < tasks; task += G) {
                const int j = task * PPW + slot;
                const bool active = j < P.B;
                z_problem<T, DT, NTM>(P, smem + slot * Lds<T, DT, NTM>::Z, active, e, h, slot_ws, active ? j : 0, wig, lane);
                __syncthreads();
            }
        }
        if (head + plan.nteams < heads) {  // the slot is overwritten by the next head's R phase
            team_barrier(ts);
        }
    }

    MA_STAMP();
#undef MA_STAMP
    // Every member has read the team's base epoch before it first arrived, and
    // every barrier of this launch is behind member 0 here: record where the
    // next launch on this workspace continues.
    if (G > 1 && member == 0 && threadIdx.x == 0)
        __hip_atomic_store(ts.base, ts.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace mfma
}  // namespace ma
