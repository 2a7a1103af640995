// Host-side planning and dispatch of the fused forward kernel.  Included by one
// .hip file per (dtype, head-dim class) so the instantiations compile in parallel.
#pragma once

#include <type_traits>

#include "ma_fused.h"
#include "ma_mfma_launch.h"

namespace ma {
namespace mfma {

// Team size and team count for `heads` heads when `capacity` workgroups are co-resident: as many
// workgroups per head as there are tasks in the widest phase if all heads can then run at once,
// else narrower teams (tasks dealt evenly) and, below one workgroup per head, teams of one that
// take the heads in turn.  Teams of several workgroups come in multiples of 8, so that the ids
// x, x + 8, ... of a team sit on one XCD; the grid is rounded up, surplus teams have no head.
inline FusedPlan plan_teams(long long heads, int tasks_r, int tasks_l, int capacity) {
    FusedPlan pl;
    const int widest = tasks_r > tasks_l ? tasks_r : tasks_l;
    const long long heads8 = (heads + 7) / 8 * 8;
    long long g = capacity / heads8;
    if (g > widest) g = widest;
    if (g > kMaxTeamSize) g = kMaxTeamSize;
    if (g < 1) g = 1;
    const int per_wg = static_cast<int>((widest + g - 1) / g);
    pl.G = (widest + per_wg - 1) / per_wg;
    long long nteams = pl.G > 1 ? heads8 : (heads < capacity ? heads : capacity);
    pl.nteams = static_cast<int>(nteams);
    pl.xcd_map = (pl.G > 1 && pl.nteams % 8 == 0) ? 1 : 0;
    pl.spin_limit = 1u << 18;   // a legitimate wait lasts one phase of one head (well under a millisecond)
    return pl;
}

template <class T, int DT, int NTB, int NTM, int W>
int launch_fused_w(const Problem& P, bool sync_ready, hipStream_t s) {
    using FL = FusedLds<T, DT, NTB, NTM, W>;
    if (FL::bytes > 160 * 1024) return MA_ERR_UNSUPPORTED;
    auto kernel = fused_fwd_mfma<T, DT, NTB, NTM, W>;
    const int lds_err = set_lds_limit(kernel, FL::bytes);
    if (lds_err) return lds_err;
    const DeviceCaps dc = device_caps(kernel, 64 * W, FL::bytes);
    if (dc.err) return dc.err;
    const int capacity = dc.cus * dc.per_cu;
    if (capacity < 1) return MA_ERR_UNSUPPORTED;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const int tasks_r = (P.M + Split<NTB, W>::PPW - 1) / Split<NTB, W>::PPW;
    const int tasks_l = (P.B + Split<NTM, W>::PPW - 1) / Split<NTM, W>::PPW;
    FusedPlan pl = plan_teams(heads, tasks_r, tasks_l, capacity);
    if (P.test_no_spin) pl.spin_limit = 0;
    // the grid must be co-resident (workgroups wait for each other) and the teams need their sync sectors
    if (pl.nteams < 1 || pl.G < 1 || pl.G > kMaxTeamSize) return MA_ERR_UNSUPPORTED;
    if (static_cast<long long>(pl.nteams) * pl.G > capacity) return MA_ERR_UNSUPPORTED;
    if (pl.G > 1 && pl.nteams > kMaxTeams) return MA_ERR_UNSUPPORTED;
    if (!sync_ready) {
        const int err = launch_zero_sync(P.sync, s);
        if (err) return err;
    }
    hipLaunchKernelGGL((fused_fwd_mfma<T, DT, NTB, NTM, W>), dim3(pl.nteams * pl.G), dim3(64 * W), FL::bytes, s, P, pl);
    return static_cast<int>(hipGetLastError());
}

template <class T, int DT, int NTB, int NTM>
int launch_fused_one(const Problem& P, bool sync_ready, hipStream_t s) {
    return launch_fused_w<T, DT, NTB, NTM, kWaves>(P, sync_ready, s);
}

template <class T, int DT>
int launch_fused(const Problem& P, bool sync_ready, hipStream_t s) {
    const int ntb = nt_class_one_launch(P.B), ntm = nt_class_one_launch(P.M);
#define MA_NTM(NB)                                                              \
    switch (ntm) {                                                              \
        case 1: return launch_fused_one<T, DT, NB, 1>(P, sync_ready, s);        \
        case 2: return launch_fused_one<T, DT, NB, 2>(P, sync_ready, s);        \
        case 3: return launch_fused_one<T, DT, NB, 3>(P, sync_ready, s);        \
        case 4: return launch_fused_one<T, DT, NB, 4>(P, sync_ready, s);        \
        default: return launch_fused_one<T, DT, NB, 8>(P, sync_ready, s);       \
    }
    switch (ntb) {
        case 1: MA_NTM(1)
        case 2: MA_NTM(2)
        case 3: MA_NTM(3)
        case 4: MA_NTM(4)
        default: MA_NTM(8)
    }
#undef MA_NTM
}

}  // namespace mfma
}  // namespace ma
