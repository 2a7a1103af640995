// Host-side planning and dispatch of the chained forward kernel.  Included by one
// .hip file per (dtype, head-dim class) so the instantiations compile in parallel.
#pragma once

#include <type_traits>

#include "ma_chain.h"
#include "ma_mfma_launch.h"

namespace ma {
namespace mfma {

template <class T, int DT, int NTB, int NTM>
int launch_chain_one(const Problem& P, bool sync_ready, hipStream_t s) {
    constexpr int W = kWaves;
    using FL = FusedLds<T, DT, NTB, NTM, W>;   // the three kinds of block problems share one LDS allocation
    if (FL::bytes > 160 * 1024) return MA_ERR_UNSUPPORTED;
    auto kernel = chain_fwd_mfma<T, DT, NTB, NTM, W>;
    const int lds_err = set_lds_limit(kernel, FL::bytes);
    if (lds_err) return lds_err;
    const long long heads = static_cast<long long>(P.E) * P.H;
    ChainPlan pl;
    pl.hx = static_cast<int>((heads + 7) / 8);
    pl.tR = (P.M + Split<NTB, W>::PPW - 1) / Split<NTB, W>::PPW;
    const int per = NTM == 1 ? 16 >> P.pack_shift : 1;   // in-block positions per L / Z problem (heads of few blocks share tiles)
    pl.tL = ((P.B + per - 1) / per + Split<NTM, W>::PPW - 1) / Split<NTM, W>::PPW;
    pl.stride = chain_stride(P.T);
    pl.go_off = chain_go_offset(P.T);
    pl.spin_limit = P.test_no_spin ? 0u : 1u << 18;   // a legitimate wait lasts one phase of one head (well under a millisecond)
    // the task count of a phase is a 16-bit field of its arrival counter (and so are the sums of the
    // XCC ids: at most 15 and 225 per task); the heads' sync words must fit their part of the sync area;
    // the grid must stay a 31-bit count
    if (pl.tR > 128 || pl.tL > 128) return MA_ERR_UNSUPPORTED;
    if (heads * pl.stride > kChainWords) return MA_ERR_UNSUPPORTED;
    const long long grid = 8ll * pl.hx * P.T * (pl.tR + pl.tL);
    if (grid > 0x7fffffffll) return MA_ERR_UNSUPPORTED;
    if (!sync_ready) {
        const int err = launch_zero_sync(P.sync, s);
        if (err) return err;
    }
    hipLaunchKernelGGL((chain_fwd_mfma<T, DT, NTB, NTM, W>), dim3(static_cast<unsigned>(grid)), dim3(64 * W), FL::bytes, s, P, pl);
    return static_cast<int>(hipGetLastError());
}

template <class T, int DT>
int launch_chain(const Problem& P, bool sync_ready, hipStream_t s) {
    const int ntb = nt_class_chain(P.B), ntm = nt_class_chain(P.M);
#define MA_NTM(NB)                                                              \
    switch (ntm) {                                                              \
        case 1: return launch_chain_one<T, DT, NB, 1>(P, sync_ready, s);        \
        case 2: return launch_chain_one<T, DT, NB, 2>(P, sync_ready, s);        \
        case 3: return launch_chain_one<T, DT, NB, 3>(P, sync_ready, s);        \
        case 4: return launch_chain_one<T, DT, NB, 4>(P, sync_ready, s);        \
        case 6: return launch_chain_one<T, DT, NB, 6>(P, sync_ready, s);        \
        default: return launch_chain_one<T, DT, NB, 8>(P, sync_ready, s);       \
    }
    switch (ntb) {
        case 1: MA_NTM(1)
        case 2: MA_NTM(2)
        case 3: MA_NTM(3)
        case 4: MA_NTM(4)
        case 6: MA_NTM(6)
        default: MA_NTM(8)
    }
#undef MA_NTM
}

}  // namespace mfma
}  // namespace ma
