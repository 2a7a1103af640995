// One-launch fp32 forward for small heads (state in LDS), see ma_head32.h.
#include "ma_head32.h"
#include "ma_head32_t1.h"
#include "ma_mfma_launch.h"

namespace ma {
namespace {

template <int DTF>
int launch_head32_dtf(const Problem& P, bool dry_run, hipStream_t s) {
    using HG = mfma32::Head32<DTF>;
    static_assert(HG::lds_bytes <= 160 * 1024, "two state tiles and the statistics must fit the LDS of a CU");
    if (dry_run) return MA_OK;
    auto kernel = mfma32::head_fwd_f32<DTF>;
    const int lds_err = mfma::set_lds_limit(kernel, HG::lds_bytes);
    if (lds_err) return lds_err;
    const mfma::DeviceCaps caps = mfma::device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long grid = heads < caps.cus ? heads : caps.cus;
    hipLaunchKernelGGL((mfma32::head_fwd_f32<DTF>), dim3(grid), dim3(64 * HG::W), HG::lds_bytes, s, P);
    return static_cast<int>(hipGetLastError());
}

template <int DTF>
int launch_head32_t1_dtf(const Problem& P, hipStream_t s) {
    using HG = mfma32::HeadT1<DTF>;
    static_assert(HG::lds_bytes <= 160 * 1024, "the head's K and V tiles and the row tiles must fit the LDS of a CU");
    auto kernel = mfma32::head_t1_f32<DTF>;
    const int lds_err = mfma::set_lds_limit(kernel, HG::lds_bytes);
    if (lds_err) return lds_err;
    const long long grid = static_cast<long long>(P.E) * P.H * P.B;
    hipLaunchKernelGGL((mfma32::head_t1_f32<DTF>), dim3(grid), dim3(256), HG::lds_bytes, s, P);
    return static_cast<int>(hipGetLastError());
}

}  // namespace

// dry_run: only report whether the problem fits (MA_OK / MA_ERR_UNSUPPORTED), launch nothing
int launch_head32(const Problem& P, bool dry_run, hipStream_t s) {
    if (P.B > 16 || P.M > 16 || P.D > 64 || P.D % 4 != 0 || P.Dv != P.D) return MA_ERR_UNSUPPORTED;
    if (!dry_run && head32_single_step(P)) {   // few heads, one step: a workgroup per (head, position), no exchange
        if (P.D <= 32) return launch_head32_t1_dtf<2>(P, s);
        if (P.D <= 48) return launch_head32_t1_dtf<3>(P, s);
        return launch_head32_t1_dtf<4>(P, s);
    }
    if (P.D <= 32) return launch_head32_dtf<2>(P, dry_run, s);
    if (P.D <= 48) return launch_head32_dtf<3>(P, dry_run, s);
    return launch_head32_dtf<4>(P, dry_run, s);
}

}  // namespace ma
