// Host-side dispatch of the fp32 MFMA stage kernels over (16-column groups DTF,
// strip count NWT).  Included by one .hip file per stage.
#pragma once

#include <type_traits>

#include "ma_mfma32.h"
#include "ma_mfma_launch.h"

namespace ma {
namespace mfma32 {

inline int dtf_class(int D) { return D <= 32 ? 2 : D <= 48 ? 3 : D <= 64 ? 4 : 8; }

template <class F>
int for_classes32(int dtf, int nt, F&& f) {
#define MA_NT(DTV)                                                                            \
    switch (nt) {                                                                             \
        case 1: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 1>{}); \
        case 2: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 2>{}); \
        case 4: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 4>{}); \
        default: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 8>{}); \
    }
    switch (dtf) {
        case 2: MA_NT(2)
        case 3: MA_NT(3)
        case 4: MA_NT(4)
        default: MA_NT(8)
    }
#undef MA_NT
}

constexpr size_t kLdsLimit = 160 * 1024;

inline int launch_r(const Problem& P, bool first, bool with_v, hipStream_t s) {
    return for_classes32(dtf_class(P.D), mfma::nt_class(P.B), [&](auto dt, auto nt) {
        constexpr int DTF = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr size_t lds = Lds32<DTF, NWT>::R;
        if (lds > kLdsLimit) return static_cast<int>(MA_ERR_UNSUPPORTED);
        const int attr = mfma::set_lds_limit(r_step_f32<DTF, NWT>, lds);
        if (attr) return attr;
        const long long problems = static_cast<long long>(P.E) * P.H * P.M;
        if constexpr (NWT == 8) {   // two strips per wave: as two workgroups each while that still leaves compute units idle
            const mfma::DeviceCaps caps = mfma::device_caps(r_step_f32<DTF, NWT>, 0, 0);
            if (caps.err) return caps.err;
            if (2 * problems <= caps.cus) {
                const int attr2 = mfma::set_lds_limit(r_step_f32<DTF, NWT, 2>, lds);
                if (attr2) return attr2;
                hipLaunchKernelGGL((r_step_f32<DTF, NWT, 2>), dim3(2 * problems), dim3(64 * Split<NWT>::WPP), lds, s, P, first ? 1 : 0, with_v ? 1 : 0);
                return static_cast<int>(hipGetLastError());
            }
        }
        hipLaunchKernelGGL((r_step_f32<DTF, NWT>), dim3(problems), dim3(64 * Split<NWT>::WPP), lds, s, P, first ? 1 : 0, with_v ? 1 : 0);
        return static_cast<int>(hipGetLastError());
    });
}

inline int launch_l(const Problem& P, hipStream_t s) {
    return for_classes32(dtf_class(P.D), mfma::nt_class(P.M), [&](auto dt, auto nt) {
        constexpr int DTF = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr size_t lds = Lds32<DTF, NWT>::L;
        if (lds > kLdsLimit) return static_cast<int>(MA_ERR_UNSUPPORTED);
        const int attr = mfma::set_lds_limit(l_step_f32<DTF, NWT>, lds);
        if (attr) return attr;
        const long long problems = static_cast<long long>(P.E) * P.H * P.B;
        hipLaunchKernelGGL((l_step_f32<DTF, NWT>), dim3(problems), dim3(64 * Split<NWT>::WPP), lds, s, P);
        return static_cast<int>(hipGetLastError());
    });
}

inline int launch_z(const Problem& P, hipStream_t s) {
    return for_classes32(dtf_class(P.D), mfma::nt_class(P.M), [&](auto dt, auto nt) {
        constexpr int DTF = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr size_t lds = Lds32<DTF, NWT>::Z;
        if (lds > kLdsLimit) return static_cast<int>(MA_ERR_UNSUPPORTED);
        const int attr = mfma::set_lds_limit(z_step_f32<DTF, NWT>, lds);
        if (attr) return attr;
        const long long problems = static_cast<long long>(P.E) * P.H * P.B;
        hipLaunchKernelGGL((z_step_f32<DTF, NWT>), dim3(problems), dim3(64 * Split<NWT>::WPP), lds, s, P);
        return static_cast<int>(hipGetLastError());
    });
}

// LDS bytes of the largest stage for a shape (host-side feasibility check, no HIP call)
inline size_t lds_needed(int D, int B, int M) {
    size_t need = 0;
    for_classes32(dtf_class(D), mfma::nt_class(B), [&](auto dt, auto nt) {
        need = Lds32<decltype(dt)::value, decltype(nt)::value>::R;
        return 0;
    });
    for_classes32(dtf_class(D), mfma::nt_class(M), [&](auto dt, auto nt) {
        const size_t l = Lds32<decltype(dt)::value, decltype(nt)::value>::L;
        if (l > need) need = l;
        return 0;
    });
    return need;
}

}  // namespace mfma32
}  // namespace ma
