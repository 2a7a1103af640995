// Host-side dispatch of the staged MFMA kernels over (head-dim tiles DT,
// strip count NWT).  Included by one .hip file per (dtype, stage) so that the
// instantiations compile in parallel.
#pragma once

#include <map>
#include <utility>
#include <mutex>

#include "ma_mfma.h"

namespace ma {
namespace mfma {

inline int dt_class(int D) { return D <= 32 ? 2 : D <= 64 ? 4 : D <= 80 ? 5 : 8; }
// the team kernel is built for fewer classes: 96-row problems run as 128-row ones there
inline int nt_class_one_launch(int n) {
    const int t = (n + 15) / 16;
    return t <= 4 ? (t < 1 ? 1 : t) : 8;
}
// the chained kernel has the 96-row class as well
inline int nt_class_chain(int n) {
    const int t = (n + 15) / 16;
    return t <= 4 ? (t < 1 ? 1 : t) : t <= 6 ? 6 : 8;
}
// (129 .. 256 rows: classes of 12 and 16 strips, per-stage launches only; a head of 32768 tokens in
// blocks of floor(sqrt(N)) = 181 rows runs in the 12-strip class both ways)
inline int nt_class(int n) {
    const int t = (n + 15) / 16;
    return t <= 4 ? (t < 1 ? 1 : t) : t <= 6 ? 6 : t <= 8 ? 8 : t <= 12 ? 12 : 16;
}

// Raises a kernel's dynamic-LDS limit to `bytes`, once per (kernel, device): the attribute belongs
// to the device's copy of the code object, so a process that drives several devices needs it on
// each of them.  Returns 0 or a hipError_t.
template <class K>
int set_lds_limit(K kernel, size_t bytes) {
    static std::mutex mu;
    static std::map<const void*, unsigned> done;   // kernel -> bit d set: limit raised on device d
    int dev = 0;
    const hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return static_cast<int>(err);
    const void* key = reinterpret_cast<const void*>(kernel);
    const unsigned bit = 1u << (dev & 31);
    std::lock_guard<std::mutex> lock(mu);
    unsigned& mask = done[key];
    if (mask & bit) return 0;
    const int rc = static_cast<int>(hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    if (rc == 0) mask |= bit;
    return rc;
}

// What the current device offers a kernel: its CU count and, when `threads` > 0, how many workgroups
// of `threads` lanes and `lds` bytes a CU holds at once.  Looked up once per (kernel, device): a
// process may drive devices that differ.
struct DeviceCaps {
    int err = 0, cus = 0, per_cu = 0;
};
template <class K>
DeviceCaps device_caps(K kernel, int threads, size_t lds) {
    static std::mutex mu;
    static std::map<std::pair<const void*, int>, DeviceCaps> known;
    DeviceCaps c;
    int dev = 0;
    c.err = static_cast<int>(hipGetDevice(&dev));
    if (c.err) return c;
    const void* key = reinterpret_cast<const void*>(kernel);
    std::lock_guard<std::mutex> lock(mu);
    const auto it = known.find({key, dev});
    if (it != known.end()) return it->second;
    c.err = static_cast<int>(hipDeviceGetAttribute(&c.cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (!c.err && threads > 0) c.err = static_cast<int>(hipOccupancyMaxActiveBlocksPerMultiprocessor(&c.per_cu, key, threads, lds));
    if (!c.err) known[{key, dev}] = c;
    return c;
}

// calls f(dt_tag, nt_tag) with integral_constant tags for the problem's classes
template <class F>
int for_classes(int dt, int nt, F&& f) {
#define MA_NT(DTV)                                                                            \
    switch (nt) {                                                                             \
        case 1: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 1>{}); \
        case 2: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 2>{}); \
        case 3: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 3>{}); \
        case 4: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 4>{}); \
        case 6: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 6>{}); \
        case 8: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 8>{}); \
        case 12: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 12>{}); \
        default: return f(std::integral_constant<int, DTV>{}, std::integral_constant<int, 16>{}); \
    }
    switch (dt) {
        case 2: MA_NT(2)
        case 4: MA_NT(4)
        case 5: MA_NT(5)
        default: MA_NT(8)
    }
#undef MA_NT
}

// Problems of 6 or 8 strips (one per workgroup, two strips per wave) can run as two workgroups of one strip
// per wave each.  That pays when the launch does not fill the device: with both halves of every problem
// inside the workgroup slots the device offers at once, twice as many waves work on the same bytes (8 heads
// of 64 128-row blocks: 21.9 -> 20.2 us per forward, 2 heads: 13.8 -> 11.6).  Launches of more than one
// round of slots gain nothing from halves (the dispatcher refills slots as workgroups end; measured 55.1 ->
// 56.8 us for 1536 problems on 1024 slots) and stay whole.  *err is set when the device cannot be queried.
template <class K>
bool halves_pay(K whole, int threads, size_t lds, long long problems, int* err) {
    const DeviceCaps caps = device_caps(whole, threads, lds);
    *err = caps.err;
    const long long slots = static_cast<long long>(caps.cus) * caps.per_cu;
    return !caps.err && 2 * problems <= slots;
}

template <class T>
int launch_r(const Problem& P, bool first, bool with_v, hipStream_t s) {
    return for_classes(dt_class(P.D), nt_class(P.B), [&](auto dt, auto nt) {
        constexpr int DT = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr int WG = Split<NWT>::WG, PPW = Split<NWT, WG>::PPW;
        constexpr size_t lds = PPW * Lds<T, DT, NWT>::R;
        const int attr = set_lds_limit(r_step_mfma<T, DT, NWT>, lds);
        if (attr) return attr;
        const long long problems = static_cast<long long>(P.E) * P.H * P.M;
        if constexpr (NWT == 6 || NWT == 8) {
            int err = 0;
            if (halves_pay(r_step_mfma<T, DT, NWT>, 64 * WG, lds, problems, &err)) {
                const int attr2 = set_lds_limit(r_step_mfma<T, DT, NWT, 2>, lds);
                if (attr2) return attr2;
                hipLaunchKernelGGL((r_step_mfma<T, DT, NWT, 2>), dim3(16 * ((problems + 7) / 8)), dim3(64 * WG), lds, s, P,
                                   first ? 1 : 0, with_v ? 1 : 0);
                return static_cast<int>(hipGetLastError());
            }
            if (err) return err;
        }
        hipLaunchKernelGGL((r_step_mfma<T, DT, NWT>), dim3((problems + PPW - 1) / PPW), dim3(64 * WG), lds, s, P,
                           first ? 1 : 0, with_v ? 1 : 0);
        return static_cast<int>(hipGetLastError());
    });
}

template <class T>
int launch_l(const Problem& P, hipStream_t s) {
    return for_classes(dt_class(P.D), nt_class(P.M), [&](auto dt, auto nt) {
        constexpr int DT = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr int WG = Split<NWT>::WG, PPW = Split<NWT, WG>::PPW;
        constexpr size_t lds = PPW * Lds<T, DT, NWT>::L;
        const int attr = set_lds_limit(l_step_mfma<T, DT, NWT>, lds);
        if (attr) return attr;
        const long long per = NWT == 1 ? (16 >> P.pack_shift) : 1;   // positions per problem (see TileIndex)
        const long long problems = static_cast<long long>(P.E) * P.H * ((P.B + per - 1) / per);
        hipLaunchKernelGGL((l_step_mfma<T, DT, NWT>), dim3((problems + PPW - 1) / PPW), dim3(64 * WG), lds, s, P);
        return static_cast<int>(hipGetLastError());
    });
}

template <class T>
int launch_z(const Problem& P, hipStream_t s) {
    return for_classes(dt_class(P.D), nt_class(P.M), [&](auto dt, auto nt) {
        constexpr int DT = decltype(dt)::value, NWT = decltype(nt)::value;
        constexpr int WG = Split<NWT>::WG, PPW = Split<NWT, WG>::PPW;
        constexpr size_t lds = PPW * Lds<T, DT, NWT>::Z;
        const int attr = set_lds_limit(z_step_mfma<T, DT, NWT>, lds);
        if (attr) return attr;
        const long long per = NWT == 1 ? (16 >> P.pack_shift) : 1;
        const long long problems = static_cast<long long>(P.E) * P.H * ((P.B + per - 1) / per);
        if constexpr (NWT == 6 || NWT == 8) {
            int err = 0;
            if (halves_pay(z_step_mfma<T, DT, NWT>, 64 * WG, lds, problems, &err)) {
                const int attr2 = set_lds_limit(z_step_mfma<T, DT, NWT, 2>, lds);
                if (attr2) return attr2;
                hipLaunchKernelGGL((z_step_mfma<T, DT, NWT, 2>), dim3(16 * ((problems + 7) / 8)), dim3(64 * WG), lds, s, P);
                return static_cast<int>(hipGetLastError());
            }
            if (err) return err;
        }
        hipLaunchKernelGGL((z_step_mfma<T, DT, NWT>), dim3((problems + PPW - 1) / PPW), dim3(64 * WG), lds, s, P);
        return static_cast<int>(hipGetLastError());
    });
}

}  // namespace mfma
}  // namespace ma
