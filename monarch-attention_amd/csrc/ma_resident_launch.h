// Host-side dispatch of the resident (state-in-LDS) forward kernel.  Included by
// one .hip file per (dtype, head-dim class).
#pragma once

#include <type_traits>

#include "ma_mfma_launch.h"
#include "ma_resident.h"
#include "ma_resident_head.h"
#include "ma_resident_head2.h"

namespace ma {
namespace mfma {

constexpr size_t kLdsPerCu = 160 * 1024;
constexpr int kResidentWaves = 8;       // workgroup size in waves ...
constexpr int kResidentWavesWide = 16;  // ... and for blocks of up to 32 rows when the staging of 16 waves still fits

template <class T, int DT, int NTB, int NTM, int W, bool ONE>
int launch_resident_mode(const Problem& P, int mode, size_t lds, hipStream_t s) {
    auto kernel = resident_fwd_mfma<T, DT, NTB, NTM, W, ONE>;
    const int lds_err = set_lds_limit(kernel, kLdsPerCu);
    if (lds_err) return lds_err;
    const DeviceCaps caps = device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    // one workgroup per CU at a time when the state takes more than half the LDS, else two;
    // the workgroups are independent (no waiting on each other), so any grid size is safe
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long per_cu = lds * 2 <= kLdsPerCu ? 2 : 1;
    long long grid = caps.cus * per_cu;
    if (grid > heads) grid = heads;
    hipLaunchKernelGGL((resident_fwd_mfma<T, DT, NTB, NTM, W, ONE>), dim3(grid), dim3(64 * W), lds, s, P, mode);
    return static_cast<int>(hipGetLastError());
}

template <class T, int DT, int NTB, int NTM, int W>
int launch_resident_w(const Problem& P, bool dry_run, hipStream_t s) {
    using RS = Resident<T, DT, NTB, NTM, W>;
    const int Np = P.M * P.B;
    // Y in a tile of its own if that fits, else in aR's place where the kernel allows it, else
    // aL and aR in one tile and Y through the workspace
    int mode = RS::kThreeTiles;
    size_t lds = RS::lds_bytes(Np, P.M, P.B, mode);
    if (lds > kLdsPerCu && RS::y_on_x_possible(P.M)) {
        mode = RS::kYOnX;
        lds = RS::lds_bytes(Np, P.M, P.B, mode);
    }
    if (lds > kLdsPerCu && P.one_tile_ok) {
        mode = RS::kOneTile;
        lds = RS::lds_bytes(Np, P.M, P.B, mode);
    }
    if (lds > kLdsPerCu) return MA_ERR_UNSUPPORTED;   // the head's state does not fit in LDS
    if (dry_run) return MA_OK;
    return mode == RS::kOneTile ? launch_resident_mode<T, DT, NTB, NTM, W, true>(P, mode, lds, s)
                                : launch_resident_mode<T, DT, NTB, NTM, W, false>(P, mode, lds, s);
}

// Heads whose inputs fit the LDS beside the state: the head-resident kernel (one workgroup per CU).
template <class T, int DT, int NTB, int NTM, int W, int NI>
int launch_resident_head_ni(const Problem& P, bool dry_run, hipStream_t s) {
    using HR = HeadRes<T, DT, NTB, NTM, W, NI>;
    const int Np = P.M * P.B;
    if (!HR::fits(Np, P.B, P.M, kLdsPerCu)) return MA_ERR_UNSUPPORTED;
    if (dry_run) return MA_OK;
    auto kernel = resident_head_mfma<T, DT, NTB, NTM, W, NI>;
    const int lds_err = set_lds_limit(kernel, kLdsPerCu);
    if (lds_err) return lds_err;
    const DeviceCaps caps = device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long grid = heads < caps.cus ? heads : caps.cus;
    hipLaunchKernelGGL((resident_head_mfma<T, DT, NTB, NTM, W, NI>), dim3(grid), dim3(64 * W), HR::layout(Np, P.B, P.M).total, s, P);
    return static_cast<int>(hipGetLastError());
}
template <class T, int DT, int NTB, int NTM>
int launch_resident_head(const Problem& P, bool dry_run, hipStream_t s) {
    constexpr int W = (NTB <= 2 && NTM <= 2) ? 16 : 8;
    // two 16-byte chunks per thread and input tile where that covers the head (fewer registers held through the rounds), else three
    const int err = launch_resident_head_ni<T, DT, NTB, NTM, W, 2>(P, dry_run, s);
    if (err != MA_ERR_UNSUPPORTED) return err;
    return launch_resident_head_ni<T, DT, NTB, NTM, W, 3>(P, dry_run, s);
}

// Heads of about twice that length: the state and one input tile at a time in LDS (ma_resident_head2.h).
template <class T, int DT, int NTB, int NTM, int W, int NI>
int launch_resident_head2_ni(const Problem& P, bool dry_run, hipStream_t s) {
    using H2 = HeadRes2<T, DT, NTB, NTM, W, NI>;
    const int Np = P.M * P.B;
    if (!H2::fits(Np, P.B, P.M, kLdsPerCu)) return MA_ERR_UNSUPPORTED;
    if (dry_run) return MA_OK;
    auto kernel = resident_head2_mfma<T, DT, NTB, NTM, W, NI>;
    const int lds_err = set_lds_limit(kernel, kLdsPerCu);
    if (lds_err) return lds_err;
    const DeviceCaps caps = device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long grid = heads < caps.cus ? heads : caps.cus;
    hipLaunchKernelGGL((resident_head2_mfma<T, DT, NTB, NTM, W, NI>), dim3(grid), dim3(64 * W), H2::layout(Np, P.B, P.M).total, s, P);
    return static_cast<int>(hipGetLastError());
}
template <class T, int DT, int NTB, int NTM>
int launch_resident_head2(const Problem& P, bool dry_run, hipStream_t s) {
    // (16 waves on 64-row blocks spill ~20 registers: 0.91 of the eight-wave time for few heads, 1.02 - 1.08 from 128 heads on)
    constexpr int W = (NTB <= 2 && NTM <= 2) ? 16 : 8;
    // 4096 or 5120 16-byte chunks per tile (the larger covers every tile that fits the LDS twice)
    const int err = launch_resident_head2_ni<T, DT, NTB, NTM, W, 4096 / (64 * W)>(P, dry_run, s);
    if (err != MA_ERR_UNSUPPORTED) return err;
    return launch_resident_head2_ni<T, DT, NTB, NTM, W, 5120 / (64 * W)>(P, dry_run, s);
}

// Many short heads: the head-resident kernels in workgroups of 8 or 4 waves, two or four of them per compute unit.  A
// head's phases are chains of small block problems with barriers between them; workgroups that share a compute unit
// are out of step with each other and fill each other's waits, which one sixteen-wave workgroup walking its heads in
// turn cannot.  Measured on heads of 48 .. 288 tokens, 256 .. 6144 heads, D = 32 / 64 / 72 / 128, T = 1 .. 3, against
// the four-tile form in one workgroup per compute unit: the two-tile form 0.56 - 0.97 of its time where the rule below
// takes it, the four-tile form in narrow workgroups another 0.79 - 1.04 of that at head dims of up to 80 (and it needs
// no rule beyond "more heads than compute units": it was never behind the wide workgroup).
constexpr int kPolicyCus = 256;   // compute units of the device the rules were measured on

// The four-tile form, W waves per workgroup, 16 / W workgroups per compute unit
template <class T, int DT, int NTB, int NTM, int W, int NI>
int launch_resident_head_packed_ni(const Problem& P, bool dry_run, hipStream_t s) {
    constexpr int WGS = 16 / W;
    using HR = HeadRes<T, DT, NTB, NTM, W, NI>;
    const int Np = P.M * P.B;
    if (!HR::fits(Np, P.B, P.M, kLdsPerCu / WGS)) return MA_ERR_UNSUPPORTED;
    if (dry_run) return MA_OK;
    auto kernel = resident_head_mfma<T, DT, NTB, NTM, W, NI, WGS>;
    const int lds_err = set_lds_limit(kernel, kLdsPerCu);
    if (lds_err) return lds_err;
    const DeviceCaps caps = device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long grid = heads < WGS * caps.cus ? heads : WGS * caps.cus;
    hipLaunchKernelGGL((resident_head_mfma<T, DT, NTB, NTM, W, NI, WGS>), dim3(grid), dim3(64 * W), HR::layout(Np, P.B, P.M).total, s, P);
    return static_cast<int>(hipGetLastError());
}
template <class T, int DT, int NTB, int NTM>
int launch_resident_head_packed(const Problem& P, bool dry_run, hipStream_t s) {
    const long long heads = static_cast<long long>(P.E) * P.H;
    if (heads <= kPolicyCus) return MA_ERR_UNSUPPORTED;   // a head per compute unit at most: the widest workgroup
    if (heads >= 3 * kPolicyCus) {   // as many workgroups per compute unit as there are heads for it
        const int err = launch_resident_head_packed_ni<T, DT, NTB, NTM, 4, 2>(P, dry_run, s);
        if (err != MA_ERR_UNSUPPORTED) return err;
        const int err3 = launch_resident_head_packed_ni<T, DT, NTB, NTM, 4, 3>(P, dry_run, s);
        if (err3 != MA_ERR_UNSUPPORTED) return err3;
    }
    const int err = launch_resident_head_packed_ni<T, DT, NTB, NTM, 8, 2>(P, dry_run, s);
    if (err != MA_ERR_UNSUPPORTED) return err;
    return launch_resident_head_packed_ni<T, DT, NTB, NTM, 8, 3>(P, dry_run, s);
}

// The two-tile form in narrow workgroups, for heads whose four tiles do not fit a share of the LDS: how many waves
// per workgroup (0: the wide workgroup does better)
template <class T, int DT, int NTB, int NTM>
int head2_packed_waves(const Problem& P) {
    const long long heads = static_cast<long long>(P.E) * P.H;
    const int Np = P.M * P.B;
    if (heads <= kPolicyCus) return 0;
    const bool fits8 = HeadRes2<T, DT, NTB, NTM, 8, 4>::fits(Np, P.B, P.M, kLdsPerCu / 2);
    const bool fits4 = fits8 && HeadRes2<T, DT, NTB, NTM, 4, 4>::fits(Np, P.B, P.M, kLdsPerCu / 4);
    if (!fits8) return 0;
    const bool wide = P.D > 80;   // (the four-tile form holds three 16-byte pieces per thread and tile there: 0.5 - 0.97 for any head count)
    const bool mid = P.D > 64 && !wide;
    if (fits4) {
        // a single step of very many heads of 100+ tokens stays with the wide four-tile form (1.03 - 1.2)
        if (!(wide || P.T >= 2 || heads <= 4 * kPolicyCus || Np <= 96 || P.D <= 32)) return 0;
        return heads <= 2 * kPolicyCus ? 8 : 4;
    }
    // eight waves only (heads of ~130 .. 270 tokens at D = 64): up to two heads per compute unit, or up to four in
    // 16-row blocks with more than one step; beyond that the wide four-tile form is 1.0 - 1.25 ahead
    // (head dims of 65 .. 80 in longer blocks: 1.02 - 1.05 at up to two heads per compute unit, 1.02 - 1.3 beyond)
    if (wide || (heads <= 2 * kPolicyCus && !(mid && P.B > 16)) || (heads <= 4 * kPolicyCus && P.T >= 2 && P.B <= 16 && Np <= 208)) return 8;
    return 0;
}
template <class T, int DT, int NTB, int NTM, int W>
int launch_resident_head2_packed(const Problem& P, bool dry_run, hipStream_t s) {
    constexpr int WGS = 16 / W, NI = 4;
    using H2 = HeadRes2<T, DT, NTB, NTM, W, NI>;
    const int Np = P.M * P.B;
    if (!H2::fits(Np, P.B, P.M, kLdsPerCu / WGS)) return MA_ERR_UNSUPPORTED;
    if (dry_run) return MA_OK;
    auto kernel = resident_head2_mfma<T, DT, NTB, NTM, W, NI, WGS>;
    const int lds_err = set_lds_limit(kernel, kLdsPerCu);
    if (lds_err) return lds_err;
    const DeviceCaps caps = device_caps(kernel, 0, 0);
    if (caps.err) return caps.err;
    if (caps.cus < 1) return MA_ERR_DEVICE;
    const long long heads = static_cast<long long>(P.E) * P.H;
    const long long grid = heads < WGS * caps.cus ? heads : WGS * caps.cus;
    hipLaunchKernelGGL((resident_head2_mfma<T, DT, NTB, NTM, W, NI, WGS>), dim3(grid), dim3(64 * W), H2::layout(Np, P.B, P.M).total, s, P);
    return static_cast<int>(hipGetLastError());
}

// The problems of a head are small and latency-bound: more waves per workgroup run more of
// them at once, so the wide workgroup is preferred wherever its staging fits beside the state - unless there are
// more heads than compute units and several narrow workgroups fit one.
// P.resident_head_only (queries, dry runs): 1 - the four-tile form or nothing, 2 - a head-resident form or nothing
// (both: does it fit?); 3 - a form in narrow workgroups or nothing, 4 - the four-tile form in narrow workgroups or
// nothing (both: is it what a launch would run?)
template <class T, int DT, int NTB, int NTM>
int launch_resident_one(const Problem& P, bool dry_run, hipStream_t s) {
    if (P.resident_head_only == 0 || P.resident_head_only >= 3) {
        if constexpr (NTB <= 2 && NTM <= 2) {
            // (in the 128-column class the four-tile kernel spills 75 - 113 registers at this budget: 1.05 - 1.44 of the two-tile form's time)
            if constexpr (DT <= 5) {
                const int err = launch_resident_head_packed<T, DT, NTB, NTM>(P, dry_run, s);
                if (err != MA_ERR_UNSUPPORTED) return err;
            }
            if (P.resident_head_only == 4) return MA_ERR_UNSUPPORTED;
            const int w = head2_packed_waves<T, DT, NTB, NTM>(P);
            if (w == 4) return launch_resident_head2_packed<T, DT, NTB, NTM, 4>(P, dry_run, s);
            if (w == 8) return launch_resident_head2_packed<T, DT, NTB, NTM, 8>(P, dry_run, s);
        }
        if (P.resident_head_only >= 3) return MA_ERR_UNSUPPORTED;
    }
    {   // everything in LDS where the head is short enough for that
        const int err = launch_resident_head<T, DT, NTB, NTM>(P, dry_run, s);
        if (err != MA_ERR_UNSUPPORTED || P.resident_head_only == 1) return err;
    }
    {
        const int err = launch_resident_head2<T, DT, NTB, NTM>(P, dry_run, s);
        if (err != MA_ERR_UNSUPPORTED || P.resident_head_only) return err;
    }
    if constexpr (NTB <= 2 && NTM <= 2) {
        const int err = launch_resident_w<T, DT, NTB, NTM, kResidentWavesWide>(P, dry_run, s);
        if (err != MA_ERR_UNSUPPORTED) return err;
    }
    return launch_resident_w<T, DT, NTB, NTM, kResidentWaves>(P, dry_run, s);
}

template <class T, int DT>
int launch_resident(const Problem& P, bool dry_run, hipStream_t s) {
    if (P.B > 64 || P.M > 64) return MA_ERR_UNSUPPORTED;
    // one strip per wave and whole tiles of 16, 32 or 64 rows: 48-row blocks run as 64-row ones here
    const int ntb = nt_class(P.B) == 3 ? 4 : nt_class(P.B), ntm = nt_class(P.M) == 3 ? 4 : nt_class(P.M);
#define MA_NTM(NB)                                                            \
    switch (ntm) {                                                            \
        case 1: return launch_resident_one<T, DT, NB, 1>(P, dry_run, s);      \
        case 2: return launch_resident_one<T, DT, NB, 2>(P, dry_run, s);      \
        default: return launch_resident_one<T, DT, NB, 4>(P, dry_run, s);     \
    }
    switch (ntb) {
        case 1: MA_NTM(1)
        case 2: MA_NTM(2)
        default: MA_NTM(4)
    }
#undef MA_NTM
}

}  // namespace mfma
}  // namespace ma
