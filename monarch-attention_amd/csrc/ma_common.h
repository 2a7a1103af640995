// Internal declarations shared by the kernels and the C-ABI layer of libma_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ma_hip.h"

namespace ma {

using f16 = _Float16;
using bf16 = __bf16;

// Device-side view of one forward call.  Indices follow the reference
// (ma/ma_torch.py:74-90): token p = m*B + j of the PADDED sequence is block m,
// in-block position j; the real token is t = p - pad_off, valid iff 0 <= t < N.
struct Problem {
    const char* q;
    const char* k;
    const char* v;
    const uint8_t* mask;
    char* out;
    char* aR;      // (E,H,M,B,D)  q/k dtype
    char* aL;      // (E,H,B,M,D)  q/k dtype
    char* Y;       // (E,H,B,M,Dv) v dtype
    float* cR;     // (E,H,M,B)
    float* cL;     // (E,H,B,M)
    float* stats;  // (E,H,B,M,2)  row max / row sum of the generic L step
    unsigned* sync;
    int E, H, N, D, Dv, B, M, T, pad_off;
    long long qs[3], ks[3], vs[3], os[3], ms[2];
    float sm_scale, eps;
    int mask_shift;      // log2 of the mask element size in bytes (ms strides are in elements)
    int mask_float;      // the mask holds floating-point values: -0.0 counts as zero
    int stream_stores;   // state / output rows that are whole 128-byte lines go out as streaming stores
    int state_agent;     // state written by other workgroups is read with agent-scope loads instead of streaming ones
    // Per-stage launches of heads with few blocks (M <= 8): a 16-row tile of an L / Z problem holds 16 >> pack_shift
    // in-block positions of pack_m = 1 << pack_shift rows each (4: one position per tile, as everywhere else).
    int pack_shift;
    // The resident kernel may keep aL and aR in ONE LDS tile and pass Y through the workspace where two or
    // three tiles do not fit (heads of up to ~512 tokens at d = 64).
    int one_tile_ok;
    // Query only: does a head-resident form of the resident kernel take this head?  1: the one that keeps Q, K and V
    // in LDS beside the state; 2: that one or the two-tile form (the state and one input tile at a time); 3: would a
    // launch run a head-resident form in narrow workgroups, several to a compute unit?  4: ... the four-tile form?
    int resident_head_only;
    int test_no_spin;    // waits between workgroups give up at once (failure-path tests)
    // Copy of the error word in host memory the device can write (or null): a workgroup that raises the
    // word in the sync area stores the code here as well, where the host reads it without a copy.
    unsigned* host_error;
};

// First statement of a kernel: one scalar load from every 64-byte line of a by-value kernel argument, all in flight
// together.  The scalar cache starts every launch cold, and a kernel that reads its arguments where it needs them
// (so that they are not held in registers) pays a miss per line, one after the other, before its first global load
// is issued.  Measured: the team kernel gains 0.8 us per launch (17.9 -> 17.2 us on 16 heads of 4096 tokens); the
// chained, resident and per-stage kernels measure the same or 0.2 - 0.3 us slower with it and do not call it.
template <class A>
__device__ __forceinline__ void warm_args(const A& a) {
    const unsigned* w = reinterpret_cast<const unsigned*>(&a);
    unsigned acc = 0;
#pragma unroll
    for (unsigned i = 0; i < sizeof(A) / 4; i += 16) acc |= w[i];
    asm volatile("" ::"s"(acc));
}

// Raise the sticky error word of the one-launch kernels: in the sync area of the workspace, and in the
// caller's host-visible word if there is one.
__device__ __forceinline__ void raise_error(unsigned* error, unsigned* host_error, unsigned code) {
    __hip_atomic_store(error, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (host_error != nullptr) __hip_atomic_store(host_error, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Is a mask element non-zero (torch.logical_and's truthiness, ma/ma_torch.py:98)?  `lo` / `hi` are
// its low and high 32 bits (zero-extended for narrow elements); for floating-point masks the
// sign bit, which is the top bit of the element, does not count (-0.0 is false, NaN is true).
__device__ __forceinline__ bool mask_nonzero(const Problem& P, unsigned lo, unsigned hi) {
    if (P.mask_float) {
        if (P.mask_shift == 3) hi &= 0x7fffffffu;
        else if (P.mask_shift == 2) lo &= 0x7fffffffu;
        else lo &= 0x7fffu;
    }
    return (lo | hi) != 0u;
}

__device__ __forceinline__ bool token_ok(const Problem& P, int e, int t) {
    if (t < 0 || t >= P.N) return false;
    if (P.mask == nullptr) return true;
    const uint8_t* p = P.mask + ((e * P.ms[0] + t * P.ms[1]) << P.mask_shift);
    unsigned lo = 0, hi = 0;
    switch (P.mask_shift) {
        case 0: lo = *p; break;
        case 1: lo = *reinterpret_cast<const uint16_t*>(p); break;
        case 2: lo = *reinterpret_cast<const uint32_t*>(p); break;
        default: lo = reinterpret_cast<const uint32_t*>(p)[0]; hi = reinterpret_cast<const uint32_t*>(p)[1]; break;
    }
    return mask_nonzero(P, lo, hi);
}

template <class T>
__device__ __forceinline__ float to_f(T x) { return static_cast<float>(x); }
template <class T>
__device__ __forceinline__ T from_f(float x) { return static_cast<T>(x); }  // round to nearest even
template <class T>
__device__ __forceinline__ float round_to(float x) { return to_f<T>(from_f<T>(x)); }
template <>
__device__ __forceinline__ float round_to<float>(float x) { return x; }

// Launchers (defined next to their kernels).  All return a hipError_t.
int launch_generic_r(const Problem& P, int dt_qk, int dt_v, bool first, bool with_v, hipStream_t s);
int launch_generic_l(const Problem& P, int dt_qk, hipStream_t s);
int launch_generic_z(const Problem& P, int dt_qk, int dt_v, hipStream_t s);
// dense (E,H,N,N) fp32 matrix from the state of the last R step; MA_ERR_UNSUPPORTED beyond the LDS
constexpr size_t kMatrixLdsBytes = 160 * 1024;
bool generic_matrix_fits(const Problem& P);
int launch_generic_matrix(const Problem& P, int dt_qk, float* A, bool first, hipStream_t s);

// Backward pass (FMA kernels).  Gradients of the per-step state and the padded fp32 accumulators
// of the input gradients; `dout` is the caller's output gradient (v dtype, element strides dos).
struct BwdBuffers {
    float* gaR;   // (E,H,M,B,D)
    float* gcR;   // (E,H,M,B)
    float* gaL;   // (E,H,B,M,D)
    float* gcL;   // (E,H,B,M)
    float* gY;    // (E,H,B,M,Dv)
    float* dq;    // (E,H,Np,D)   accumulated over the stages, zeroed first
    float* dk;    // (E,H,Np,D)
    float* dv;    // (E,H,Np,Dv)
    const char* dout;
    long long dos[3];
    int fma_only;  // take the FMA kernels even where the matrix-core ones apply
    float* pk;     // (parts,E,H,Np,D) / (parts,E,H,Np,Dv): per-tile parts of dk / dv of an R stage whose
    float* pv;     //   tiles of query rows run in different workgroups; nullptr: never split
    int jt_split;  // set by the launcher: workgroups per block (0 = one workgroup walks all tiles)
    int state16;   // gaL, gY, gaR hold the operand dtype instead of fp32 (see bwd_state16_ok)
    // direct != 0 (register kernels in every stage, see bwd_all_reg): the stage that completes a gradient
    // rounds it into the caller's tensor itself - dv in the R stage that forms it, dq and dk in the R stage
    // of the first step - and no conversion kernel runs.  out = {dq, dk, dv} of the caller, outs their
    // element strides (e, h, token); rows of four elements are 8-byte aligned (checked by the host).
    int direct;
    char* out[3];
    long long outs[3][3];
};
bool bwd_state16_ok(const Problem& P, int dt_qk, int dt_v);
// partial buffers the R stage wants for this problem (0: it does not split blocks over workgroups)
int bwd_r_split_tiles(const Problem& P, int dt_qk, int dt_v);
// every stage on a register kernel: dq, dk, dv are written before they are added to (no zeroing needed)
bool bwd_all_reg(const Problem& P, int dt_qk, int dt_v);
bool bwd_fits(const Problem& P);
// matrix-core backward stages: MA_ERR_UNSUPPORTED when the problem's tiles do not fit the LDS
int launch_bwd_lz_mfma(const Problem& P, const BwdBuffers& G, int dt_qk, bool z, hipStream_t s);
int launch_bwd_r_mfma(const Problem& P, const BwdBuffers& G, int dt_qk, bool first, bool with_v, hipStream_t s);
int launch_bwd_lz_mfma_f32(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s);
int launch_bwd_lz_mfma_f16(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s);
int launch_bwd_lz_mfma_bf16(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s);
int launch_bwd_r_mfma_f32(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s);
int launch_bwd_r_mfma_f16(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s);
int launch_bwd_r_mfma_bf16(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s);
int launch_bwd_zero(float* p, long long n, hipStream_t s);
int launch_bwd_z(const Problem& P, const BwdBuffers& G, int dt_qk, int dt_v, hipStream_t s);
int launch_bwd_l(const Problem& P, const BwdBuffers& G, int dt_qk, hipStream_t s);
int launch_bwd_r(const Problem& P, const BwdBuffers& G, int dt_qk, int dt_v, bool first, bool with_v, hipStream_t s);
int launch_bwd_out(int n, const float* const* src, void* const* dst, const long long (*st)[3], int dt, const Problem& P, int W,
                   hipStream_t s);

// MFMA stage kernels (fp16 / bf16, Dv == D <= 128, D % 8 == 0, B, M <= 256,
// 16-byte aligned rows).
int launch_mfma_r_f16(const Problem& P, bool first, bool with_v, hipStream_t s);
int launch_mfma_l_f16(const Problem& P, hipStream_t s);
int launch_mfma_z_f16(const Problem& P, hipStream_t s);
int launch_mfma_r_bf16(const Problem& P, bool first, bool with_v, hipStream_t s);
int launch_mfma_l_bf16(const Problem& P, hipStream_t s);
int launch_mfma_z_bf16(const Problem& P, hipStream_t s);

// fp32 MFMA stage kernels (v_mfma_f32_16x16x4_f32; Dv == D <= 128, D % 4 == 0, B, M <= 128,
// 16-byte aligned rows) and the LDS their largest stage needs for a shape.
int launch_mfma32_r(const Problem& P, bool first, bool with_v, hipStream_t s);
int launch_mfma32_l(const Problem& P, hipStream_t s);
int launch_mfma32_z(const Problem& P, hipStream_t s);
size_t mfma32_lds_needed(int D, int B, int M);

// Fused forward (one launch), by dtype and head-dim class (D <= 32/64/80/128).
// sync_ready: the workspace's sync area is known to be zero.
int launch_fused_f16_d2(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_f16_d4(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_f16_d5(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_f16_d8(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_bf16_d2(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_bf16_d4(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_bf16_d5(const Problem& P, bool sync_ready, hipStream_t s);
int launch_fused_bf16_d8(const Problem& P, bool sync_ready, hipStream_t s);

// Resident forward (one launch, per-head state kept in LDS).  dry_run: only report
// whether the problem fits (MA_OK / MA_ERR_UNSUPPORTED), launch nothing.
int launch_resident_f16_d2(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_f16_d4(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_f16_d5(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_f16_d8(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_bf16_d2(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_bf16_d4(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_bf16_d5(const Problem& P, bool dry_run, hipStream_t s);
int launch_resident_bf16_d8(const Problem& P, bool dry_run, hipStream_t s);

// fp32 heads of at most 16 blocks of at most 16 rows, head dim up to 64: one launch, state in LDS.
int launch_head32(const Problem& P, bool dry_run, hipStream_t s);
// ... of which few heads with a single step run as one workgroup per (head, in-block position) that
// recomputes the rows of the R step it needs (no exchange between workgroups): every workgroup reads
// the head's whole K and V, so only while the launch stays within kHead32T1MaxGroups workgroups.
constexpr long long kHead32T1MaxGroups = 256;
inline bool head32_single_step(const Problem& P) {
    return P.T == 1 && P.B <= 16 && P.M <= 16 && P.D <= 64 && P.D % 4 == 0 && P.Dv == P.D &&
           static_cast<long long>(P.E) * P.H * P.B <= kHead32T1MaxGroups;
}

// Chained forward (one launch, one workgroup per block problem, flags between phases).
int launch_chain_f16_d2(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_f16_d4(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_f16_d5(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_f16_d8(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_bf16_d2(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_bf16_d4(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_bf16_d5(const Problem& P, bool sync_ready, hipStream_t s);
int launch_chain_bf16_d8(const Problem& P, bool sync_ready, hipStream_t s);

constexpr uint64_t kTeamSyncBytes = 4 * (32 + 256 * 1024);   // header + one 1 KiB sector per multi-workgroup team
constexpr uint64_t kChainSyncBytes = 4 * 256 * 1024;                  // flag words of the chained kernel
constexpr uint64_t kSyncAreaBytes = kTeamSyncBytes + kChainSyncBytes;
// Zero-fills the sync area of a workspace (a small fill kernel, graph-capture safe).
int launch_zero_sync(unsigned* sync, hipStream_t s);

}  // namespace ma
