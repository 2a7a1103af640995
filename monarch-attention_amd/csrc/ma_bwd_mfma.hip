// Dispatch of the matrix-core backward stages over the operand dtype, and the host-side questions
// the C-ABI layer asks about them.  The kernels are instantiated in ma_bwd_{lz,r}_{f32,f16,bf16}.hip.
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_lz_mfma(const Problem& P, const BwdBuffers& G, int dt_qk, bool z, hipStream_t s) {
    switch (dt_qk) {
        case MA_F32: return launch_bwd_lz_mfma_f32(P, G, z, s);
        case MA_F16: return launch_bwd_lz_mfma_f16(P, G, z, s);
        default: return launch_bwd_lz_mfma_bf16(P, G, z, s);
    }
}

int launch_bwd_r_mfma(const Problem& P, const BwdBuffers& G, int dt_qk, bool first, bool with_v, hipStream_t s) {
    switch (dt_qk) {
        case MA_F32: return launch_bwd_r_mfma_f32(P, G, first, with_v, s);
        case MA_F16: return launch_bwd_r_mfma_f16(P, G, first, with_v, s);
        default: return launch_bwd_r_mfma_bf16(P, G, first, with_v, s);
    }
}

bool bwd_state16_ok(const Problem& P, int dt_qk, int dt_v) { return state16_ok(P, dt_qk, dt_v); }
int bwd_r_split_tiles(const Problem& P, int dt_qk, int dt_v) { return r_split_tiles(P, dt_qk, dt_v); }
bool bwd_all_reg(const Problem& P, int dt_qk, int dt_v) { return all_reg(P, dt_qk, dt_v); }

}  // namespace ma
