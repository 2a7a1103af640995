// Backward R stage on the matrix cores, f32 operands (one translation unit per stage and dtype so that the
// instantiations compile in parallel).
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_r_mfma_f32(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s) {
    return launch_r_t<float>(P, G, first, with_v, s);
}

}  // namespace ma
