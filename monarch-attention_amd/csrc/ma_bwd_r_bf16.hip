// Backward R stage on the matrix cores, bf16 operands (one translation unit per stage and dtype so that the
// instantiations compile in parallel).
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_r_mfma_bf16(const Problem& P, const BwdBuffers& G, bool first, bool with_v, hipStream_t s) {
    return launch_r_t<bf16>(P, G, first, with_v, s);
}

}  // namespace ma
