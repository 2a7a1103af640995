// Backward L / Z stages on the matrix cores, bf16 operands (one translation unit per stage and dtype so that
// the instantiations compile in parallel).
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_lz_mfma_bf16(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s) { return launch_lz_t<bf16>(P, G, z, s); }

}  // namespace ma
