// Backward L / Z stages on the matrix cores, f32 operands (one translation unit per stage and dtype so that
// the instantiations compile in parallel).
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_lz_mfma_f32(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s) { return launch_lz_t<float>(P, G, z, s); }

}  // namespace ma
