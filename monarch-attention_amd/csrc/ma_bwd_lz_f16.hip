// Backward L / Z stages on the matrix cores, f16 operands (one translation unit per stage and dtype so that
// the instantiations compile in parallel).
#include "ma_bwd_mfma.h"

namespace ma {

int launch_bwd_lz_mfma_f16(const Problem& P, const BwdBuffers& G, bool z, hipStream_t s) { return launch_lz_t<f16>(P, G, z, s); }

}  // namespace ma
