// R-step MFMA kernels, f16 operands.
#include <type_traits>

#include "ma_mfma_launch.h"

namespace ma {
int launch_mfma_r_f16(const Problem& P, bool first, bool with_v, hipStream_t s) { return mfma::launch_r<f16>(P, first, with_v, s); }
}  // namespace ma
