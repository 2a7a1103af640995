// L-step MFMA kernels, f16 operands.
#include <type_traits>

#include "ma_mfma_launch.h"

namespace ma {
int launch_mfma_l_f16(const Problem& P, hipStream_t s) { return mfma::launch_l<f16>(P, s); }
}  // namespace ma
