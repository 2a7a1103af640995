// Z-step MFMA kernels, bf16 operands.
#include <type_traits>

#include "ma_mfma_launch.h"

namespace ma {
int launch_mfma_z_bf16(const Problem& P, hipStream_t s) { return mfma::launch_z<bf16>(P, s); }
}  // namespace ma
