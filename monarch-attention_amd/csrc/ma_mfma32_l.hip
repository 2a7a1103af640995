// L-step MFMA kernels, fp32 operands.
#include "ma_mfma32_launch.h"

namespace ma {
int launch_mfma32_l(const Problem& P, hipStream_t s) { return mfma32::launch_l(P, s); }
}  // namespace ma
