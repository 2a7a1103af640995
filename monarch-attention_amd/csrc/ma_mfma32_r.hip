// R-step MFMA kernels, fp32 operands.
#include "ma_mfma32_launch.h"

namespace ma {
int launch_mfma32_r(const Problem& P, bool first, bool with_v, hipStream_t s) { return mfma32::launch_r(P, first, with_v, s); }
size_t mfma32_lds_needed(int D, int B, int M) { return mfma32::lds_needed(D, B, M); }
}  // namespace ma
