// Fused forward kernels, bf16 operands, head-dim class 4 (D <= 64).
#include "ma_fused_launch.h"

namespace ma {
int launch_fused_bf16_d4(const Problem& P, bool sync_ready, hipStream_t s) { return mfma::launch_fused<bf16, 4>(P, sync_ready, s); }
}  // namespace ma
