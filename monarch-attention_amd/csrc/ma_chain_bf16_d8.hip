// Chained forward kernels, bf16 operands, head-dim class 8 (D <= 128).
#include "ma_chain_launch.h"

namespace ma {
int launch_chain_bf16_d8(const Problem& P, bool sync_ready, hipStream_t s) { return mfma::launch_chain<bf16, 8>(P, sync_ready, s); }
}  // namespace ma
