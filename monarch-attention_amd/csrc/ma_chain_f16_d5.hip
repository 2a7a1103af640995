// Chained forward kernels, f16 operands, head-dim class 5 (D <= 80).
#include "ma_chain_launch.h"

namespace ma {
int launch_chain_f16_d5(const Problem& P, bool sync_ready, hipStream_t s) { return mfma::launch_chain<f16, 5>(P, sync_ready, s); }
}  // namespace ma
