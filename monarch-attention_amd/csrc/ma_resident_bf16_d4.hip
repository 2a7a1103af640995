// Resident forward kernels, bf16 operands, head-dim class 4 (D <= 64).
#include "ma_resident_launch.h"

namespace ma {
int launch_resident_bf16_d4(const Problem& P, bool dry_run, hipStream_t s) { return mfma::launch_resident<bf16, 4>(P, dry_run, s); }
}  // namespace ma
