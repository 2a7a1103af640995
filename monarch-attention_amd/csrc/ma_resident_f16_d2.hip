// Resident forward kernels, f16 operands, head-dim class 2 (D <= 32).
#include "ma_resident_launch.h"

namespace ma {
int launch_resident_f16_d2(const Problem& P, bool dry_run, hipStream_t s) { return mfma::launch_resident<f16, 2>(P, dry_run, s); }
}  // namespace ma
