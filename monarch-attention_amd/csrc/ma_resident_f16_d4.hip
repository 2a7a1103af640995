// Resident forward kernels, f16 operands, head-dim class 4 (D <= 64).
#include "ma_resident_launch.h"

namespace ma {
int launch_resident_f16_d4(const Problem& P, bool dry_run, hipStream_t s) { return mfma::launch_resident<f16, 4>(P, dry_run, s); }
}  // namespace ma
