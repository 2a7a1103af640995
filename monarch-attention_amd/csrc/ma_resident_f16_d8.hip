// Resident forward kernels, f16 operands, head-dim class 8 (D <= 128).
#include "ma_resident_launch.h"

namespace ma {
int launch_resident_f16_d8(const Problem& P, bool dry_run, hipStream_t s) { return mfma::launch_resident<f16, 8>(P, dry_run, s); }
}  // namespace ma
