// Norm forward kernels with an activation epilogue, F64 storage.
#include "thn_fused_dispatch.h"

namespace thn {
THN_DEFINE_FUSED_FWD_LAUNCHER(f64, F64)
}  // namespace thn
