// Norm backward kernels for an activation epilogue, F16 storage.
#include "thn_fused_dispatch.h"

namespace thn {
THN_DEFINE_FUSED_BWD_LAUNCHER(f16, F16)
}  // namespace thn
