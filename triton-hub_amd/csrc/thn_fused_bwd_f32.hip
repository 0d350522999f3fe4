// Norm backward kernels for an activation epilogue, F32 storage.
#include "thn_fused_dispatch.h"

namespace thn {
THN_DEFINE_FUSED_BWD_LAUNCHER(f32, F32)
}  // namespace thn
