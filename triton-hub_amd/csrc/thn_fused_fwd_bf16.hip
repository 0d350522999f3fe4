// Norm forward kernels with an activation epilogue, BF16 storage.
#include "thn_fused_dispatch.h"

namespace thn {
THN_DEFINE_FUSED_FWD_LAUNCHER(bf16, BF16)
}  // namespace thn
