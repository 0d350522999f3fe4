// Row p-norm / normalize forward kernel instances for BF16 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_FWD_LAUNCHERS(bf16, BF16)
}  // namespace thn
