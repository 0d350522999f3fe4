// Row p-norm / normalize backward kernel instances for BF16 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_BWD_LAUNCHERS(bf16, BF16)
}  // namespace thn
