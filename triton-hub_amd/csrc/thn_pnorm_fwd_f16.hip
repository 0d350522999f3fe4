// Row p-norm / normalize forward kernel instances for F16 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_FWD_LAUNCHERS(f16, F16)
}  // namespace thn
