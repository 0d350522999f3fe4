// Row p-norm / normalize forward kernel instances for F64 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_FWD_LAUNCHERS(f64, F64)
}  // namespace thn
