// Row p-norm / normalize backward kernel instances for F64 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_BWD_LAUNCHERS(f64, F64)
}  // namespace thn
