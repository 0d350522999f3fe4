// Row p-norm / normalize backward kernel instances for F16 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_BWD_LAUNCHERS(f16, F16)
}  // namespace thn
