// Row p-norm / normalize forward kernel instances for F32 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_FWD_LAUNCHERS(f32, F32)
}  // namespace thn
