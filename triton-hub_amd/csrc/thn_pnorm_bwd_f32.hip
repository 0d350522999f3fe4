// Row p-norm / normalize backward kernel instances for F32 storage.
#include "thn_pnorm_dispatch.h"

namespace thn {
THN_DEFINE_PNORM_BWD_LAUNCHERS(f32, F32)
}  // namespace thn
