// Backward kernel instances for F32 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_BWD_LAUNCHER(f32, F32)
}  // namespace thn
