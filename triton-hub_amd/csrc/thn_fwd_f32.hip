// Forward kernel instances for F32 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_FWD_LAUNCHER(f32, F32)
}  // namespace thn
