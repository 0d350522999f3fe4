// Backward kernel instances for F16 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_BWD_LAUNCHER(f16, F16)
}  // namespace thn
