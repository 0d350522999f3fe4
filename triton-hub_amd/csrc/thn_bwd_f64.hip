// Backward kernel instances for F64 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_BWD_LAUNCHER(f64, F64)
}  // namespace thn
