// Forward kernel instances for F64 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_FWD_LAUNCHER(f64, F64)
}  // namespace thn
