// Element-wise activation kernel instances for F64 storage.
#include "thn_act_dispatch.h"

namespace thn {
THN_DEFINE_ACT_LAUNCHER(f64, F64)
}  // namespace thn
