// Element-wise activation kernel instances for F16 storage.
#include "thn_act_dispatch.h"

namespace thn {
THN_DEFINE_ACT_LAUNCHER(f16, F16)
}  // namespace thn
