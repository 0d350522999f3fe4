// Element-wise activation kernel instances for F32 storage.
#include "thn_act_dispatch.h"

namespace thn {
THN_DEFINE_ACT_LAUNCHER(f32, F32)
}  // namespace thn
