// Element-wise activation kernel instances for BF16 storage.
#include "thn_act_dispatch.h"

namespace thn {
THN_DEFINE_ACT_LAUNCHER(bf16, BF16)
}  // namespace thn
