// Forward kernel instances for BF16 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_FWD_LAUNCHER(bf16, BF16)
}  // namespace thn
