// Forward kernel instances for F16 storage.
#include "thn_dispatch.h"

namespace thn {
THN_DEFINE_FWD_LAUNCHER(f16, F16)
}  // namespace thn
