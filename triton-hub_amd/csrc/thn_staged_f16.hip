// LDS-staged norm kernels for narrow rows, F16 storage.
#include "thn_staged.h"

namespace thn {
THN_DEFINE_STAGED_LAUNCHERS(f16, F16)
}  // namespace thn
