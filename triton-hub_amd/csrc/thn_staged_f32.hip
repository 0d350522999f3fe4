// LDS-staged norm kernels for narrow rows, F32 storage.
#include "thn_staged.h"

namespace thn {
THN_DEFINE_STAGED_LAUNCHERS(f32, F32)
}  // namespace thn
