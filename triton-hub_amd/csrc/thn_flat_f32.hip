// Flat-mapped norm kernels for narrow rows, F32 storage.
#include "thn_flat.h"

namespace thn {
THN_DEFINE_FLAT_LAUNCHERS(f32, F32)
}  // namespace thn
