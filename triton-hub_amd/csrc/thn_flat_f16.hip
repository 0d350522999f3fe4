// Flat-mapped norm kernels for narrow rows, F16 storage.
#include "thn_flat.h"

namespace thn {
THN_DEFINE_FLAT_LAUNCHERS(f16, F16)
}  // namespace thn
