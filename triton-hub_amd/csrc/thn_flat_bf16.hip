// Flat-mapped norm kernels for narrow rows, BF16 storage.
#include "thn_flat.h"

namespace thn {
THN_DEFINE_FLAT_LAUNCHERS(bf16, BF16)
}  // namespace thn
