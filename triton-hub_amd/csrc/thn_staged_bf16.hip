// LDS-staged norm kernels for narrow rows, BF16 storage.
#include "thn_staged.h"

namespace thn {
THN_DEFINE_STAGED_LAUNCHERS(bf16, BF16)
}  // namespace thn
