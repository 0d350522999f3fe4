// Flat-mapped row p-norm / normalize kernels for narrow rows, BF16 storage.
#include "thn_pnorm_flat.h"

namespace thn {
THN_DEFINE_PNORM_FLAT_LAUNCHERS(bf16, BF16)
}  // namespace thn
