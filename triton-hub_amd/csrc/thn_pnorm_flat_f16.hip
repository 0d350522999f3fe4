// Flat-mapped row p-norm / normalize kernels for narrow rows, F16 storage.
#include "thn_pnorm_flat.h"

namespace thn {
THN_DEFINE_PNORM_FLAT_LAUNCHERS(f16, F16)
}  // namespace thn
