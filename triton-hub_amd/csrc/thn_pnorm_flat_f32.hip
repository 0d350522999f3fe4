// Flat-mapped row p-norm / normalize kernels for narrow rows, F32 storage.
#include "thn_pnorm_flat.h"

namespace thn {
THN_DEFINE_PNORM_FLAT_LAUNCHERS(f32, F32)
}  // namespace thn
