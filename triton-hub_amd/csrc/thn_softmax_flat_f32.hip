// Flat-mapped Softmax / Softmin / LogSoftmax kernels for narrow rows, F32 storage.
#include "thn_softmax_flat.h"

namespace thn {
THN_DEFINE_SOFTMAX_FLAT_LAUNCHERS(f32, F32)
}  // namespace thn
