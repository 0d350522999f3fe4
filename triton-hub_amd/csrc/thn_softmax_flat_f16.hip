// Flat-mapped Softmax / Softmin / LogSoftmax kernels for narrow rows, F16 storage.
#include "thn_softmax_flat.h"

namespace thn {
THN_DEFINE_SOFTMAX_FLAT_LAUNCHERS(f16, F16)
}  // namespace thn
