// Flat-mapped Softmax / Softmin / LogSoftmax kernels for narrow rows, BF16 storage.
#include "thn_softmax_flat.h"

namespace thn {
THN_DEFINE_SOFTMAX_FLAT_LAUNCHERS(bf16, BF16)
}  // namespace thn
