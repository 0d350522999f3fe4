// Softmax / Softmin / LogSoftmax kernel instances for F64 storage.
#include "thn_softmax_dispatch.h"

namespace thn {
THN_DEFINE_SOFTMAX_LAUNCHERS(f64, F64)
}  // namespace thn
