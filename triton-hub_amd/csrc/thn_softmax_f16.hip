// Softmax / Softmin / LogSoftmax kernel instances for F16 storage.
#include "thn_softmax_dispatch.h"

namespace thn {
THN_DEFINE_SOFTMAX_LAUNCHERS(f16, F16)
}  // namespace thn
