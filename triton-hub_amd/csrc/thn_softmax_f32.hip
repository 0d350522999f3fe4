// Softmax / Softmin / LogSoftmax kernel instances for F32 storage.
#include "thn_softmax_dispatch.h"

namespace thn {
THN_DEFINE_SOFTMAX_LAUNCHERS(f32, F32)
}  // namespace thn
