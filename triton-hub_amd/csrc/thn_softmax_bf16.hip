// Softmax / Softmin / LogSoftmax kernel instances for BF16 storage.
#include "thn_softmax_dispatch.h"

namespace thn {
THN_DEFINE_SOFTMAX_LAUNCHERS(bf16, BF16)
}  // namespace thn
