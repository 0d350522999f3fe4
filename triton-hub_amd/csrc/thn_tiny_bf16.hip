// Lane-per-row kernels for rows shorter than one vector (softmax and p-norm families), BF16 storage.
#include "thn_tiny.h"

namespace thn {
THN_DEFINE_TINY_LAUNCHERS(bf16, BF16)
}  // namespace thn
