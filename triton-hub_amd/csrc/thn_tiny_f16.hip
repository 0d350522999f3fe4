// Lane-per-row kernels for rows shorter than one vector (softmax and p-norm families), F16 storage.
#include "thn_tiny.h"

namespace thn {
THN_DEFINE_TINY_LAUNCHERS(f16, F16)
}  // namespace thn
