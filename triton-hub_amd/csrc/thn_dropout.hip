// The dropout kernel in the four storage types.
#include "thn_dropout.h"

namespace thn {

int launch_dropout(int dtype, const DropoutArgs& a, int grid, hipStream_t st) {
    switch (dtype) {
        case kF32: hipLaunchKernelGGL(dropout_flat_kernel<F32>, dim3(grid), dim3(kDropoutBlock), 0, st, a); break;
        case kF16: hipLaunchKernelGGL(dropout_flat_kernel<F16>, dim3(grid), dim3(kDropoutBlock), 0, st, a); break;
        case kBF16: hipLaunchKernelGGL(dropout_flat_kernel<BF16>, dim3(grid), dim3(kDropoutBlock), 0, st, a); break;
        case kF64: hipLaunchKernelGGL(dropout_flat_kernel<F64>, dim3(grid), dim3(kDropoutBlock), 0, st, a); break;
        default: return 1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace thn
