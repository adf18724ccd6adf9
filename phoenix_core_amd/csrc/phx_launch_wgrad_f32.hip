// Instantiations of the fp32-MFMA filter-gradient kernels and the split-K reduction.
#include "phx_launch.h"

namespace phx {

int launch_wgrad_f32(bool half_storage, int mode, const WgradArgs& a, dim3 grid, size_t lds_bytes, hipStream_t st) {
    const dim3 b(WG_THREADS);
    if (half_storage) {
        if (mode == 16) hipLaunchKernelGGL((qconv_wgrad_f32_kernel<_Float16, 16, 3>), grid, b, lds_bytes, st, a);
        else hipLaunchKernelGGL((qconv_wgrad_f32_kernel<_Float16, 8, 1>), grid, b, lds_bytes, st, a);
    } else {
        if (mode == 16) hipLaunchKernelGGL((qconv_wgrad_f32_kernel<float, 16, 3>), grid, b, lds_bytes, st, a);
        else hipLaunchKernelGGL((qconv_wgrad_f32_kernel<float, 8, 1>), grid, b, lds_bytes, st, a);
    }
    return 0;
}

int launch_reduce_wgrad(bool half_storage, const ReduceArgs& a, int blocks, hipStream_t st) {
    if (half_storage) hipLaunchKernelGGL((reduce_wgrad_kernel<_Float16>), dim3(blocks), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((reduce_wgrad_kernel<float>), dim3(blocks), dim3(WG_THREADS), 0, st, a);
    return 0;
}

}  // namespace phx
