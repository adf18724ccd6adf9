// Instantiations of the fp16-MFMA filter-gradient kernels.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

int launch_wgrad_f16(int mode, const WgradArgs& a, dim3 grid, size_t lds_bytes, hipStream_t st) {
    const dim3 b(WG_THREADS);
    if (mode == 16) hipLaunchKernelGGL((qconv_wgrad_f16_kernel<16, 3>), grid, b, lds_bytes, st, a);
    else hipLaunchKernelGGL((qconv_wgrad_f16_kernel<8, 1>), grid, b, lds_bytes, st, a);
    return 0;
}

}  // namespace phx
