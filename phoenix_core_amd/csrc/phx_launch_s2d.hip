// Launchers of the space-to-depth rearrangement kernels.
#include "phx_kernels_s2d.h"
#include "phx_launch.h"

namespace phx {

static int blocks_for(long items) { return (int)std::min<long>((items + WG_THREADS - 1) / WG_THREADS, 1 << 16); }

int launch_s2d_input(bool half_storage, const S2dArgs& a, hipStream_t st) {
    const long items = a.planes * a.H2 * ((a.W2 + 3) / 4);
    if (half_storage) hipLaunchKernelGGL((s2d_input_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((s2d_input_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

int launch_s2d_filter(bool half_storage, const S2dFilterArgs& a, bool to_caller, hipStream_t st) {
    const long items = 4L * a.Co * 4 * a.Ci * a.K2h * a.K2w;
    if (half_storage)
        hipLaunchKernelGGL((s2d_filter_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    else hipLaunchKernelGGL((s2d_filter_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    return 0;
}

}  // namespace phx
