// Instantiations of the fp32-MFMA filter-gradient kernels and the split-K reduction.
#include "phx_launch.h"

namespace phx {

template <typename TS, bool VEC>
static void launch_ts(int mode, const WgradArgs& a, dim3 grid, size_t lds_bytes, hipStream_t st) {
    constexpr int KSETS = wgrad_f32_ksets(8, VEC);
    if (mode == 16) {
        hipLaunchKernelGGL((qconv_wgrad_f32_kernel<TS, 16, 3, VEC, 1>), grid, dim3(WG_THREADS), lds_bytes, st, a);
    } else {
        // (eight waves: one workgroup per CU, which may then use more than 64 KiB of LDS -- opted in at set-up, see BigLds)
        constexpr auto kernel = qconv_wgrad_f32_kernel<TS, 8, 1, VEC, KSETS>;
        if constexpr (KSETS == 2) {
            if (!BigLds<kernel>::registered) return;
        }
        hipLaunchKernelGGL(kernel, grid, dim3(WG_THREADS * KSETS), lds_bytes, st, a);
    }
}

int launch_wgrad_f32(bool half_storage, bool vec, int mode, const WgradArgs& a, dim3 grid, size_t lds_bytes,
                     hipStream_t st) {
    if (half_storage) vec ? launch_ts<_Float16, true>(mode, a, grid, lds_bytes, st) : launch_ts<_Float16, false>(mode, a, grid, lds_bytes, st);
    else vec ? launch_ts<float, true>(mode, a, grid, lds_bytes, st) : launch_ts<float, false>(mode, a, grid, lds_bytes, st);
    return 0;
}

int launch_reduce_wgrad(bool half_storage, const ReduceArgs& a, hipStream_t st) {
    const long groups = 4L * a.Kh * a.Kw * a.Co * ((a.Ci + 3) / 4);
    const int per_wg = WG_THREADS / reduce_slices(a.Z);
    const int blocks = (int)((groups + per_wg - 1) / per_wg);
    if (half_storage) hipLaunchKernelGGL((reduce_wgrad_kernel<_Float16>), dim3(blocks, grid_rows(a.groups)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((reduce_wgrad_kernel<float>), dim3(blocks, grid_rows(a.groups)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

}  // namespace phx
