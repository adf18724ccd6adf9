// fp16-MFMA filter-gradient kernels for channels-last tensors: 16-product, 64x64 channel tiles, one or three taps per workgroup.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

template <int TPW>
static int launch_one(const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
    constexpr auto kernel = qconv_wgrad_f16_kernel<16, 2, 2, TPW, 1, true>;
    if (!BigLds<kernel>::registered) return -1;  // (always true: naming the member makes the registration happen while the library loads)
    hipLaunchKernelGGL(kernel, dim3(nblocks, grid_rows(a.groups)), dim3(WG_THREADS), lds_bytes, st, a);
    return 0;
}

int launch_wgrad_f16_cl(int TPW, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
    if (TPW == 3) return launch_one<3>(a, nblocks, lds_bytes, st);
    if (TPW == 1) return launch_one<1>(a, nblocks, lds_bytes, st);
    return -1;
}

}  // namespace phx
