// fp16-MFMA filter-gradient kernels, 16-product, one tap per workgroup.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

template <int MODE, int MT, int NT, int TPW, int SW>
static int launch_one(const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
    constexpr auto kernel = qconv_wgrad_f16_kernel<MODE, MT, NT, TPW, SW>;
    if (!BigLds<kernel>::registered) return -1;  // (always true: naming the member makes the registration happen while the library loads)
    hipLaunchKernelGGL(kernel, dim3(nblocks, grid_rows(a.groups)), dim3(WG_THREADS), lds_bytes, st, a);
    return 0;
}

int launch_wgrad_f16_p16(int MT, int NT, int TPW, int SW, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
    if (TPW != 1) return -1;
#define PHX_CASE(MT_, NT_)                                                                      \
    if (MT == MT_ && NT == NT_)                                                                 \
        return SW == 1 ? launch_one<16, MT_, NT_, 1, 1>(a, nblocks, lds_bytes, st)              \
                       : launch_one<16, MT_, NT_, 1, 2>(a, nblocks, lds_bytes, st);
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1) PHX_CASE(2, 2)
#undef PHX_CASE
    return -1;
}

}  // namespace phx
