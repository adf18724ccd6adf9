// fp16-MFMA filter-gradient kernels, 16-product, three taps per workgroup; dispatch over all variants.
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

int launch_wgrad_f16_p16t3(int MT, int NT, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
#define PHX_CASE(MT_, NT_) \
    if (MT == MT_ && NT == NT_) return launch_one<16, MT_, NT_, 3, 1>(a, nblocks, lds_bytes, st);
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1) PHX_CASE(2, 2)
#undef PHX_CASE
    return -1;
}

// four taps per workgroup: channel tiles below 64x64 only (four taps of a 64x64 tile need 256 accumulator registers)
static int launch_wgrad_f16_p16t4(int MT, int NT, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
#define PHX_CASE(MT_, NT_) \
    if (MT == MT_ && NT == NT_) return launch_one<16, MT_, NT_, 4, 1>(a, nblocks, lds_bytes, st);
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1)
#undef PHX_CASE
    return -1;
}

int launch_wgrad_f16(int mode, int MT, int NT, int TPW, int SW, const WgradArgs& a, int nblocks, size_t lds_bytes,
                     hipStream_t st) {
    if (mode == 16 && TPW == 3 && SW == 1) return launch_wgrad_f16_p16t3(MT, NT, a, nblocks, lds_bytes, st);
    if (mode == 16 && TPW == 4 && SW == 1) return launch_wgrad_f16_p16t4(MT, NT, a, nblocks, lds_bytes, st);
    if (TPW != 1) return -1;
    return mode == 16 ? launch_wgrad_f16_p16(MT, NT, 1, SW, a, nblocks, lds_bytes, st)
                      : launch_wgrad_f16_p8(MT, NT, SW, a, nblocks, lds_bytes, st);
}

}  // namespace phx
