// Pointwise fp16-MFMA kernels with raw operand copies (phx_kernels_pw16.h): instantiations and their filter packing.
#include "phx_kernels_pw16.h"
#include "phx_launch.h"

namespace phx {

template <int WCO, bool ADD>
static int launch_pwx_one(const PwxArgs& a, int blocks, hipStream_t st) {
    constexpr auto kernel = qconv_pwx_f16_kernel<WCO, ADD>;
    if (!BigLds<kernel>::registered) return -1;  // more than 64 KiB of dynamic LDS: opted in per device at set-up, see BigLds
    hipLaunchKernelGGL(kernel, dim3(blocks, grid_rows(a.groups)), dim3(WG_THREADS), PwxShape<WCO>::lds_bytes_nchw, st, a);
    return 0;
}

int launch_pwx_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st) {
    if (a.addend) {  // the instance that adds a tensor to what it stores
        if (WCO == 4) return launch_pwx_one<4, true>(a, blocks, st);
        if (WCO == 2) return launch_pwx_one<2, true>(a, blocks, st);
        if (WCO == 1) return launch_pwx_one<1, true>(a, blocks, st);
        return -1;
    }
    if (WCO == 4) return launch_pwx_one<4, false>(a, blocks, st);
    if (WCO == 2) return launch_pwx_one<2, false>(a, blocks, st);
    if (WCO == 1) return launch_pwx_one<1, false>(a, blocks, st);
    return -1;
}

template <int WCO>
static int launch_pwx_nhwc_one(const PwxArgs& a, int blocks, hipStream_t st) {
    constexpr auto kernel = qconv_pwx_nhwc_f16_kernel<WCO>;
    if (!BigLds<kernel>::registered) return -1;
    hipLaunchKernelGGL(kernel, dim3(blocks, grid_rows(a.groups)), dim3(WG_THREADS), PwxShape<WCO>::lds_bytes, st, a);
    return 0;
}

int launch_pwx_nhwc_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st) {
    if (WCO == 4) return launch_pwx_nhwc_one<4>(a, blocks, st);
    if (WCO == 2) return launch_pwx_nhwc_one<2>(a, blocks, st);
    if (WCO == 1) return launch_pwx_nhwc_one<1>(a, blocks, st);
    return -1;
}

size_t pwx_packed_bytes(int WCO, int co_tiles, int nsteps) { return (size_t)co_tiles * nsteps * WCO * 4 * 64 * 16; }

int launch_pack_filters_pwx(int map, int WCO, int nsteps, const PackArgs& a, hipStream_t st) {
    PackPwxArgs pa{a, WCO, nsteps};
    const long total = (long)a.row_tiles * nsteps * WCO * 4 * 64;
    const int blocks = (int)std::min<long>((total + WG_THREADS - 1) / WG_THREADS, 4096);
    const dim3 grid(blocks, grid_rows(a.groups));
    if (map == MAP_FWD) hipLaunchKernelGGL((pack_filters_pwx_kernel<MAP_FWD>), grid, dim3(WG_THREADS), 0, st, pa);
    else hipLaunchKernelGGL((pack_filters_pwx_kernel<MAP_DGRAD>), grid, dim3(WG_THREADS), 0, st, pa);
    return 0;
}

}  // namespace phx
