// Pointwise fp16-MFMA kernels with the packed filter resident in LDS (phx_kernels_pwr16.h): instantiations.
#include "phx_kernels_pwr16.h"
#include "phx_launch.h"

namespace phx {

template <int WCO, bool ADD>
static int launch_pwr_one(const PwxArgs& a, int blocks, size_t lds_bytes, hipStream_t st) {
    constexpr auto kernel = qconv_pwr_f16_kernel<WCO, ADD>;
    if (!BigLds<kernel>::registered) return -1;  // more than 64 KiB of dynamic LDS: opted in per device at set-up, see BigLds
    hipLaunchKernelGGL(kernel, dim3(blocks, grid_rows(a.groups)), dim3(WG_THREADS), lds_bytes, st, a);
    return 0;
}

// LDS of a workgroup: the filter image (K steps x sub-tiles x 4 components x 64 lanes x 16 bytes) and four waves' rings
size_t pwr_lds_bytes(int WCO, int nsteps) {
    return ((size_t)nsteps * WCO * 4 * 64 + 4 * PWR_STAGES * PWR_STAGE_VEC) * 16;
}

int launch_pwr_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st) {
    const size_t lds = pwr_lds_bytes(WCO, a.nsteps);
    if (lds > 160 * 1024 || a.co_tiles != 1 || a.nsteps < 2 || a.HW % 8 != 0 || a.GI * 8 != a.HW) return -1;
    const bool add = a.addend != nullptr;
    if (WCO == 4) return add ? launch_pwr_one<4, true>(a, blocks, lds, st) : launch_pwr_one<4, false>(a, blocks, lds, st);
    if (WCO == 2) return add ? launch_pwr_one<2, true>(a, blocks, lds, st) : launch_pwr_one<2, false>(a, blocks, lds, st);
    if (WCO == 1) return add ? launch_pwr_one<1, true>(a, blocks, lds, st) : launch_pwr_one<1, false>(a, blocks, lds, st);
    return -1;
}

}  // namespace phx
