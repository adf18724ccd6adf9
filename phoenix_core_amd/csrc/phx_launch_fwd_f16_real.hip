// fp16-MFMA forward kernels with both operands through LDS, 16-product form, for a real-valued input (one stored
// component): the products with the absent components are compiled out.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

int launch_fwd_f16_lds16_real(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
#define PHX_CASE(WCO_, NTW_)                                                                                   \
    if (v.WCO == WCO_ && v.NTW == NTW_) {                                                                      \
        constexpr auto kernel = qconv_fwd_f16_lds_kernel<16, WCO_, NTW_, 8, true, false, true>;                \
        if (!BigLds<kernel>::registered) return -1; /* dynamic LDS opt-in at set-up, see BigLds */             \
        hipLaunchKernelGGL(kernel, dim3(v.wgs, grid_rows(a.groups)), dim3(WG_THREADS), v.lds_bytes, st, a);                         \
        return 0;                                                                                              \
    }
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1) PHX_CASE(2, 2) PHX_CASE(4, 1) PHX_CASE(4, 2)
#undef PHX_CASE
    return -1;
}

}  // namespace phx
