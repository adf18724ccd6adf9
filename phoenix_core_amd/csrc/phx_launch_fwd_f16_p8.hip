// fp16-MFMA forward / input-gradient kernels with both operands through LDS, factorized 8-product form.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

template <int MAP>
static int launch_lds8(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
#define PHX_CASE(WCO_, NTW_)                                                                                       \
    if (v.WCO == WCO_ && v.NTW == NTW_) {                                                                          \
        constexpr auto kernel = qconv_fwd_f16_lds_kernel<8, MAP, WCO_, NTW_, 8, true>;                             \
        /* more than 64 KiB of dynamic LDS: opted in per device at set-up, see BigLds */                           \
        if (!BigLds<kernel>::registered) return -1;                                                                \
        hipLaunchKernelGGL(kernel, dim3(v.wgs), dim3(WG_THREADS), v.lds_bytes, st, a);                             \
        return 0;                                                                                                  \
    }
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1) PHX_CASE(2, 2)
#undef PHX_CASE
    return -1;
}

int launch_fwd_f16_lds8(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    return v.map == MAP_FWD ? launch_lds8<MAP_FWD>(v, a, st) : launch_lds8<MAP_DGRAD>(v, a, st);
}

}  // namespace phx
