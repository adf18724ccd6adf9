// fp16-MFMA forward / input-gradient kernels with both operands through LDS, factorized 8-product form.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

static int launch_lds8_impl(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
#define PHX_CASE(WCO_, NTW_)                                                                                       \
    if (v.WCO == WCO_ && v.NTW == NTW_) {                                                                          \
        constexpr auto kernel = qconv_fwd_f16_lds_kernel<8, WCO_, NTW_, 8, true>;                             \
        /* more than 64 KiB of dynamic LDS: opted in per device at set-up, see BigLds */                           \
        if (!BigLds<kernel>::registered) return -1;                                                                \
        hipLaunchKernelGGL(kernel, dim3(v.wgs, grid_rows(a.groups)), dim3(WG_THREADS), v.lds_bytes, st, a);                             \
        return 0;                                                                                                  \
    }
    PHX_CASE(1, 1) PHX_CASE(1, 2) PHX_CASE(2, 1) PHX_CASE(2, 2)
#undef PHX_CASE
    return -1;
}

int launch_fwd_f16_lds8(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    // the input gradient is the forward product with the conjugated, mirrored, transposed filter: the packing
    // kernel builds that filter's lanes and the same kernel instance runs both passes
    return launch_lds8_impl(v, a, st);
}

}  // namespace phx
