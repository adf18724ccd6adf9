// Instantiations of the fp32-MFMA forward / input-gradient kernels and their filter packing.
#include "phx_launch.h"

namespace phx {

template <typename TS, int MODE>
static int launch_variant(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
#define PHX_CASE(WCO_, NTW_, CK_, P2_, VS_)                                                                   \
    if (v.WCO == WCO_ && v.NTW == NTW_ && v.CK == CK_ && v.P2LOG == P2_ && v.vstage == VS_) {                 \
        hipLaunchKernelGGL((qconv_fwd_f32_kernel<TS, MODE, WCO_, NTW_, CK_, P2_, VS_>), dim3(v.wgs, grid_rows(a.groups)),          \
                           dim3(WG_THREADS), v.lds_bytes, st, a);                                             \
        return 0;                                                                                             \
    }
    // vector staging for every window without zero insertion; the per-position form only in its general shape
#define PHX_CASES(WCO_, NTW_)                                                                       \
    PHX_CASE(WCO_, NTW_, 8, 8, true) PHX_CASE(WCO_, NTW_, 16, 7, true) PHX_CASE(WCO_, NTW_, 32, 6, true) \
    PHX_CASE(WCO_, NTW_, 8, 8, false)
    PHX_CASES(1, 1) PHX_CASES(2, 1) PHX_CASES(4, 1)
    if constexpr (MODE == 16) {
        PHX_CASES(1, 2) PHX_CASES(2, 2) PHX_CASES(4, 2)
    }
#undef PHX_CASES
#undef PHX_CASE
    return -1;
}

template <typename TS>
static int launch_ts(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    // one kernel for both passes: the input gradient differs only in how its filters are packed
    if (v.mode == 16) return launch_variant<TS, 16>(v, a, st);
    return launch_variant<TS, 8>(v, a, st);
}

int launch_fwd_f32(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    return v.half_storage ? launch_ts<_Float16>(v, a, st) : launch_ts<float>(v, a, st);
}

template <typename TS>
static int pack_ts(const FwdVariant& v, const PackArgs& a, int blocks, hipStream_t st) {
    const dim3 g(blocks, grid_rows(a.groups)), b(WG_THREADS);
    if (v.mode == 16 && v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f32_kernel<TS, 16, MAP_FWD>), g, b, 0, st, a);
    else if (v.mode == 16) hipLaunchKernelGGL((pack_filters_f32_kernel<TS, 16, MAP_DGRAD>), g, b, 0, st, a);
    else if (v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f32_kernel<TS, 8, MAP_FWD>), g, b, 0, st, a);
    else hipLaunchKernelGGL((pack_filters_f32_kernel<TS, 8, MAP_DGRAD>), g, b, 0, st, a);
    return 0;
}

int launch_pack_filters(const FwdVariant& v, const PackArgs& a, int blocks, hipStream_t st) {
    return v.half_storage ? pack_ts<_Float16>(v, a, blocks, st) : pack_ts<float>(v, a, blocks, st);
}

}  // namespace phx
