// Instantiations of the fp16-MFMA forward / input-gradient kernels and their filter packing.
#include "phx_kernels_f16.h"
#include "phx_launch.h"

namespace phx {

template <int MODE, bool PAIRS>
static int launch_variant16(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    constexpr int P2A = 8, P2B = PAIRS ? 8 : 7;  // the pair path has a single staging shape
#define PHX_CASE(WCO_, NTW_, P2_)                                                                             \
    if (v.WCO == WCO_ && v.NTW == NTW_ && (PAIRS || v.P2LOG == P2_)) {                                        \
        hipLaunchKernelGGL((qconv_fwd_f16_kernel<MODE, WCO_, NTW_, P2_, PAIRS>), dim3(v.wgs, grid_rows(a.groups)),                 \
                           dim3(WG_THREADS), v.lds_bytes, st, a);                                             \
        return 0;                                                                                             \
    }
#define PHX_CASES(WCO_, NTW_) PHX_CASE(WCO_, NTW_, P2A) PHX_CASE(WCO_, NTW_, P2B)
    PHX_CASES(1, 1) PHX_CASES(2, 1) PHX_CASES(4, 1)
    if constexpr (MODE == 16) {
        PHX_CASES(1, 2) PHX_CASES(2, 2) PHX_CASES(4, 2)
    }
#undef PHX_CASES
#undef PHX_CASE
    return -1;
}

template <bool PAIRS>
static int launch_v1(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    if (v.mode == 16) return launch_variant16<16, PAIRS>(v, a, st);
    return launch_variant16<8, PAIRS>(v, a, st);
}

template <bool CHUNKS>
static int launch_lds16(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    constexpr int P2A = 8, P2B = CHUNKS ? 8 : 7;  // chunk staging has a single shape
#define PHX_CASE(WCO_, NTW_, P2_)                                                                             \
    if (v.WCO == WCO_ && v.NTW == NTW_ && (CHUNKS || v.P2LOG == P2_)) {                                        \
        constexpr auto kernel = qconv_fwd_f16_lds_kernel<16, WCO_, NTW_, P2_, CHUNKS>;              \
        if (!BigLds<kernel>::registered) return -1; /* dynamic LDS opt-in at set-up, see BigLds */            \
        hipLaunchKernelGGL(kernel, dim3(v.wgs, grid_rows(a.groups)), dim3(WG_THREADS), v.lds_bytes, st, a);                        \
        return 0;                                                                                             \
    }
    if constexpr (CHUNKS) {
        // one filter group per chunk (pointwise problems): the variant that requests the next chunk first
        if (v.ngroups == 1 && v.NTW == 1 && !tuning_noearly()) {
            if (v.WCO == 1) {
                constexpr auto kernel = qconv_fwd_f16_lds_kernel<16, 1, 1, 8, true, true>;
                if (!BigLds<kernel>::registered) return -1;
                hipLaunchKernelGGL(kernel, dim3(v.wgs, grid_rows(a.groups)), dim3(WG_THREADS), v.lds_bytes, st, a);
                return 0;
            }
            if (v.WCO == 2) {
                constexpr auto kernel = qconv_fwd_f16_lds_kernel<16, 2, 1, 8, true, true>;
                if (!BigLds<kernel>::registered) return -1;
                hipLaunchKernelGGL(kernel, dim3(v.wgs, grid_rows(a.groups)), dim3(WG_THREADS), v.lds_bytes, st, a);
                return 0;
            }
        }
    }
    PHX_CASE(1, 1, P2A) PHX_CASE(1, 1, P2B) PHX_CASE(1, 2, P2A) PHX_CASE(1, 2, P2B)
    PHX_CASE(2, 1, P2A) PHX_CASE(2, 1, P2B) PHX_CASE(2, 2, P2A) PHX_CASE(2, 2, P2B)
    PHX_CASE(4, 1, P2A) PHX_CASE(4, 1, P2B) PHX_CASE(4, 2, P2A) PHX_CASE(4, 2, P2B)
#undef PHX_CASE
    return -1;
}

int launch_fwd_f16(const FwdVariant& v, const ConvArgs& a, hipStream_t st) {
    if (v.lds_filters && v.mode == 8) return launch_fwd_f16_lds8(v, a, st);
    // real-valued input (one stored component), several filter groups per chunk: the variant without the absent products
    if (v.lds_filters && v.chunks && a.in.ncomp == 1 && !(v.ngroups == 1 && v.NTW == 1)) return launch_fwd_f16_lds16_real(v, a, st);
    if (v.lds_filters) return v.chunks ? launch_lds16<true>(v, a, st) : launch_lds16<false>(v, a, st);
    return v.pairs ? launch_v1<true>(v, a, st) : launch_v1<false>(v, a, st);
}

int launch_pack_filters_f16(const FwdVariant& v, const PackArgs& a, int blocks, hipStream_t st) {
    const dim3 g(blocks, grid_rows(a.groups)), b(WG_THREADS);
    if (v.lds_filters) {
        PackLdsArgs la{a, v.WCO, v.ngroups, v.pw};
        if (v.mode == 16 && v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f16_lds_kernel<16, MAP_FWD>), g, b, 0, st, la);
        else if (v.mode == 16) hipLaunchKernelGGL((pack_filters_f16_lds_kernel<16, MAP_DGRAD>), g, b, 0, st, la);
        else if (v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f16_lds_kernel<8, MAP_FWD>), g, b, 0, st, la);
        else hipLaunchKernelGGL((pack_filters_f16_lds_kernel<8, MAP_DGRAD>), g, b, 0, st, la);
        return 0;
    }
    if (v.mode == 16 && v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f16_kernel<16, MAP_FWD>), g, b, 0, st, a);
    else if (v.mode == 16) hipLaunchKernelGGL((pack_filters_f16_kernel<16, MAP_DGRAD>), g, b, 0, st, a);
    else if (v.map == MAP_FWD) hipLaunchKernelGGL((pack_filters_f16_kernel<8, MAP_FWD>), g, b, 0, st, a);
    else hipLaunchKernelGGL((pack_filters_f16_kernel<8, MAP_DGRAD>), g, b, 0, st, a);
    return 0;
}

}  // namespace phx
