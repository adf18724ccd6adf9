// Grouped quaternion convolutions with very few channels per group (depthwise convolutions and their kin; `groups`
// reaches the scalar convolutions of the reference as a primitive argument, src/backend/onednn/conv2d.hpp:116-137).
// A matrix-core tile spans 32 x 32 channels of ONE group, so a group of 1..4 channels fills a percent of it and such a
// layer is bound by its tensors' bytes instead: a handful of multiply-adds per element read.  These kernels run it on
// plain fp32 FMA threads, one thread per output quaternion, straight on the caller's tensors and filter (no packing):
//   forward          y[q][n][co][ho][wo] = sum_{i,kh,kw} sum_p s(p,q) x[p][n][g*cig+i][ho*sh-pt+kh*dh][wo*sw-pl+kw*dw] w[p^q][co][i][kh][kw] (+ bias[q][co])
//   input gradient   dx[q][n][ci][h][w]  = sum_{o,kh,kw} sum_p s(p,q) g[p][n][g*cog+o][ho][wo] conj(w)[p^q][g*cog+o][i][kh][kw],  ho*sh-pt+kh*dh == h
//   filter gradient  dw[q][co][i][kh][kw] = sum_{n,ho,wo} sum_p s(p,q) conj(x)[p][n][g*cig+i][..][..] g[p^q][n][co][ho][wo]
// (the products of src/conv2d.hpp:133-160 and :402-470, group by group).  fp32 accumulation whatever the storage
// type: at least as exact as every fp16 policy asks for, and the same result in either product mode.
#include "phx_launch.h"

namespace phx {

// Forward and input gradient: grid row = one channel of the written tensor, so the filter entries a workgroup needs
// (other-side channels of the group x taps, four components each) are the same for all its threads and sit in LDS;
// consecutive threads take consecutive pixels of a row, i.e. consecutive addresses of every plane they read.
template <typename TS, bool DGRAD>
__global__ void __launch_bounds__(WG_THREADS) qconv_thin_kernel(const ThinArgs P) {
    extern __shared__ float4 thin_filter[];  // [other-side channel][tap]
    const int taps = P.Kh * P.Kw;
    const int c = blockIdx.y;  // channel of the written tensor, over all groups
    const int cside = DGRAD ? P.cig : P.cog, K = DGRAD ? P.cog : P.cig;
    const int g = c / cside, c_in_group = c - g * cside;
    const TS* W = static_cast<const TS*>(P.w);
    for (int e = threadIdx.x; e < K * taps; e += WG_THREADS) {
        const int k = e / taps, t = e - k * taps, kh = t / P.Kw, kw = t - kh * P.Kw;
        const long co = DGRAD ? g * P.cog + k : c, ci = DGRAD ? c_in_group : k;
        const TS* at = W + co * P.so + ci * P.si + kh * P.skh + kw * P.skw;
        float4 v;
        v.x = ldf<TS>(at);
        v.y = ldf<TS>(at + P.wcs);
        v.z = ldf<TS>(at + 2 * P.wcs);
        v.w = ldf<TS>(at + 3 * P.wcs);
        if (DGRAD) { v.y = -v.y; v.z = -v.z; v.w = -v.w; }  // conjugate
        thin_filter[e] = v;
    }
    __syncthreads();
    const int Hin = DGRAD ? P.Ho : P.H, Win = DGRAD ? P.Wo : P.W;    // the tensor read
    const int Hout = DGRAD ? P.H : P.Ho, Wout = DGRAD ? P.W : P.Wo;  // the tensor written
    const long opix = (long)Hout * Wout, ipix = (long)Hin * Win;
    const long idx = (long)blockIdx.x * WG_THREADS + threadIdx.x;
    if (idx >= P.N * opix) return;
    const int n = (int)(idx / opix), rem = (int)(idx - n * opix);
    const int oh = rem / Wout, ow = rem - oh * Wout;
    const long Cin_all = (long)P.groups * K, Cout_all = (long)P.groups * cside;
    const long in_cs = P.N * Cin_all * ipix, out_cs = P.N * Cout_all * opix;
    const TS* in = static_cast<const TS*>(P.in) + (n * Cin_all + (long)g * K) * ipix;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (!DGRAD && P.bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = ldf<TS>(static_cast<const TS*>(P.bias) + q * Cout_all + c);
    }
    const auto tap = [&](const TS* px, bool ok, int e) {
        float v[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float f = ldf<TS>(px + p * in_cs);
            v[p] = ok ? f : 0.f;
        }
        const float4 w4 = thin_filter[e];
        const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += (qneg(p, q) ? -v[p] : v[p]) * wv[p ^ q];
    };
    if (!DGRAD || (P.sh == 1 && P.sw == 1)) {
        // no branches around the loads: a tap outside the image reads the plane's first element and counts as zero, so
        // the loads of several taps are in flight together
        for (int k = 0; k < K; ++k, in += ipix) {
            int kh = 0, kw = 0;
#pragma unroll 3
            for (int t = 0; t < taps; ++t) {
                const int ih = DGRAD ? oh + P.pt - kh * P.dh : oh * P.sh - P.pt + kh * P.dh;
                const int iw = DGRAD ? ow + P.pl - kw * P.dw : ow * P.sw - P.pl + kw * P.dw;
                const bool ok = (unsigned)ih < (unsigned)Hin && (unsigned)iw < (unsigned)Win;
                tap(in + (ok ? (long)ih * Win + iw : 0L), ok, k * taps + t);
                if (++kw == P.Kw) { kw = 0; ++kh; }
            }
        }
    } else {
        // strided input gradient: a window entry (kh, kw) reaches this input position from the output position
        // ((h + pt - kh dh) / sh, (w + pl - kw dw) / sw) where both divisions leave no remainder; one entry in sh * sw
        // does, the others are skipped.  Exact division by multiplication: mh = ceil(2^32 / sh) (0: sh == 1).
        const auto divide = [](int t, int s, unsigned int m, int& quotient) {
            quotient = m ? (int)__umulhi((unsigned int)t, m) : t;
            return t >= 0 && quotient * s == t;
        };
        for (int k = 0; k < K; ++k, in += ipix) {
            for (int kh = 0; kh < P.Kh; ++kh) {
                int ih;
                if (!divide(oh + P.pt - kh * P.dh, P.sh, P.mh, ih) || ih >= Hin) continue;
                for (int kw = 0; kw < P.Kw; ++kw) {
                    int iw;
                    if (!divide(ow + P.pl - kw * P.dw, P.sw, P.mw, iw) || iw >= Win) continue;
                    tap(in + (long)ih * Win + iw, true, (k * P.Kh + kh) * P.Kw + kw);
                }
            }
        }
    }
    TS* out = static_cast<TS*>(P.out) + (n * Cout_all + c) * opix + rem;
#pragma unroll
    for (int q = 0; q < 4; ++q) out[q * out_cs] = (TS)acc[q];
}

// Filter gradient: a workgroup sums TB taps of one (output channel, input channel of its group) pair over a slice of
// the images; its threads stride over the slice's output pixels, then meet through the wave shuffles and LDS.  The
// slices' partial sums are added in a fixed order by thin_wgrad_reduce_kernel (no atomics: the result does not depend
// on scheduling).
template <typename TS, int TB>
__global__ void __launch_bounds__(WG_THREADS) qconv_thin_wgrad_kernel(const ThinArgs P) {
    __shared__ float red[WG_THREADS / 64][TB * 4];
    const int pair = blockIdx.x;
    const int co = pair / P.cig, i = pair - co * P.cig, g = co / P.cog;
    const int taps = P.Kh * P.Kw, tap0 = blockIdx.y * TB;
    const int n0 = (int)((long)blockIdx.z * P.N / P.Z), n1 = (int)((long)(blockIdx.z + 1) * P.N / P.Z);
    const long Ci_all = (long)P.groups * P.cig, Co_all = (long)P.groups * P.cog;
    const long xpix = (long)P.H * P.W, gpix = (long)P.Ho * P.Wo;
    const long x_cs = P.N * Ci_all * xpix, g_cs = P.N * Co_all * gpix;
    const TS* x = static_cast<const TS*>(P.in) + ((long)g * P.cig + i) * xpix;
    const TS* gr = static_cast<const TS*>(P.grad) + (long)co * gpix;
    int th[TB], tw[TB];  // window offsets of this workgroup's taps
#pragma unroll
    for (int j = 0; j < TB; ++j) {
        const int t = tap0 + j < taps ? tap0 + j : 0;
        th[j] = (t / P.Kw) * P.dh - P.pt;
        tw[j] = (t % P.Kw) * P.dw - P.pl;
    }
    float acc[TB][4];
#pragma unroll
    for (int j = 0; j < TB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[j][q] = 0.f;
    const long count = (long)(n1 - n0) * gpix;
    for (long idx = threadIdx.x; idx < count; idx += WG_THREADS) {
        const int n = n0 + (int)(idx / gpix), rem = (int)(idx % gpix);
        const int oh = rem / P.Wo, ow = rem - oh * P.Wo;
        float gv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) gv[q] = ldf<TS>(gr + n * Co_all * gpix + rem + q * g_cs);
        const TS* xn = x + n * Ci_all * xpix;
#pragma unroll
        for (int j = 0; j < TB; ++j) {
            const int ih = oh * P.sh + th[j], iw = ow * P.sw + tw[j];
            const bool ok = tap0 + j < taps && (unsigned)ih < (unsigned)P.H && (unsigned)iw < (unsigned)P.W;
            const TS* px = xn + (ok ? (long)ih * P.W + iw : 0L);  // (no branch around the loads: see qconv_thin_kernel)
            float cx[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float v = ldf<TS>(px + p * x_cs);
                cx[p] = !ok ? 0.f : p ? -v : v;  // conjugate
            }
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[j][q] += (qneg(p, q) ? -cx[p] : cx[p]) * gv[p ^ q];
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < TB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float v = acc[j][q];
#pragma unroll
            for (int s = 32; s > 0; s >>= 1) v += __shfl_xor(v, s, 64);
            if (lane == 0) red[wave][j * 4 + q] = v;
        }
    __syncthreads();
    if (threadIdx.x < TB * 4) {
        const int j = threadIdx.x >> 2, q = threadIdx.x & 3;
        if (tap0 + j < taps) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < WG_THREADS / 64; ++w) sum += red[w][threadIdx.x];
            P.partial[(((long)blockIdx.z * gridDim.x + pair) * taps + tap0 + j) * 4 + q] = sum;
        }
    }
}

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) thin_wgrad_reduce_kernel(const ThinArgs P) {
    const int taps = P.Kh * P.Kw;
    const long pairs = (long)P.groups * P.cog * P.cig, total = pairs * taps * 4;
    const long e = (long)blockIdx.x * WG_THREADS + threadIdx.x;
    if (e >= total) return;
    float sum = 0.f;
    for (int z = 0; z < P.Z; ++z) sum += P.partial[z * total + e];
    const int q = (int)(e & 3), t = (int)((e >> 2) % taps);
    const long pair = (e >> 2) / taps;
    const long co = pair / P.cig, i = pair - co * P.cig;
    const int kh = t / P.Kw, kw = t - kh * P.Kw;
    static_cast<TS*>(P.out)[q * P.wcs + co * P.so + i * P.si + kh * P.skh + kw * P.skw] = (TS)sum;
}

int thin_wgrad_taps_per_block(int taps) { return taps == 1 ? 1 : 9; }

int launch_thin(bool half_storage, int pass, const ThinArgs& a, hipStream_t st) {
    const int taps = a.Kh * a.Kw;
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        const long pairs = (long)a.groups * a.cog * a.cig;
        const int TB = thin_wgrad_taps_per_block(taps);
        if (pairs >= (1L << 31) || a.Z < 1 || a.Z > 65535 || !a.partial) return -1;
        const dim3 grid((unsigned int)pairs, (unsigned int)((taps + TB - 1) / TB), (unsigned int)a.Z), block(WG_THREADS);
        if (TB == 1) {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_kernel<_Float16, 1>), grid, block, 0, st, a);
            else hipLaunchKernelGGL((qconv_thin_wgrad_kernel<float, 1>), grid, block, 0, st, a);
        } else {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_kernel<_Float16, 9>), grid, block, 0, st, a);
            else hipLaunchKernelGGL((qconv_thin_wgrad_kernel<float, 9>), grid, block, 0, st, a);
        }
        const dim3 rgrid((unsigned int)((pairs * taps * 4 + WG_THREADS - 1) / WG_THREADS));
        if (half_storage) hipLaunchKernelGGL(thin_wgrad_reduce_kernel<_Float16>, rgrid, block, 0, st, a);
        else hipLaunchKernelGGL(thin_wgrad_reduce_kernel<float>, rgrid, block, 0, st, a);
        return 0;
    }
    const bool dgrad = pass == PHX_PASS_BWD_DATA;
    if (dgrad && (a.sh > 1 || a.sw > 1) && (long)std::max(a.H + a.pt, a.W + a.pl) * std::max(a.sh, a.sw) >= (1L << 31)) return -1;
    const long channels = (long)a.groups * (dgrad ? a.cig : a.cog);
    const long pixels = (long)a.N * (dgrad ? (long)a.H * a.W : (long)a.Ho * a.Wo);
    const long blocks = (pixels + WG_THREADS - 1) / WG_THREADS;
    const size_t lds = (size_t)(dgrad ? a.cog : a.cig) * taps * sizeof(float4);
    if (channels > 65535 || blocks >= (1L << 31) || lds > 48 * 1024) return -1;
    const dim3 grid((unsigned int)blocks, (unsigned int)channels), block(WG_THREADS);
    if (dgrad) {
        if (half_storage) hipLaunchKernelGGL((qconv_thin_kernel<_Float16, true>), grid, block, lds, st, a);
        else hipLaunchKernelGGL((qconv_thin_kernel<float, true>), grid, block, lds, st, a);
    } else {
        if (half_storage) hipLaunchKernelGGL((qconv_thin_kernel<_Float16, false>), grid, block, lds, st, a);
        else hipLaunchKernelGGL((qconv_thin_kernel<float, false>), grid, block, lds, st, a);
    }
    return 0;
}

}  // namespace phx
