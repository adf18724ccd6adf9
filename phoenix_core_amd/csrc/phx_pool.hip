// 3x3 / stride 2 / padding 1 max pooling for the ResNet harness (include/phx_pool.h).
#include <hip/hip_runtime.h>

#include <cmath>

#include "../../include/phx_pool.h"
#include "phx_device.h"

namespace phx {

struct PoolArgs {
    const void* in;        // forward: x; backward: dy
    void* out;             // forward: y; backward: dx
    unsigned char* index;  // [planes][Ho][Wo]
    int H, W, Ho, Wo;
    unsigned int per_plane;  // workgroups per plane
};

// Workgroup = (plane, run of 256 outputs of that plane): 32-bit index arithmetic throughout.
// One thread per output element: the nine window positions in row-major order, padding positions skipped.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) maxpool_fwd_kernel(const PoolArgs P) {
    const unsigned int plane = blockIdx.x / P.per_plane, run = blockIdx.x - plane * P.per_plane;
    const int pos = (int)(run * WG_THREADS + threadIdx.x);
    if (pos >= P.Ho * P.Wo) return;
    const int oh = pos / P.Wo, ow = pos - oh * P.Wo;
    const TS* xp = static_cast<const TS*>(P.in) + (long)plane * P.H * P.W;
    // the first maximum in scan order, starting from the first position inside the image; a NaN is taken
    // whenever it is met (torch's rule: `val > max || isnan(val)`)
    float best = -INFINITY;
    int arg = (oh == 0 ? 3 : 0) + (ow == 0 ? 1 : 0);
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
        const int h = 2 * oh - 1 + kh;
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
            const int w = 2 * ow - 1 + kw;
            if (h >= 0 && h < P.H && w >= 0 && w < P.W) {
                const float v = (float)xp[h * P.W + w];
                if (v > best || v != v) { best = v; arg = kh * 3 + kw; }
            }
        }
    }
    const long o = (long)plane * P.Ho * P.Wo + pos;
    static_cast<TS*>(P.out)[o] = (TS)best;
    P.index[o] = (unsigned char)arg;
}

// One thread per pair of input elements (h, 2k), (h, 2k + 1).  The window rows that cover row h are
// oh in [h / 2, (h + 1) / 2]; column 2k lies in window column k only (position 1 of its row), column 2k + 1 in
// window columns k (position 2) and k + 1 (position 0).  Sums in fp32, windows in row-major order.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) maxpool_bwd_kernel(const PoolArgs P) {
    const unsigned int plane = blockIdx.x / P.per_plane, run = blockIdx.x - plane * P.per_plane;
    const int WP = (P.W + 1) >> 1;
    const int pos = (int)(run * WG_THREADS + threadIdx.x);
    if (pos >= P.H * WP) return;
    const int h = pos / WP, k = pos - h * WP;
    const long obase = (long)plane * P.Ho * P.Wo;
    const TS* dy = static_cast<const TS*>(P.in) + obase;
    const unsigned char* index = P.index + obase;
    const int oh0 = h >> 1, oh1 = min((h + 1) >> 1, P.Ho - 1);
    const bool right = k + 1 < P.Wo;  // window column k + 1 exists
    float even = 0.f, odd = 0.f;
    for (int oh = oh0; oh <= oh1; ++oh) {
        const int kh3 = (h - (2 * oh - 1)) * 3;
        const int o = oh * P.Wo + k;
        const int a = index[o];
        const float ga = (float)dy[o];
        if (a == kh3 + 1) even += ga;
        if (a == kh3 + 2) odd += ga;
        if (right && index[o + 1] == kh3) odd += (float)dy[o + 1];
    }
    TS* dx = static_cast<TS*>(P.out) + (long)plane * P.H * P.W + h * P.W + 2 * k;
    if (2 * k + 1 < P.W) {
        if constexpr (sizeof(TS) == 2) {
            if (!(P.W & 1)) {  // rows start on 4-byte boundaries: one store for the pair
                f16x2 v;
                v[0] = (TS)even; v[1] = (TS)odd;
                *reinterpret_cast<f16x2*>(dx) = v;
                return;
            }
        }
        dx[0] = (TS)even;
        dx[1] = (TS)odd;
    } else {
        dx[0] = (TS)even;
    }
}

// fp16 forms with 16-byte accesses (2-byte alignment is all a row start guarantees: the loads and stores below
// are declared so).  Forward: a thread makes 4 consecutive outputs of a row from input columns 8m - 1 .. 8m + 7.
typedef unsigned int u32_a1 __attribute__((aligned(1)));

__global__ void __launch_bounds__(WG_THREADS) maxpool_fwd_f16x4_kernel(const PoolArgs P) {
    const unsigned int plane = blockIdx.x / P.per_plane, run = blockIdx.x - plane * P.per_plane;
    const int WQ = (P.Wo + 3) >> 2;  // threads per output row
    const int pos = (int)(run * WG_THREADS + threadIdx.x);
    if (pos >= P.Ho * WQ) return;
    const int oh = pos / WQ, ow0 = (pos - oh * WQ) * 4;
    const _Float16* xp = static_cast<const _Float16*>(P.in) + (long)plane * P.H * P.W;
    const int c0 = 2 * ow0;
    float best[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    int arg[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) arg[q] = (oh == 0 ? 3 : 0) + (ow0 + q == 0 ? 1 : 0);
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
        const int h = 2 * oh - 1 + kh;
        if (h < 0 || h >= P.H) continue;
        const _Float16* row = xp + h * P.W;
        float v[9];  // columns c0 - 1 .. c0 + 7; NaN-free filler outside the image is never looked at (see `in` below)
        v[0] = c0 > 0 ? (float)row[c0 - 1] : 0.f;
        if (c0 + 8 <= P.W) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // four dword loads at consecutive addresses (merged by the compiler)
                const f16x2 pair = __builtin_bit_cast(f16x2, load4_a2(row + c0 + 2 * i));
                v[1 + 2 * i] = (float)pair[0];
                v[2 + 2 * i] = (float)pair[1];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[1 + i] = c0 + i < P.W ? (float)row[c0 + i] : 0.f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int w = c0 + 2 * q - 1 + kw;
                const bool in = w >= 0 && w < P.W;
                const float val = v[2 * q + kw];
                if (in && (val > best[q] || val != val)) { best[q] = val; arg[q] = kh * 3 + kw; }
            }
    }
    const long o = (long)plane * P.Ho * P.Wo + oh * P.Wo + ow0;
    _Float16* y = static_cast<_Float16*>(P.out) + o;
    if (ow0 + 4 <= P.Wo) {
        f16x2 lo, hi;
        lo[0] = (_Float16)best[0]; lo[1] = (_Float16)best[1]; hi[0] = (_Float16)best[2]; hi[1] = (_Float16)best[3];
        u32x2 yv;
        yv[0] = __builtin_bit_cast(unsigned int, lo); yv[1] = __builtin_bit_cast(unsigned int, hi);
        *reinterpret_cast<u32x2_a2*>(y) = yv;
        *reinterpret_cast<u32_a1*>(P.index + o) = (unsigned int)arg[0] | (unsigned int)arg[1] << 8 | (unsigned int)arg[2] << 16 |
                                                  (unsigned int)arg[3] << 24;
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (ow0 + q < P.Wo) { y[q] = (_Float16)best[q]; P.index[o + q] = (unsigned char)arg[q]; }
    }
}

// Backward: a thread makes 8 consecutive input elements of a row (pairs k0 .. k0 + 3) from window columns
// k0 .. k0 + 4 of the one or two window rows that cover the row.
__global__ void __launch_bounds__(WG_THREADS) maxpool_bwd_f16x8_kernel(const PoolArgs P) {
    const unsigned int plane = blockIdx.x / P.per_plane, run = blockIdx.x - plane * P.per_plane;
    const int WO = (P.W + 7) >> 3;  // threads per input row
    const int pos = (int)(run * WG_THREADS + threadIdx.x);
    if (pos >= P.H * WO) return;
    const int h = pos / WO, w0 = (pos - h * WO) * 8, k0 = w0 >> 1;
    const long obase = (long)plane * P.Ho * P.Wo;
    const _Float16* dy = static_cast<const _Float16*>(P.in) + obase;
    const unsigned char* index = P.index + obase;
    const int oh0 = h >> 1, oh1 = min((h + 1) >> 1, P.Ho - 1);
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int oh = oh0; oh <= oh1; ++oh) {
        const int kh3 = (h - (2 * oh - 1)) * 3;
        const int o = oh * P.Wo + k0;
        int a[5];
        float g[5];
        if (k0 + 5 <= P.Wo) {
            const unsigned int a4 = *reinterpret_cast<const u32_a1*>(index + o);
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = (a4 >> (8 * i)) & 0xff;
            a[4] = index[o + 4];
            const f16x2 g01 = __builtin_bit_cast(f16x2, load4_a2(dy + o)), g23 = __builtin_bit_cast(f16x2, load4_a2(dy + o + 2));
            g[0] = (float)g01[0]; g[1] = (float)g01[1]; g[2] = (float)g23[0]; g[3] = (float)g23[1];
            g[4] = (float)dy[o + 4];
        } else {
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                const bool in = k0 + i < P.Wo;
                a[i] = in ? index[o + i] : 255;
                g[i] = in ? (float)dy[o + i] : 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // pair k0 + i: columns 2(k0 + i) and 2(k0 + i) + 1
            if (a[i] == kh3 + 1) sum[2 * i] += g[i];
            if (a[i] == kh3 + 2) sum[2 * i + 1] += g[i];
            if (a[i + 1] == kh3) sum[2 * i + 1] += g[i + 1];
        }
    }
    _Float16* dx = static_cast<_Float16*>(P.out) + (long)plane * P.H * P.W + h * P.W + w0;
    if (w0 + 8 <= P.W) {
        u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f16x2 pr;
            pr[0] = (_Float16)sum[2 * i]; pr[1] = (_Float16)sum[2 * i + 1];
            v[i] = __builtin_bit_cast(unsigned int, pr);
        }
        *reinterpret_cast<u32x4_a2*>(dx) = v;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (w0 + i < P.W) dx[i] = (_Float16)sum[i];
    }
}

static int check(int32_t dtype, int64_t planes, int32_t h, int32_t w) {
    if ((dtype != PHX_F32 && dtype != PHX_F16) || planes < 0 || h < 0 || w < 0) return PHX_ERR_INVALID_ARGUMENT;
    // (32-bit positions inside a plane, and one grid dimension for planes x runs)
    if ((long)h * w >= (1L << 30) || (planes > 0 && h > 0 && w > 0 && planes * (((long)h * w + 255) / 256) >= (1L << 31)))
        return PHX_ERR_NOT_SUPPORTED;
    return PHX_OK;
}

}  // namespace phx

using namespace phx;

extern "C" {

int phx_maxpool3x3s2_fwd(int32_t dtype, int64_t planes, int32_t h, int32_t w, phx_stream_t stream, const void* x, void* y,
                         uint8_t* index) {
    if (const int rc = check(dtype, planes, h, w)) return rc;
    if (planes == 0 || h == 0 || w == 0) return PHX_OK;
    if (!x || !y || !index) return PHX_ERR_INVALID_ARGUMENT;
    PoolArgs a{x, y, index, h, w, (h - 1) / 2 + 1, (w - 1) / 2 + 1, 0};
    const int per_row = dtype == PHX_F16 ? (a.Wo + 3) / 4 : a.Wo;  // threads per output row
    a.per_plane = (unsigned int)((a.Ho * per_row + WG_THREADS - 1) / WG_THREADS);
    const dim3 grid((unsigned int)(planes * a.per_plane));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == PHX_F16) hipLaunchKernelGGL(maxpool_fwd_f16x4_kernel, grid, dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL(maxpool_fwd_kernel<float>, grid, dim3(WG_THREADS), 0, st, a);
    return hipGetLastError() == hipSuccess ? PHX_OK : PHX_ERR_RUNTIME;
}

int phx_maxpool3x3s2_bwd(int32_t dtype, int64_t planes, int32_t h, int32_t w, phx_stream_t stream, const void* dy,
                         const uint8_t* index, void* dx) {
    if (const int rc = check(dtype, planes, h, w)) return rc;
    if (planes == 0 || h == 0 || w == 0) return PHX_OK;
    if (!dy || !dx || !index) return PHX_ERR_INVALID_ARGUMENT;
    PoolArgs a{dy, dx, const_cast<uint8_t*>(index), h, w, (h - 1) / 2 + 1, (w - 1) / 2 + 1, 0};
    const int per_row = dtype == PHX_F16 ? (w + 7) / 8 : (w + 1) / 2;  // threads per input row
    a.per_plane = (unsigned int)((h * per_row + WG_THREADS - 1) / WG_THREADS);
    const dim3 grid((unsigned int)(planes * a.per_plane));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == PHX_F16) hipLaunchKernelGGL(maxpool_bwd_f16x8_kernel, grid, dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL(maxpool_bwd_kernel<float>, grid, dim3(WG_THREADS), 0, st, a);
    return hipGetLastError() == hipSuccess ? PHX_OK : PHX_ERR_RUNTIME;
}

}  // extern "C"
