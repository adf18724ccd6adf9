// Training-mode batch normalisation (+ optional ReLU) over [rows, C, H*W] activations: the entry points
// of include/phx_bn.h.  HBM-bound streaming kernels; a channel's rows are split over many workgroups and
// the per-split partial sums are combined in a fixed order, so results do not depend on scheduling.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../include/phx_bn.h"
#include "phx_device.h"

namespace phx {

struct BnArgs {
    const void* x;
    const void* dy;      // backward only
    const void* res;     // optional residual added in front of the ReLU (null = none)
    void* out;           // y (forward) or dx (backward)
    void* dres;          // backward with a residual: its gradient (the gradient behind the ReLU)
    const float* gamma;
    const float* beta;
    float* partial;      // [C][S][2]
    float* save_mean;
    float* save_invstd;
    float* run_mean;
    float* run_var;
    float* dgamma;
    float* dbeta;
    int rows, C, hw;
    int S, rows_per_split;  // splits of the row range per channel
    int nchunk;             // 16-byte chunks per (row, channel) plane, the last one possibly partial
    float eps, momentum;
    int relu;
};

template <typename TS>
struct Vec;
template <>
struct Vec<_Float16> {
    static constexpr int N = 8;
};
template <>
struct Vec<float> {
    static constexpr int N = 4;
};

// One 16-byte chunk of a plane as floats; elements past the end of the plane read as zero.  Planes of fp16
// tensors start at 2-byte alignment in general (odd H*W), which the 16-byte access tolerates.
template <typename TS>
__device__ __forceinline__ void load_chunk(const TS* p, int n, float (&v)[Vec<TS>::N]) {
    constexpr int V = Vec<TS>::N;
    if (n == V) {
        const u32x4 raw = load16_a2(reinterpret_cast<const _Float16*>(p));
        if constexpr (sizeof(TS) == 2) {
            const f16x8 h = __builtin_bit_cast(f16x8, raw);
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = (float)h[i];
        } else {
            const f32x4 f = __builtin_bit_cast(f32x4, raw);
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = f[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] = i < n ? (float)p[i] : 0.f;
    }
}

template <typename TS>
__device__ __forceinline__ void store_chunk(TS* p, int n, const float (&v)[Vec<TS>::N]) {
    constexpr int V = Vec<TS>::N;
    if (n == V) {
        u32x4 raw;
        if constexpr (sizeof(TS) == 2) {
            f16x8 h;
#pragma unroll
            for (int i = 0; i < V; ++i) h[i] = (_Float16)v[i];
            raw = __builtin_bit_cast(u32x4, h);
        } else {
            f32x4 f;
#pragma unroll
            for (int i = 0; i < V; ++i) f[i] = v[i];
            raw = __builtin_bit_cast(u32x4, f);
        }
        *reinterpret_cast<__attribute__((address_space(1))) u32x4_a2*>((__attribute__((address_space(1))) _Float16*)p) = raw;
    } else {
        for (int i = 0; i < n; ++i) p[i] = (TS)v[i];
    }
}

// Sum of two values over the workgroup (256 threads), result in every thread.
__device__ __forceinline__ void wg_sum2(float& a, float& b, float (*red)[2]) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        a += __shfl_xor(a, off, 64);
        b += __shfl_xor(b, off, 64);
    }
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // red may still be read from a previous use
    if ((threadIdx.x & 63) == 0) { red[wave][0] = a; red[wave][1] = b; }
    __syncthreads();
    a = red[0][0] + red[1][0] + red[2][0] + red[3][0];
    b = red[0][1] + red[1][1] + red[2][1] + red[3][1];
}

// The channel's totals from its S partial pairs (fixed order inside the reduction tree).
__device__ __forceinline__ void channel_totals(const BnArgs& P, int c, float& t0, float& t1, float (*red)[2]) {
    t0 = 0.f; t1 = 0.f;
    if ((int)threadIdx.x < P.S) {
        t0 = P.partial[((long)c * P.S + threadIdx.x) * 2];
        t1 = P.partial[((long)c * P.S + threadIdx.x) * 2 + 1];
    }
    wg_sum2(t0, t1, red);
}

// MODE 0: sum (x - K), sum (x - K)^2 (forward statistics) with the shift K = the channel's first element: the
// variance is E[(x-K)^2] - E[x-K]^2 whatever K is, and with K inside the data's range the two terms are of the size
// of the variance itself -- the plain E[x^2] - E[x]^2 loses every significant bit of a channel whose mean is large
// against its spread (activations behind a ReLU or a residual add, in fp16).
// MODE 1: sum dy', sum dy' * xhat with dy' the gradient behind the optional ReLU (backward sums).
template <typename TS, int MODE>
__global__ void __launch_bounds__(256) bn_sums_kernel(const BnArgs P) {
    constexpr int V = Vec<TS>::N;
    __shared__ float red[4][2];
    const int c = blockIdx.x, s = blockIdx.y;
    const int b0 = s * P.rows_per_split;
    const int nb = min(P.rows_per_split, P.rows - b0);
    const TS* x = static_cast<const TS*>(P.x);
    const TS* dy = static_cast<const TS*>(P.dy);
    const TS* res = static_cast<const TS*>(P.res);
    float mean = 0.f, invstd = 0.f, g = 0.f, be = 0.f;
    if constexpr (MODE == 1) { mean = P.save_mean[c]; invstd = P.save_invstd[c]; g = P.gamma[c]; be = P.beta[c]; }
    const float shift = (MODE == 0) ? (float)x[(long)c * P.hw] : 0.f;
    float a0 = 0.f, a1 = 0.f;
    const int total = nb * P.nchunk;
    for (int idx = threadIdx.x; idx < total; idx += 256) {
        const int b = idx / P.nchunk, ch = idx - b * P.nchunk;
        long off = ((long)(b0 + b) * P.C + c) * P.hw + ch * V;
        int n = min(V, P.hw - ch * V);
        // The last chunk of a plane that is not a whole number of chunks is read as the full chunk that ENDS at the
        // plane's end (one 16-byte load like the others, no element-wise path that every lane of the wave would walk
        // through); its first `seen` elements belong to the chunk before and are left out of the sums.
        int seen = 0;
        if (n < V && P.hw >= V) { seen = V - n; off -= seen; n = V; }
        float xv[V];
        load_chunk<TS>(x + off, n, xv);
        if constexpr (MODE == 0) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float d = (i < n && i >= seen) ? xv[i] - shift : 0.f;
                a0 += d;
                a1 += d * d;
            }
        } else {
            float dv[V], rv[V];
            load_chunk<TS>(dy + off, n, dv);
            if (res) load_chunk<TS>(res + off, n, rv);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float xh = (xv[i] - mean) * invstd;
                const float dm = (P.relu && g * xh + be + (res ? rv[i] : 0.f) <= 0.f) ? 0.f : dv[i];
                dv[i] = dm;
                const float d = i < seen ? 0.f : dm;
                a0 += d;
                a1 += d * xh;  // (elements past the plane carry dy = 0)
            }
            // With a residual, the gradient behind the ReLU is the residual's gradient: written here, it also saves
            // the apply kernel the reads of dy and the residual and the mask.
            if (P.dres) store_chunk<TS>(static_cast<TS*>(P.dres) + off, n, dv);
        }
    }
    wg_sum2(a0, a1, red);
    if (threadIdx.x == 0) {
        P.partial[((long)c * P.S + s) * 2] = a0;
        P.partial[((long)c * P.S + s) * 2 + 1] = a1;
    }
}

// MODE 0: y = gamma * xhat + beta (ReLU optional); split 0 also records the statistics.
// MODE 1: dx = gamma * invstd * (dy' - mean(dy') - xhat * mean(dy' * xhat)); split 0 writes dgamma, dbeta.
template <typename TS, int MODE>
__global__ void __launch_bounds__(256) bn_apply_kernel(const BnArgs P) {
    constexpr int V = Vec<TS>::N;
    __shared__ float red[4][2];
    const int c = blockIdx.x, s = blockIdx.y;
    const int b0 = s * P.rows_per_split;
    const int nb = min(P.rows_per_split, P.rows - b0);
    const float m = (float)P.rows * (float)P.hw;
    float t0, t1;
    channel_totals(P, c, t0, t1, red);
    const float g = P.gamma[c], be = P.beta[c];
    float mean, invstd;
    if constexpr (MODE == 0) {
        const float shifted = t0 / m;  // mean of x - K, K as in bn_sums_kernel
        mean = (float)static_cast<const TS*>(P.x)[(long)c * P.hw] + shifted;
        const float var = fmaxf(t1 / m - shifted * shifted, 0.f);
        invstd = 1.f / sqrtf(var + P.eps);
        if (s == 0 && threadIdx.x == 0) {
            P.save_mean[c] = mean;
            P.save_invstd[c] = invstd;
            if (P.run_mean) P.run_mean[c] = (1.f - P.momentum) * P.run_mean[c] + P.momentum * mean;
            if (P.run_var) P.run_var[c] = (1.f - P.momentum) * P.run_var[c] + P.momentum * var * (m > 1.f ? m / (m - 1.f) : 1.f);
        }
    } else {
        mean = P.save_mean[c];
        invstd = P.save_invstd[c];
        if (s == 0 && threadIdx.x == 0) { P.dbeta[c] = t0; P.dgamma[c] = t1; }
    }
    const float k0 = t0 / m, k1 = t1 / m, scale = g * invstd;
    const TS* x = static_cast<const TS*>(P.x);
    const TS* dy = static_cast<const TS*>(P.dy);
    const TS* res = static_cast<const TS*>(P.res);
    TS* out = static_cast<TS*>(P.out);
    TS* dres = static_cast<TS*>(P.dres);
    const int total = nb * P.nchunk;
    for (int idx = threadIdx.x; idx < total; idx += 256) {
        const int b = idx / P.nchunk, ch = idx - b * P.nchunk;
        long off = ((long)(b0 + b) * P.C + c) * P.hw + ch * V;
        int n = min(V, P.hw - ch * V);
        // (a plane's last, partial chunk: the full chunk ending at the plane's end instead, as in bn_sums_kernel; the
        // elements it shares with the chunk before are computed and stored twice, with the same values)
        if (n < V && P.hw >= V) { off -= V - n; n = V; }
        float xv[V], ov[V], rv[V];
        load_chunk<TS>(x + off, n, xv);
        if (res && (MODE == 0 || !dres)) load_chunk<TS>(res + off, n, rv);
        if constexpr (MODE == 0) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float y = scale * (xv[i] - mean) + be + (res ? rv[i] : 0.f);
                ov[i] = (P.relu && y < 0.f) ? 0.f : y;
            }
        } else {
            float dv[V];
            if (dres) {  // the masked gradient, as bn_sums_kernel left it
                load_chunk<TS>(dres + off, n, dv);
#pragma unroll
                for (int i = 0; i < V; ++i) ov[i] = scale * (dv[i] - k0 - (xv[i] - mean) * invstd * k1);
            } else {
                load_chunk<TS>(dy + off, n, dv);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float xh = (xv[i] - mean) * invstd;
                    const float d = (P.relu && g * xh + be + (res ? rv[i] : 0.f) <= 0.f) ? 0.f : dv[i];
                    ov[i] = scale * (d - k0 - xh * k1);
                }
            }
        }
        store_chunk<TS>(out + off, n, ov);
    }
}

static int plan(const phx_bn_desc* d, BnArgs& a) {
    if (!d || (d->dtype != PHX_F32 && d->dtype != PHX_F16) || d->rows < 0 || d->c <= 0 || d->hw < 0 || !(d->eps > 0.f))
        return PHX_ERR_INVALID_ARGUMENT;
    if ((long)d->rows * ((d->hw + 3) / 4) >= (1L << 31)) return PHX_ERR_NOT_SUPPORTED;  // chunk indices are 32-bit
    a.rows = d->rows; a.C = d->c; a.hw = d->hw; a.eps = d->eps; a.momentum = d->momentum; a.relu = d->relu;
    const int V = d->dtype == PHX_F16 ? 8 : 4;
    a.nchunk = (d->hw + V - 1) / V;
    // enough workgroups to fill the chip several times over, at most 256 splits (one partial per thread)
    // (fewer, longer-lived workgroups on the small layers -- at least four chunks per thread -- measured slower)
    int S = (2048 + d->c - 1) / d->c;
    S = std::max(1, std::min(S, std::min(std::max(d->rows, 1), 256)));
    a.rows_per_split = (std::max(d->rows, 1) + S - 1) / S;
    a.S = (std::max(d->rows, 1) + a.rows_per_split - 1) / a.rows_per_split;
    return PHX_OK;
}

template <typename TS>
static void launch_all(const BnArgs& a, bool backward, hipStream_t st) {
    const dim3 grid(a.C, a.S);
    if (!backward) {
        hipLaunchKernelGGL((bn_sums_kernel<TS, 0>), grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bn_apply_kernel<TS, 0>), grid, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((bn_sums_kernel<TS, 1>), grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bn_apply_kernel<TS, 1>), grid, dim3(256), 0, st, a);
    }
}

}  // namespace phx

using namespace phx;

extern "C" {

size_t phx_bn_workspace_bytes(const phx_bn_desc* desc) {
    BnArgs a{};
    if (plan(desc, a) != PHX_OK) return 0;
    return ((size_t)a.C * a.S * 2 * sizeof(float) + 255) / 256 * 256;
}

int phx_bn_fwd_train(const phx_bn_desc* desc, phx_stream_t stream, const void* x, const void* residual_or_null,
                     const float* gamma, const float* beta, void* y, float* save_mean, float* save_invstd,
                     float* running_mean_or_null, float* running_var_or_null, void* workspace, size_t workspace_bytes) {
    BnArgs a{};
    const int rc = plan(desc, a);
    if (rc != PHX_OK) return rc;
    if (desc->rows == 0 || desc->hw == 0) return PHX_OK;
    if (!x || !gamma || !beta || !y || !save_mean || !save_invstd) return PHX_ERR_INVALID_ARGUMENT;
    if (!workspace || workspace_bytes < (size_t)a.C * a.S * 2 * sizeof(float)) return PHX_ERR_WORKSPACE;
    a.x = x; a.res = residual_or_null; a.out = y; a.gamma = gamma; a.beta = beta; a.partial = static_cast<float*>(workspace);
    a.save_mean = save_mean; a.save_invstd = save_invstd; a.run_mean = running_mean_or_null; a.run_var = running_var_or_null;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (desc->dtype == PHX_F16) launch_all<_Float16>(a, false, st);
    else launch_all<float>(a, false, st);
    if (hipGetLastError() != hipSuccess) return PHX_ERR_RUNTIME;
    return PHX_OK;
}

int phx_bn_bwd(const phx_bn_desc* desc, phx_stream_t stream, const void* x, const void* residual_or_null, const void* dy,
               const float* gamma, const float* beta, const float* save_mean, const float* save_invstd, void* dx,
               void* dresidual_or_null, float* dgamma, float* dbeta, void* workspace, size_t workspace_bytes) {
    BnArgs a{};
    const int rc = plan(desc, a);
    if (rc != PHX_OK) return rc;
    if (!dgamma || !dbeta) return PHX_ERR_INVALID_ARGUMENT;
    if (desc->rows == 0 || desc->hw == 0) return PHX_OK;
    if (!x || !dy || !gamma || !beta || !save_mean || !save_invstd || !dx) return PHX_ERR_INVALID_ARGUMENT;
    if (!workspace || workspace_bytes < (size_t)a.C * a.S * 2 * sizeof(float)) return PHX_ERR_WORKSPACE;
    if (residual_or_null && !desc->relu) return PHX_ERR_INVALID_ARGUMENT;  // without the ReLU its gradient is dy itself
    a.x = x; a.res = residual_or_null; a.dres = dresidual_or_null; a.dy = dy; a.out = dx; a.gamma = gamma; a.beta = beta; a.partial = static_cast<float*>(workspace);
    a.save_mean = const_cast<float*>(save_mean); a.save_invstd = const_cast<float*>(save_invstd);
    a.dgamma = dgamma; a.dbeta = dbeta;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (desc->dtype == PHX_F16) launch_all<_Float16>(a, true, st);
    else launch_all<float>(a, true, st);
    if (hipGetLastError() != hipSuccess) return PHX_ERR_RUNTIME;
    return PHX_OK;
}

}  // extern "C"
