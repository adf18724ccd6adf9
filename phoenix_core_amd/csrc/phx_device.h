// Shared device-side helpers of the gfx950 quaternion kernels: vector types, storage<->compute
// conversions, the Hamilton sign table, the lane maps of the factorized product and the generic
// global->LDS tile loader.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace phx {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;
constexpr int WG_THREADS = 256;

// y = x (x) w as a real block matrix: y_q = sum_p M[p][q] * x_p with M[p][q] = sign(p,q) * w_{p^q}
// (rows = input component, columns = output component; src/algebras.cc:28-49 of the reference).
// Negative entries: (1,0) (1,2) (2,0) (2,3) (3,0) (3,1).
__host__ __device__ constexpr bool qneg(int p, int q) { return (0x3950u >> (p * 4 + q)) & 1u; }

template <typename T>
__device__ __forceinline__ float ldf(const T* p);
template <>
__device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ldf<_Float16>(const _Float16* p) { return (float)*p; }

template <typename T>
__device__ __forceinline__ void stf(T* p, float v);
template <>
__device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void stf<_Float16>(_Float16* p, float v) { *p = (_Float16)v; }

// Lane maps of the factorized (8-product) Hamilton product.  Same arithmetic as the reference's
// TensorManipulations lane maps (src/backend/onednn/tensor.hpp:61-170), applied to registers.
template <typename V>
__device__ __forceinline__ void lanes_left(const V (&x)[4], V (&L)[8]) {
    L[0] = x[3] + x[1];
    L[1] = x[0] - x[2];
    L[2] = x[0] + x[2];
    L[3] = x[3] - x[1];
    L[4] = x[3] - x[2];
    L[5] = x[1] + x[0];
    L[6] = x[0] - x[1];
    L[7] = x[3] + x[2];
}

template <typename V>
__device__ __forceinline__ void lanes_right(const V (&w)[4], V (&R)[8]) {
    R[0] = w[1] + w[2];
    R[1] = w[0] + w[3];
    R[2] = w[0] - w[3];
    R[3] = w[1] - w[2];
    R[4] = w[2] - w[3];
    R[5] = w[1] + w[0];
    R[6] = w[2] + w[3];
    R[7] = w[0] - w[1];
}

template <typename V, typename S>
__device__ __forceinline__ void lanes_grad(const V (&g)[4], V (&G)[8], S half) {
    const V t1 = g[0] + g[1], t3 = g[0] - g[1], t2 = g[2] + g[3], t4 = g[2] - g[3];
    G[0] = (t2 - t1) * half;
    G[1] = (t3 - t4) * half;
    G[2] = (t3 + t4) * half;
    G[3] = (t1 + t2) * half;
    G[4] = g[0];
    G[5] = g[1];
    G[6] = g[2];
    G[7] = g[3];
}

// 8 product lanes -> 4 output components (recomposeQuaternionOutput)
template <typename V>
__device__ __forceinline__ void merge_output(const V (&P)[8], V (&y)[4]) {
    const V a2 = P[0] + P[1] + P[2];
    const V a5 = (a2 + P[3]) * 0.5f;
    y[0] = a5 - P[0] + P[4];
    y[1] = a5 - a2 + P[5];
    y[2] = a5 - P[1] + P[6];
    y[3] = a5 - P[2] + P[7];
}

// 8 lane gradients -> left-operand (input) gradient
template <typename V>
__device__ __forceinline__ void merge_left_grad(const V (&d)[8], V (&y)[4]) {
    y[0] = d[1] + d[2] + d[5] + d[6];
    y[1] = d[0] - d[3] + d[5] - d[6];
    y[2] = d[2] - d[1] - d[4] + d[7];
    y[3] = d[0] + d[3] + d[4] + d[7];
}

// 8 lane gradients -> right-operand (filter) gradient
template <typename V>
__device__ __forceinline__ void merge_right_grad(const V (&d)[8], V (&y)[4]) {
    y[0] = d[1] + d[2] + d[5] + d[7];
    y[1] = d[0] + d[3] + d[5] - d[7];
    y[2] = d[0] - d[3] + d[4] + d[6];
    y[3] = d[1] - d[2] - d[4] + d[6];
}

// Hardware workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Map the
// hardware id to a logical id such that consecutive logical ids share an XCD, so that tiles
// reading the same activations (neighbouring pixel tiles, the filter tiles of one pixel tile)
// meet in one L2.
__device__ __forceinline__ int xcd_remap(int hw_id, int total) {
    constexpr int XCDS = 8;
    const int xcd = hw_id % XCDS, slot = hw_id / XCDS;
    const int base = total / XCDS, rem = total % XCDS;
    return xcd * base + (xcd < rem ? xcd : rem) + slot;
}

// A rectangular window of a component-stacked NCHW tensor t[4][N][C][Hd][Wd], seen through an
// optional zero-insertion (virtual coordinate v maps to stored v/u when v % u == 0, else zero).
struct TileSrc {
    const void* base;
    long comp_stride;  // elements between components
    int N, C, Hd, Wd;  // stored dims per component
    int uh, uw;        // zero-insertion factors (1 = none)
};

// Copies the window [n0, n0+NB) x [c0, c0+NCH) x [h0, h0+HTH) x [w0, w0+HTW) of all four
// components into LDS as dst[(p*NCH + c)*pitch + (nb*HTH + hr)*HTW + hc], zero-filling whatever
// falls outside the tensor.  Rows are dealt to groups of `lpr` adjacent lanes so that global
// reads run along W.
template <typename TS, int NCH, typename TD>
__device__ __forceinline__ void stage_window(TD* dst, const TileSrc& s, int n0, int c0, int h0, int w0, int NB,
                                             int HTH, int HTW, int pitch, int lpr_log2) {
    const TS* base = static_cast<const TS*>(s.base);
    const int lpr = 1 << lpr_log2;
    const int rl = threadIdx.x & (lpr - 1);
    const int worker = threadIdx.x >> lpr_log2;
    const int workers = WG_THREADS >> lpr_log2;
    const int rows_per_c = NB * HTH;
    const int rows = 4 * NCH * rows_per_c;
    const long plane = (long)s.Hd * s.Wd;
    for (int row = worker; row < rows; row += workers) {
        const int pc = row / rows_per_c;
        const int rr = row - pc * rows_per_c;
        const int nb = rr / HTH;
        const int hr = rr - nb * HTH;
        const int p = pc / NCH, c = pc - p * NCH;
        int vh = h0 + hr;
        bool ok = (c0 + c < s.C) && (n0 + nb < s.N) && vh >= 0;
        if (s.uh > 1) {
            ok = ok && (vh % s.uh == 0);
            vh /= s.uh;
        }
        ok = ok && vh < s.Hd;
        const TS* src = base + p * s.comp_stride + ((long)(n0 + nb) * s.C + c0 + c) * plane + (long)vh * s.Wd;
        TD* out = dst + (long)pc * pitch + rr * HTW;
        if (s.uw == 1) {
            for (int hc = rl; hc < HTW; hc += lpr) {
                const int vw = w0 + hc;
                float v = 0.f;
                if (ok && vw >= 0 && vw < s.Wd) v = ldf<TS>(src + vw);
                out[hc] = (TD)v;
            }
        } else {
            for (int hc = rl; hc < HTW; hc += lpr) {
                const int vw = w0 + hc;
                float v = 0.f;
                if (ok && vw >= 0 && (vw % s.uw == 0) && (vw / s.uw) < s.Wd) v = ldf<TS>(src + vw / s.uw);
                out[hc] = (TD)v;
            }
        }
    }
}

}  // namespace phx
