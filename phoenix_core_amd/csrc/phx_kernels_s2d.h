// Space-to-depth rewriting of stride-2 convolutions with very few input channels (network stems).
//   y[ho][wo] = sum_{kh,kw} x[2ho + kh - pt][2wo + kw - pl] * w[kh][kw]
// With kh - pt = 2a + b (b in {0,1}) and x'[(c,bh,bw)][i][j] = x[c][2i + bh][2j + bw] this is a
// unit-stride convolution of x' (4x the channels, half the extent) with
//   w'[(c,bh,bw)][ah - amin][aw - amin] = w[c][2ah + bh + pt][2aw + bw + pl]   (zero outside the filter).
// A 7x7 stride-2 stem on 3 channels becomes a 4x4 unit-stride convolution on 12 channels, which the
// tiled kernels run at their usual efficiency; the strided form would stage a 4x larger halo window
// for every output tile and pad 3 channels to a 16-channel K step.
// The three kernels here are the elementwise rearrangements: activations, filters, filter gradient.
#pragma once

#include "phx_device.h"

namespace phx {

struct S2dArgs {
    const void* src;
    void* dst;
    long planes;        // 4N * C image planes
    int H, W, H2, W2;   // source extent, destination extent (ceil(H/2), ceil(W/2))
};

// one thread per (plane, destination row, 4 destination columns): reads 2 rows x 8 source columns
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) s2d_input_kernel(const S2dArgs A) {
    const int wq = (A.W2 + 3) / 4;
    const long total = A.planes * A.H2 * wq;
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const long dplane = (long)A.H2 * A.W2;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int jq = idx % wq;
        const long rest = idx / wq;
        const int i = rest % A.H2;
        const long plane = rest / A.H2;
        const int j0 = jq * 4;
#pragma unroll
        for (int bh = 0; bh < 2; ++bh) {
            const int h = 2 * i + bh;
            TS v[8];
            const TS* row = src + (plane * A.H + h) * A.W + 2 * j0;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = (h < A.H && 2 * j0 + k < A.W) ? row[k] : (TS)0;
#pragma unroll
            for (int bw = 0; bw < 2; ++bw) {
                TS* out = dst + (plane * 4 + bh * 2 + bw) * dplane + (long)i * A.W2 + j0;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (j0 + k < A.W2) out[k] = v[2 * k + bw];
            }
        }
    }
}

// dst[plane][i][j] = src[plane][i * sh + oh][j * sw + ow], zero where that lies outside the source: the input rows and
// columns that one residue class of filter taps reads in a strided convolution (the origin may lie in the padding).
struct StridedGatherArgs {
    const void* src;
    void* dst;
    long planes;        // components x images x channels
    int H, W, H2, W2;   // source and destination extent
    int sh, sw, oh, ow;
};

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) strided_gather_kernel(const StridedGatherArgs A) {
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const long total = A.planes * A.H2 * A.W2;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int j = idx % A.W2;
        const long rest = idx / A.W2;
        const int i = rest % A.H2;
        const long plane = rest / A.H2;
        const long yi = (long)i * A.sh + A.oh, xj = (long)j * A.sw + A.ow;
        dst[idx] = (yi >= 0 && yi < A.H && xj >= 0 && xj < A.W) ? src[(plane * A.H + yi) * A.W + xj] : (TS)0;
    }
}

// e / d for e < 2^24 (exact in fp32), rd = 1.0f / d: the rounded quotient is off by one at most, which the remainder shows
__device__ __forceinline__ unsigned int div24(unsigned int e, unsigned int d, float rd) {
    unsigned int q = (unsigned int)((float)e * rd);
    const int r = (int)(e - q * d);
    if (r < 0) --q;
    else if (r >= (int)d) ++q;
    return q;
}

// Patches to depth.  A convolution whose stride equals its filter extent (patch embeddings, 2x2 / stride 2
// downsampling) reads every input position once, for one output position: with the kh x kw positions of a patch
// laid out as channels,
//   patches[row][q][i][j] = x[row][c][i * kh + a][j * kw + b]   (zero outside the image),
//   q = (c * kh + a) * kw + b (tap_major == 0) or (a * kw + b) * C + c (tap_major == 1),
// it is a pointwise convolution over C * kh * kw channels.  to_caller copies the other way and zeroes the positions
// of the caller's tensor that no patch holds (rows and columns behind the last whole patch).
struct PatchArgs {
    const void* src;
    void* dst;
    long rows;          // components x images
    int C, H, W;        // channels and extent of the caller's tensor
    int Ho, Wo;         // patches per column / row
    int kh, kw;
    int tap_major;
    int CB;             // channels per workgroup item (divides C; set by launch_patch_depth)
};

// 8 consecutive elements of a tensor, stored as one vector where the run is whole and its address aligned
template <typename TS>
struct alignas(8 * sizeof(TS)) PatchRun {
    TS v[8];
};
template <typename TS>
__device__ __forceinline__ void store_run(TS* dst, const PatchRun<TS>& run, unsigned int n) {
    if (n == 8 && (reinterpret_cast<unsigned long>(dst) & (sizeof(PatchRun<TS>) - 1)) == 0) {
        *reinterpret_cast<PatchRun<TS>*>(dst) = run;
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if ((unsigned int)u < n) dst[u] = run.v[u];
    }
}

// A workgroup takes one (component x image, block of CB channels, row a of the patch) at a time: the rows of the
// caller's tensor that hold it serve all kw columns of the patch at once, so each of their cache lines is fetched (or
// written) once, and on the patches' side it touches whole planes.  Index arithmetic is 32-bit, its divisions by fp32 reciprocal (an item has fewer than 2^24 elements).
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) patch_depth_kernel(const PatchArgs A, int to_caller) {
    const int cblocks = A.C / A.CB;
    const long items = A.rows * cblocks * A.kh;
    const unsigned int plane = (unsigned int)A.Ho * A.Wo;
    const long Cq = (long)A.C * A.kh * A.kw;
    // from one patch column to the next, and from one channel to the next, in planes of the patches' tensor
    const long plane_b = A.tap_major ? A.C : 1, plane_c = A.tap_major ? 1 : A.kh * A.kw;
    for (long item = blockIdx.x; item < items; item += gridDim.x) {
        const int a = (int)(item % A.kh);
        const long rest = item / A.kh;
        const int c0 = (int)(rest % cblocks) * A.CB;
        const long row = rest / cblocks;
        const long caller0 = (row * A.C + c0) * A.H * A.W;
        const long q0 = A.tap_major ? (long)a * A.kw * A.C + c0 : ((long)c0 * A.kh + a) * A.kw;  // plane of (c0, a, column 0)
        const long patch0 = (row * Cq + q0) * plane;
        if (!to_caller) {  // every position of the patches is written: those outside the caller's image are zero
            // (one element per thread: neighbouring threads read kw elements apart, from lines that the workgroup's other
            // patch columns use; runs of 8 per thread, as below, spread a wave's reads over 64 lines and measured slower)
            const TS* x = static_cast<const TS*>(A.src) + caller0;
            TS* pt = static_cast<TS*>(A.dst) + patch0;
            const unsigned int per_c = (unsigned int)A.kw * plane, count = per_c * A.CB;
            const float r_per_c = 1.0f / per_c, r_plane = 1.0f / plane, r_Wo = 1.0f / A.Wo;
            if (plane >= 4 * WG_THREADS) {  // large planes: one after the other, one division per element (14 x 14 planes measured slower so)
                for (unsigned int seg = 0; seg < (unsigned int)(A.CB * A.kw); ++seg) {
                    const unsigned int cin = seg / A.kw, b = seg - cin * A.kw;
                    const TS* src = x + (long)cin * A.H * A.W + b;
                    TS* dst = pt + (cin * plane_c + b * plane_b) * plane;
                    for (unsigned int ij = threadIdx.x; ij < plane; ij += WG_THREADS) {
                        const unsigned int i = div24(ij, A.Wo, r_Wo), j = ij - i * A.Wo;
                        const unsigned int yi = i * A.kh + a, xj = j * A.kw;
                        dst[ij] = (yi < (unsigned int)A.H && xj + b < (unsigned int)A.W) ? src[(long)yi * A.W + xj] : (TS)0;
                    }
                }
                continue;
            }
            for (unsigned int e = threadIdx.x; e < count; e += WG_THREADS) {
                const unsigned int cin = div24(e, per_c, r_per_c), r = e - cin * per_c;
                const unsigned int b = div24(r, plane, r_plane), ij = r - b * plane;
                const unsigned int i = div24(ij, A.Wo, r_Wo), j = ij - i * A.Wo;
                const unsigned int yi = i * A.kh + a, xj = j * A.kw + b;
                pt[(cin * plane_c + b * plane_b) * plane + ij] =
                    (yi < (unsigned int)A.H && xj < (unsigned int)A.W) ? x[((long)cin * A.H + yi) * A.W + xj] : (TS)0;
            }
        } else {  // every position of the caller's tensor is written: those outside the patches are zero
            // (a thread works on 8 consecutive elements of a row -- one division set for the first, increments for the
            // rest -- and stores them as one vector where the run is whole and aligned)
            const TS* pt = static_cast<const TS*>(A.src) + patch0;
            TS* x = static_cast<TS*>(A.dst) + caller0;
            const unsigned int Hi = (A.H + A.kh - 1) / A.kh;                // patch rows that touch the caller's image
            const unsigned int gpr = ((unsigned int)A.W + 7) / 8;           // groups of 8 per row of the caller's image
            const unsigned int count = gpr * Hi * A.CB;
            const float r_gpr = 1.0f / gpr, r_Hi = 1.0f / Hi, r_kw = 1.0f / A.kw;
            for (unsigned int g = threadIdx.x; g < count; g += WG_THREADS) {
                const unsigned int rowid = div24(g, gpr, r_gpr), xj0 = (g - rowid * gpr) * 8;
                const unsigned int cin = div24(rowid, Hi, r_Hi), i = rowid - cin * Hi;
                const unsigned int yi = i * A.kh + a;
                if (yi >= (unsigned int)A.H) continue;
                unsigned int j = div24(xj0, A.kw, r_kw), b = xj0 - j * A.kw;
                const unsigned int n = min(8u, (unsigned int)A.W - xj0);
                const TS* src = pt + cin * plane_c * plane + (long)i * A.Wo;
                PatchRun<TS> run;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    run.v[u] = ((unsigned int)u < n && i < (unsigned int)A.Ho && j < (unsigned int)A.Wo) ? src[b * plane_b * plane + j] : (TS)0;
                    if (++b == (unsigned int)A.kw) { b = 0; ++j; }
                }
                store_run(x + ((long)cin * A.H + yi) * A.W + xj0, run, n);
            }
        }
    }
}

// Dilation phases.  With unit stride, an output position and every input position it reads lie dh rows and dw columns
// apart: counted from an origin (oh, ow) = padding before the image modulo the dilation in front of the input (from
// the first position of the output), they share their row modulo dh and their column modulo dw.  The convolution is
// then dh x dw independent UNDILATED convolutions on the phase images, which run as one convolution on a batch
// dh x dw times as long:
//   phases[(row * dh + a) * dw + b][c][i][j] = x[row][c][i * dh + a - oh][j * dw + b - ow]   (zero outside the image)
// to_caller copies the other way (positions of the phase images outside the caller's image are dropped).
struct DilationPhaseArgs {
    const void* src;
    void* dst;
    long rows;          // components x images of the caller's tensor
    int C, H, W;        // channels and extent of the caller's tensor
    int Hp, Wp;         // extent of a phase image: at least ceil((H + oh) / dh), ceil((W + ow) / dw)
    int dh, dw;
    int oh, ow;         // rows / columns of the origin in front of the tensor's first
    int CB;             // channels per workgroup item (divides C; set by launch_dilation_phases)
};

// A workgroup takes one (component x image, block of CB channels, row phase a) at a time: the rows of the caller's
// tensor that it touches are shared by all dw column phases, so each of their cache lines is fetched once, and the
// phase images it touches are runs of CB * Hp * Wp consecutive elements.  Index arithmetic per element is 32-bit, its divisions by fp32 reciprocal (an item has fewer than 2^24 elements).
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) dilation_phase_kernel(const DilationPhaseArgs A, int to_caller) {
    const int cblocks = A.C / A.CB;
    const long items = A.rows * cblocks * A.dh;
    const unsigned int plane = (unsigned int)A.Hp * A.Wp;
    for (long item = blockIdx.x; item < items; item += gridDim.x) {
        const int a = (int)(item % A.dh);
        const long rest = item / A.dh;
        const int c0 = (int)(rest % cblocks) * A.CB;
        const long row = rest / cblocks;
        const long caller0 = (row * A.C + c0) * A.H * A.W;                       // channel c0 of this row in the caller's tensor
        const long phase0 = (row * A.dh + a) * A.dw * A.C * (long)plane + (long)c0 * plane;  // column phase 0, channel c0
        const long phase_b = (long)A.C * plane;                                  // from one column phase to the next
        if (!to_caller) {
            const TS* x = static_cast<const TS*>(A.src) + caller0;
            TS* ph = static_cast<TS*>(A.dst) + phase0;
            const unsigned int per_b = (unsigned int)A.CB * plane, count = per_b * A.dw;
            const float r_per_b = 1.0f / per_b, r_plane = 1.0f / plane, r_Wp = 1.0f / A.Wp;
            for (unsigned int e = threadIdx.x; e < count; e += WG_THREADS) {
                const unsigned int b = div24(e, per_b, r_per_b), in_b = e - b * per_b;  // in_b = (channel, i, j) of the phase image
                const unsigned int cin = div24(in_b, plane, r_plane), ij = in_b - cin * plane;
                const unsigned int i = div24(ij, A.Wp, r_Wp), j = ij - i * A.Wp;
                const int yi = (int)i * A.dh + a - A.oh, xj = (int)j * A.dw + (int)b - A.ow;
                ph[b * phase_b + in_b] =
                    (yi >= 0 && yi < A.H && xj >= 0 && xj < A.W) ? x[((long)cin * A.H + yi) * A.W + xj] : (TS)0;
            }
        } else {
            const TS* ph = static_cast<const TS*>(A.src) + phase0;
            TS* x = static_cast<TS*>(A.dst) + caller0;
            // (one element per thread: the rows of atrous layers' images are short and odd -- 33, 65, 129 -- so runs of 8
            // per thread, as in patch_depth_kernel, rarely store a vector and measured no faster)
            const unsigned int per_c = (unsigned int)A.Hp * A.W, count = per_c * A.CB;
            const float r_per_c = 1.0f / per_c, r_W = 1.0f / A.W, r_dw = 1.0f / A.dw;
            for (unsigned int e = threadIdx.x; e < count; e += WG_THREADS) {
                const unsigned int cin = div24(e, per_c, r_per_c), ix = e - cin * per_c;
                const unsigned int i = div24(ix, A.W, r_W), xj = ix - i * A.W;
                const int yi = (int)i * A.dh + a - A.oh;
                if (yi < 0 || yi >= A.H) continue;
                const unsigned int xo = xj + A.ow, j = div24(xo, A.dw, r_dw), b = xo - j * A.dw;
                x[((long)cin * A.H + yi) * A.W + xj] = ph[b * phase_b + (long)cin * plane + i * A.Wp + j];
            }
        }
    }
}

// Strided pointwise convolutions read every sh-th row and sw-th column of their input and nothing else:
// dst[plane][i][j] = src[plane][i * sh][j * sw] turns them into unit-stride pointwise convolutions, which have the
// streaming kernels.  One thread per 8 destination columns (one 16-byte store).
struct SubsampleArgs {
    const void* src;
    void* dst;
    long planes;        // components x images x channels
    int H, W, H2, W2;   // source and destination extent
    int sh, sw;
};

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) subsample_kernel(const SubsampleArgs A) {
    const int wq = (A.W2 + 7) / 8;
    const long total = A.planes * A.H2 * wq;
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int jq = idx % wq;
        const long rest = idx / wq;
        const int i = rest % A.H2;
        const long plane = rest / A.H2;
        const int j0 = jq * 8;
        const TS* row = src + (plane * A.H + (long)i * A.sh) * A.W;
        TS* out = dst + (plane * A.H2 + i) * A.W2 + j0;
        TS v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = (j0 + k < A.W2) ? row[(long)(j0 + k) * A.sw] : (TS)0;
        if (j0 + 8 <= A.W2 && (reinterpret_cast<size_t>(out) & (8 * sizeof(TS) - 1)) == 0) {
            typedef TS vec8 __attribute__((ext_vector_type(8)));
            vec8 o;
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = v[k];
            *reinterpret_cast<vec8*>(out) = o;
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (j0 + k < A.W2) out[k] = v[k];
        }
    }
}

struct S2dFilterArgs {
    const void* w;      // caller's filters, element (r, o, i, kh, kw) at r*wcs + o*so + i*si + kh*skh + kw*skw
    void* w2;           // rearranged filters [4][Co][4*Ci][K2h][K2w] (OIHW)
    long wcs, so, si, skh, skw;
    int Co, Ci, Kh, Kw, K2h, K2w;
    int pt, pl, aminh, aminw;
};

// to_caller == false: w -> w2;  to_caller == true: dw2 -> dw (every caller element has exactly one image)
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) s2d_filter_kernel(const S2dFilterArgs A, bool to_caller) {
    const TS* src = static_cast<const TS*>(to_caller ? A.w2 : A.w);
    TS* dst = static_cast<TS*>(to_caller ? const_cast<void*>(A.w) : A.w2);
    const int C2 = 4 * A.Ci;
    const long total = 4L * A.Co * C2 * A.K2h * A.K2w;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        long s = idx;
        const int aw = s % A.K2w; s /= A.K2w;
        const int ah = s % A.K2h; s /= A.K2h;
        const int c2 = s % C2; s /= C2;
        const int o = s % A.Co;
        const int r = s / A.Co;
        const int c = c2 >> 2, bh = (c2 >> 1) & 1, bw = c2 & 1;
        const int kh = 2 * (ah + A.aminh) + bh + A.pt, kw = 2 * (aw + A.aminw) + bw + A.pl;
        const bool inside = kh >= 0 && kh < A.Kh && kw >= 0 && kw < A.Kw;
        const long off = r * A.wcs + o * A.so + c * A.si + kh * A.skh + kw * A.skw;
        if (to_caller) {
            if (inside) dst[off] = src[idx];
        } else {
            dst[idx] = inside ? src[off] : (TS)0;
        }
    }
}

// Input gradient of a strided convolution, computed per phase: dx(h, w) with (h % sh, w % sw) = (a, b) is a
// unit-stride correlation of the output gradient with the filter taps that can reach that phase.  The phases
// are computed densely into buffers [4N*C][Hp][Wp] (phase (a, b) at ph[a*sw + b]; an offset of -1 marks a
// phase no tap reaches, which is zero) and interleaved into dx here: coalesced writes, one pass.
struct PhaseMergeArgs {
    const void* buf;      // start of the phase buffers
    void* dx;
    long off[64];         // element offset of each phase buffer (a * sw + b), -1 = all zero
    long planes;          // 4N * C
    int H, W, sh, sw;
};

// A thread per 16 bytes of a dx row: whole-word stores (rows start at element alignment only, which the store
// tolerates), loads along the sw phase rows that feed the row.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) phase_merge_kernel(const PhaseMergeArgs A) {
    constexpr int V = 16 / sizeof(TS);
    const TS* buf = static_cast<const TS*>(A.buf);
    TS* dx = static_cast<TS*>(A.dx);
    const int cpr = (A.W + V - 1) / V;  // 16-byte words per row
    const long total = A.planes * A.H * cpr;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / cpr;
        const int w0 = (int)(idx - r * cpr) * V;
        const long plane = r / A.H;
        const int h = (int)(r - plane * A.H);
        const int a = h % A.sh, hp = h / A.sh;
        const int Hp = (A.H - a + A.sh - 1) / A.sh;
        TS v[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const int w = w0 + i;
            const int b = w % A.sw;
            const long o = A.off[a * A.sw + b];
            const int Wp = (A.W - b + A.sw - 1) / A.sw;
            v[i] = (o >= 0 && w < A.W) ? buf[o + (plane * Hp + hp) * Wp + w / A.sw] : (TS)0;
        }
        TS* dst = dx + r * A.W + w0;
        if (w0 + V <= A.W) {
            u32x4 raw;
            __builtin_memcpy(&raw, v, 16);
            *reinterpret_cast<__attribute__((address_space(1))) u32x4_a2*>((__attribute__((address_space(1))) _Float16*)dst) = raw;
        } else {
            for (int i = 0; w0 + i < A.W; ++i) dst[i] = v[i];
        }
    }
}

// Channels-last activations: [rows][H][W][C] <-> [rows][C][H][W], i.e. a batch of matrix transposes
// src[b][R][Cc] -> dst[b][Cc][R] (R = H*W, Cc = C towards the kernels' layout; R = C, Cc = H*W back).
struct TransposeArgs {
    const void* src;
    void* dst;
    long batch;
    int R, Cc;
};

// A lane owns a square block of 16-byte rows (8x8 halves, 4x4 floats): it loads the block's rows, transposes it in
// registers (byte permutes for halves, plain register renaming for floats) and stores the transposed rows; the
// 64 lanes of a wave form an 8x8 grid of blocks, so that each load instruction covers 128 contiguous bytes of
// eight source rows and each store instruction 128 contiguous bytes of eight destination rows.  Rows start at
// element alignment only, which the 16-byte accesses tolerate.  Blocks cut by the matrix edge go element by element.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) transpose_kernel(const TransposeArgs A) {
    constexpr int V = 16 / sizeof(TS), T = 8 * V;
    typedef const __attribute__((address_space(1))) u32x4_a2* gload;
    typedef __attribute__((address_space(1))) u32x4_a2* gstore;
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rg = lane >> 3, cg = lane & 7;
    const int tr = (A.R + T - 1) / T, tc = (A.Cc + T - 1) / T;
    const long tiles = A.batch * tr * tc;
    constexpr int WAVES = WG_THREADS / 64;
    for (long t = (long)blockIdx.x * WAVES + wave; t < tiles; t += (long)gridDim.x * WAVES) {
        const long b = t / ((long)tr * tc);
        const int rem = (int)(t - b * tr * tc);
        const int r0 = (rem / tc) * T + rg * V, c0 = (rem % tc) * T + cg * V;
        const TS* s = src + b * A.R * (long)A.Cc;
        TS* d = dst + b * A.R * (long)A.Cc;
        if (r0 + V <= A.R && c0 + V <= A.Cc) {
            u32x4 in[V], out[V];
#pragma unroll
            for (int i = 0; i < V; ++i) in[i] = *(gload)(s + (long)(r0 + i) * A.Cc + c0);
            if constexpr (sizeof(TS) == 4) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i) out[j][i] = in[i][j];
            } else {
                // dword m of output row j: element j of input rows 2m and 2m+1
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int m = 0; m < 4; ++m)
                        out[j][m] = __builtin_amdgcn_perm(in[2 * m + 1][j >> 1], in[2 * m][j >> 1],
                                                          (j & 1) ? 0x07060302u : 0x05040100u);
            }
#pragma unroll
            for (int j = 0; j < V; ++j) *(gstore)(d + (long)(c0 + j) * A.R + r0) = out[j];
        } else if (r0 < A.R && c0 < A.Cc) {
            for (int i = 0; i < V && r0 + i < A.R; ++i)
                for (int j = 0; j < V && c0 + j < A.Cc; ++j) d[(long)(c0 + j) * A.R + r0 + i] = s[(long)(r0 + i) * A.Cc + c0 + j];
        }
    }
}

// Merged groups (see merged_groups in phx_qconv.hip): m consecutive groups of a grouped convolution run as one group of
// m * ci -> m * co channels whose filter is block-diagonal.  to_caller == false: w -> w2, the merged filter
// [4][Co][m * ci][Kh][Kw] with zeros off the diagonal blocks; to_caller == true: the diagonal blocks of dw2 -> dw.
struct MergeFilterArgs {
    const void* w;  // caller's filter (or its gradient): element (r, o, i, kh, kw) at r*wcs + o*so + i*si + kh*skh + kw*skw
    void* w2;       // merged filter (or its gradient), OIHW
    long wcs, so, si, skh, skw;
    int Co, ci, co, m, Kh, Kw;  // all output channels; channels of one original group; groups merged into one
};

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) merge_filter_kernel(const MergeFilterArgs A, bool to_caller) {
    const int taps = A.Kh * A.Kw, cim = A.m * A.ci;
    const long total = 4L * A.Co * cim * taps;
    for (long e = (long)blockIdx.x * WG_THREADS + threadIdx.x; e < total; e += (long)gridDim.x * WG_THREADS) {
        const int t = (int)(e % taps);
        long rest = e / taps;
        const int im = (int)(rest % cim);
        rest /= cim;
        const int o = (int)(rest % A.Co), r = (int)(rest / A.Co);
        const int j = im / A.ci, i = im - j * A.ci;
        const bool diagonal = j == (o / A.co) % A.m;
        const int kh = t / A.Kw, kw = t - kh * A.Kw;
        const long at = r * A.wcs + o * A.so + i * A.si + kh * A.skh + kw * A.skw;
        if (to_caller) {
            if (diagonal) static_cast<TS*>(const_cast<void*>(A.w))[at] = static_cast<const TS*>(A.w2)[e];
        } else {
            static_cast<TS*>(A.w2)[e] = diagonal ? static_cast<const TS*>(A.w)[at] : (TS)0.f;
        }
    }
}

}  // namespace phx
