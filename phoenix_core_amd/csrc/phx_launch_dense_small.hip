// Quaternion Dense for small problems (a classifier head, the reference's own 128 -> 128 benchmark layer): the
// matrix-core kernels serve Dense as a 1x1 convolution on 1x1 images, where a batch of 32..64 rows is a single
// pixel tile -- one or two workgroups walking the whole reduction with a pack kernel in front and a split-K
// reduction behind (55 us per pass for 17 MFLOP).  Below a few million quaternion products plain fp32 FMA threads
// are faster: one thread per output quaternion, no packing, no workspace, one launch per pass.
//   forward          y[q][n][o]  = sum_i sum_p s(p,q) x[p][n][i] w[p^q][i][o] (+ bias[q][o])      (src/dense.hpp:77-180)
//   input gradient   dx[q][n][i] = sum_o sum_p s(p,q) g[p][n][o] conj(w)[p^q][i][o]               (src/dense.hpp:252-377)
//   filter gradient  dw[q][i][o] = sum_n sum_p s(p,q) conj(x)[p][n][i] g[p^q][n][o]
// fp32 accumulation whatever the storage type (at least as exact as every fp16 policy asks for); the same result in
// either product mode.
#include "phx_launch.h"

namespace phx {

// Forward and input gradient share one kernel: out[q][a][b] = sum_k sum_p s(p,q) A[p][a][k] B[p^q][k][b], B the
// filter (conjugated for the input gradient), read at the strides of its layout.  A workgroup makes 16 outputs b of
// one row a; its 256 threads split the reduction 16 ways (short dependent-load chains: a thread's loop is nk / 16
// steps) and meet in LDS.  The 16 lanes that run along the filter's contiguous index read 64-byte runs.
struct DenseRowArgs {
    const void* a;     // [4][na][nk]
    const void* b;     // filter: element (c, k, b) at c * b_cs + k * b_ks + b * b_bs
    const void* bias;  // [4][nb] or null
    void* out;         // [4][na][nb]
    long b_cs, b_ks, b_bs;
    int na, nb, nk;
    int kfast;         // the filter is contiguous along k: lanes run along k (else along b)
};

template <typename TS, bool CONJB>
__global__ void __launch_bounds__(WG_THREADS) dense_small_row_kernel(const DenseRowArgs P) {
    __shared__ float part[4][16][17];
    const int tiles_b = (P.nb + 15) >> 4;
    const int a = blockIdx.x / tiles_b, b0 = (blockIdx.x - a * tiles_b) * 16;
    const int lo = threadIdx.x & 15, hi = threadIdx.x >> 4;
    const int bl = P.kfast ? hi : lo, ks = P.kfast ? lo : hi;
    const int b = b0 + bl;
    const bool live = b < P.nb;
    const TS* A = static_cast<const TS*>(P.a) + (long)a * P.nk;
    const TS* B = static_cast<const TS*>(P.b) + (live ? b : 0) * P.b_bs;
    const long acs = (long)P.na * P.nk;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int k = ks; k < P.nk; k += 16) {
        float av[4], bv[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            av[c] = ldf<TS>(A + c * acs + k);
            const float v = ldf<TS>(B + c * P.b_cs + k * P.b_ks);
            bv[c] = (CONJB && c) ? -v : v;
        }
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += (qneg(p, q) ? -av[p] : av[p]) * bv[p ^ q];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) part[q][bl][ks] = acc[q];
    __syncthreads();
    if (threadIdx.x < 64) {  // thread = (component, output): sums the 16 reduction slices in a fixed order
        const int q = threadIdx.x >> 4, ob = threadIdx.x & 15;
        if (b0 + ob < P.nb) {
            float sum = 0.f;
#pragma unroll
            for (int s = 0; s < 16; ++s) sum += part[q][ob][s];
            if (P.bias) sum += ldf<TS>(static_cast<const TS*>(P.bias) + q * P.nb + b0 + ob);
            static_cast<TS*>(P.out)[((long)q * P.na + a) * P.nb + b0 + ob] = (TS)sum;
        }
    }
}

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) dense_small_wgrad_kernel(const DenseSmallArgs P) {
    const int idx = blockIdx.x * WG_THREADS + threadIdx.x;
    if (idx >= P.ni * P.no) return;
    const int i = idx / P.no, o = idx - i * P.no;
    const TS* x = static_cast<const TS*>(P.a) + i;
    const TS* g = static_cast<const TS*>(P.b) + o;
    const long xcs = (long)P.n * P.ni, gcs = (long)P.n * P.no;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int n = 0; n < P.n; ++n) {
        float cx[4], gv[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float xv = ldf<TS>(x + c * xcs + (long)n * P.ni);
            cx[c] = c ? -xv : xv;  // conjugate
            gv[c] = ldf<TS>(g + c * gcs + (long)n * P.no);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += (qneg(p, q) ? -cx[p] : cx[p]) * gv[p ^ q];
    }
    TS* dw = static_cast<TS*>(P.out);
#pragma unroll
    for (int q = 0; q < 4; ++q) dw[q * P.wcs + o * P.so + i * P.si] = (TS)acc[q];
}

int launch_dense_small(bool half_storage, int pass, const DenseSmallArgs& a, hipStream_t st) {
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        const long threads = (long)a.ni * a.no;
        if (threads == 0) return 0;
        const dim3 grid((unsigned int)((threads + WG_THREADS - 1) / WG_THREADS)), block(WG_THREADS);
        if (half_storage) hipLaunchKernelGGL(dense_small_wgrad_kernel<_Float16>, grid, block, 0, st, a);
        else hipLaunchKernelGGL(dense_small_wgrad_kernel<float>, grid, block, 0, st, a);
        return 0;
    }
    const bool fwd = pass == PHX_PASS_FWD;
    DenseRowArgs r{a.a, a.b, fwd ? a.bias : nullptr, a.out, a.wcs, fwd ? a.si : a.so, fwd ? a.so : a.si,
                   a.n, fwd ? a.no : a.ni, fwd ? a.ni : a.no, 0};
    r.kfast = r.b_ks == 1 && r.b_bs != 1;
    const long blocks = (long)r.na * ((r.nb + 15) / 16);
    if (blocks == 0) return 0;
    if (blocks >= (1L << 31)) return -1;
    const dim3 grid((unsigned int)blocks), block(WG_THREADS);
    if (fwd) {
        if (half_storage) hipLaunchKernelGGL((dense_small_row_kernel<_Float16, false>), grid, block, 0, st, r);
        else hipLaunchKernelGGL((dense_small_row_kernel<float, false>), grid, block, 0, st, r);
    } else {
        if (half_storage) hipLaunchKernelGGL((dense_small_row_kernel<_Float16, true>), grid, block, 0, st, r);
        else hipLaunchKernelGGL((dense_small_row_kernel<float, true>), grid, block, 0, st, r);
    }
    return 0;
}

}  // namespace phx
