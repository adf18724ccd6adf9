// Conv2D and Dense of the reference's other algebras -- REAL, COMPLEX, GA_300 (src/algebras.hpp:17-22, sign
// tables src/algebras.cc:5-145) -- as compositions on the quaternion entry points.
//
// GA_300 has the blades 1, e1, e2, e3, e12, e13, e23, e123 (src/algebras.cc:58-131).  Its even part
// {1, e12, e13, -e23} multiplies like the quaternion units {1, i, j, k}; the pseudoscalar I = e123 commutes with
// every blade and squares to -1.  Every multivector is therefore M = A + I B with quaternion-like
// A = (m0, m4, m5, -m6), B = (m7, -m3, m2, m1), and
//     (A1 + I B1)(A2 + I B2) = (A1 A2 - B1 B2) + I (A1 B2 + B1 A2),
// i.e. a GA_300 convolution of Ci -> Co channels is one quaternion convolution of 2 Ci -> 2 Co channels on the
// activations [A | B] with the filter blocks [[A2, B2], [-B2, A2]] (input half x output half): 64 real products
// per multivector product, as many as the algebra's own table holds.
//
// COMPLEX and REAL are the sub-algebras {1, i} and {1} of the quaternions.  Embedding their tensors with zero
// components is correct but runs the full quaternion arithmetic on zeros (4x / 16x the products these algebras
// need); it remains the path for batches that cannot be paired.  With an even batch a COMPLEX problem is instead
// run as a quaternion problem on HALF the batch, in place: images A (first half) and B (second half) form
//     q = z_A + conj(z_B) j,      q (x) u = z_A u + conj(z_B u) j      for a complex filter u  (j u = conj(u) j),
// so one quaternion product yields both complex products, and the factorized 8-product form spends 4 real
// multiplications per complex product -- what a 2x2-block kernel of its own would.  The layout needs no copy: in
// the basis (1, j, i, -k) the coefficients of q are (re A, re B, im A, im B), which is how a complex tensor
// [re(0..N) | im(0..N)] lies in memory, and relabelling the units by i <-> j, k -> -k is an automorphism of the
// quaternions, so the kernels' (1, i, j, k) arithmetic on those coefficients computes the same product provided the
// filter is relabelled too: u = u0 + u1 i goes in as (u0, 0, u1, 0).  The output (z_A u, z_B u) comes out in the
// complex layout, the input gradient g (x) conj(u) likewise, and the complex filter gradient is the (1, i) part
// (components 0 and 2) of the quaternion one, conj(q) (x) g = conj(z_A) g_A + conj(z_B) g_B + (...) j.  A bias b
// enters as (b0, b0, b1, b1).  REAL: four images per quaternion, filter (w, 0, 0, 0), bias (b, b, b, b).
//
// The kernels here only rearrange (signed blade permutation, channel concatenation) into workspace buffers
// around one call of the quaternion path; the backward passes use the transposes of the same maps.
#include <algorithm>

#include "../../include/phx_qconv.h"
#include "phx_device.h"

namespace phx {

// quaternion component p of half h is sign * blade (blade < 0: zero)
struct BladeMap {
    int dims, halves;
    int blade[8], sign[8];  // [h * 4 + p]
    int slot[8];            // inverse: blade b sits in slot h * 4 + p
};

// the paired forms described at the top: filter map and bias map
static bool packed_maps(int algebra, BladeMap& filter, BladeMap& bias, int& images) {
    auto fill = [](BladeMap& m, int dims, const int (&blade)[4]) {
        m.dims = dims; m.halves = 1;
        for (int s = 0; s < 8; ++s) { m.blade[s] = s < 4 ? blade[s] : -1; m.sign[s] = (s < 4 && blade[s] >= 0) ? 1 : 0; m.slot[s] = -1; }
        for (int s = 3; s >= 0; --s)
            if (blade[s] >= 0) m.slot[blade[s]] = s;
    };
    if (algebra == PHX_COMPLEX) { fill(filter, 2, {0, -1, 1, -1}); fill(bias, 2, {0, 0, 1, 1}); images = 2; return true; }
    if (algebra == PHX_REAL) { fill(filter, 1, {0, -1, -1, -1}); fill(bias, 1, {0, 0, 0, 0}); images = 4; return true; }
    return false;
}

static bool blade_map(int algebra, BladeMap& m) {
    auto fill = [&](int dims, int halves, const int (&blade)[8], const int (&sign)[8]) {
        m.dims = dims; m.halves = halves;
        for (int s = 0; s < 8; ++s) { m.blade[s] = blade[s]; m.sign[s] = sign[s]; m.slot[s] = -1; }
        for (int s = 0; s < 4 * halves; ++s)
            if (blade[s] >= 0) m.slot[blade[s]] = s;
    };
    switch (algebra) {
        case PHX_REAL: fill(1, 1, {0, -1, -1, -1, -1, -1, -1, -1}, {1, 0, 0, 0, 0, 0, 0, 0}); return true;
        case PHX_COMPLEX: fill(2, 1, {0, 1, -1, -1, -1, -1, -1, -1}, {1, 1, 0, 0, 0, 0, 0, 0}); return true;
        case PHX_GA_300: fill(8, 2, {0, 4, 5, 6, 7, 3, 2, 1}, {1, 1, 1, -1, 1, -1, 1, 1}); return true;
        default: return false;
    }
}

struct BladeArgs {
    const void* src;
    void* dst;
    BladeMap m;
    long n;   // images (bias: 1)
    int C;    // channels of the algebra's tensor
    long hw;  // positions per plane
};

// 16 bytes of one plane, sign applied (rows start at element alignment only, which 16-byte accesses tolerate)
template <typename TS>
__device__ __forceinline__ void copy_signed16(const TS* src, TS* dst, int sign) {
    constexpr int V = 16 / sizeof(TS);
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (src) raw = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a2*>((const __attribute__((address_space(1))) TS*)src);
    if (sign < 0) {
        const unsigned int flip = sizeof(TS) == 2 ? 0x80008000u : 0x80000000u;
        raw = raw ^ u32x4{flip, flip, flip, flip};
    }
    (void)V;
    *reinterpret_cast<__attribute__((address_space(1))) u32x4_a2*>((__attribute__((address_space(1))) TS*)dst) = raw;
}

// algebra tensor [dims][n][C][hw] -> quaternion tensor [4][n][halves * C][hw].  For a given blade and image the
// C * hw elements are contiguous on both sides, so a thread moves V consecutive elements of such a block
// (V = 16 bytes when C * hw allows, else 1).
template <typename TS, int V>
__global__ void __launch_bounds__(WG_THREADS) blade_gather_kernel(const BladeArgs A) {
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const long chw = (long)A.C * A.hw, per = chw / V;
    const int H = A.m.halves;
    const long total = 4 * A.n * H * per;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long e = (idx % per) * V;
        long r = idx / per;
        const int h = (int)(r % H);
        r /= H;
        const long nn = r % A.n;
        const int p = (int)(r / A.n);
        const int b = A.m.blade[h * 4 + p], sg = A.m.sign[h * 4 + p];
        const TS* s = b >= 0 ? src + ((long)b * A.n + nn) * chw + e : nullptr;
        TS* d = dst + (((long)p * A.n + nn) * H + h) * chw + e;
        if constexpr (V > 1) copy_signed16<TS>(s, d, sg);
        else *d = s ? (TS)((float)sg * (float)*s) : (TS)0.f;
    }
}

// quaternion tensor [4][n][halves * C][hw] -> algebra tensor [dims][n][C][hw]
template <typename TS, int V>
__global__ void __launch_bounds__(WG_THREADS) blade_scatter_kernel(const BladeArgs A) {
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const long chw = (long)A.C * A.hw, per = chw / V;
    const int H = A.m.halves;
    const long total = (long)A.m.dims * A.n * per;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long e = (idx % per) * V;
        long r = idx / per;
        const long nn = r % A.n;
        const int b = (int)(r / A.n);
        const int sl = A.m.slot[b], h = sl >> 2, p = sl & 3;
        const TS* s = src + (((long)p * A.n + nn) * H + h) * chw + e;
        TS* d = dst + ((long)b * A.n + nn) * chw + e;
        if constexpr (V > 1) copy_signed16<TS>(s, d, A.m.sign[sl]);
        else *d = (TS)((float)A.m.sign[sl] * (float)*s);
    }
}

// The same two maps for channels-last tensors, [dims][n][hw][C] <-> [4][n][hw][halves * C] (and channel groups, see
// Composition): the channel axis is the contiguous one and the halves interleave along it, so these go element by
// element.  A.C is the channel count per group here, A.G the number of groups.
struct BladeLastArgs {
    const void* src;
    void* dst;
    BladeMap m;
    long n, hw;
    int Cg, G;
};

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) blade_gather_last_kernel(const BladeLastArgs A) {
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const int H = A.m.halves;
    const long C = (long)A.Cg * A.G, C2 = C * H;
    const long total = 4 * A.n * A.hw * C2;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long c2 = idx % C2;
        long r = idx / C2;
        const long pos = r % A.hw;
        r /= A.hw;
        const long nn = r % A.n;
        const int p = (int)(r / A.n);
        const int g = (int)(c2 / ((long)H * A.Cg)), h = (int)((c2 / A.Cg) % H), cin = (int)(c2 % A.Cg);
        const int b = A.m.blade[h * 4 + p], sg = A.m.sign[h * 4 + p];
        float v = 0.f;
        if (b >= 0) v = (float)sg * (float)src[(((long)b * A.n + nn) * A.hw + pos) * C + (long)g * A.Cg + cin];
        dst[idx] = (TS)v;
    }
}

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) blade_scatter_last_kernel(const BladeLastArgs A) {
    const TS* src = static_cast<const TS*>(A.src);
    TS* dst = static_cast<TS*>(A.dst);
    const int H = A.m.halves;
    const long C = (long)A.Cg * A.G, C2 = C * H;
    const long total = (long)A.m.dims * A.n * A.hw * C;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long c = idx % C;
        long r = idx / C;
        const long pos = r % A.hw;
        r /= A.hw;
        const long nn = r % A.n;
        const int b = (int)(r / A.n);
        const int sl = A.m.slot[b], h = sl >> 2, p = sl & 3;
        const long g = c / A.Cg, cin = c % A.Cg;
        const long c2 = (g * H + h) * A.Cg + cin;
        dst[idx] = (TS)((float)A.m.sign[sl] * (float)src[(((long)p * A.n + nn) * A.hw + pos) * C2 + c2]);
    }
}

struct BladeFilterArgs {
    const void* w;   // algebra filter (forward: read; fold: written)
    void* q;         // quaternion filter with halves * Co x halves * Cig channels
    BladeMap m;
    int Co, Cog, Cig, taps;    // output channels in all and per group, input channels per group (the filter's own axis)
    long wcs, wso, wsi, wst;   // algebra filter: elements between blades, output channels, input channels, taps
    long qcs, qso, qsi, qst;   // the same for the quaternion filter
};

// filter blocks (input half x output half): [[A, B], [-B, A]]; with channel groups, group g of the quaternion
// problem holds the two halves of the algebra's group g side by side: output channel (g * halves + ho) * Cog + o
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) blade_filter_build_kernel(const BladeFilterArgs A) {
    const TS* w = static_cast<const TS*>(A.w);
    TS* q = static_cast<TS*>(A.q);
    const int H = A.m.halves;
    const long HO = (long)H * A.Co, HI = (long)H * A.Cig;
    const long total = 4 * HO * HI * A.taps;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int tap = (int)(idx % A.taps);
        long r = idx / A.taps;
        const int i2 = (int)(r % HI);
        r /= HI;
        const int o2 = (int)(r % HO);
        const int p = (int)(r / HO);
        const int g = o2 / (H * A.Cog), ho = (o2 / A.Cog) % H, o = g * A.Cog + o2 % A.Cog;
        const int hi = i2 / A.Cig, i = i2 - hi * A.Cig;
        const int part = (ho != hi) ? 1 : 0;
        const float block_sign = (ho == 0 && hi == 1) ? -1.f : 1.f;
        const int s = part * 4 + p, b = A.m.blade[s];
        float v = 0.f;
        if (b >= 0) v = block_sign * (float)A.m.sign[s] * (float)w[b * A.wcs + o * A.wso + i * A.wsi + tap * A.wst];
        q[p * A.qcs + o2 * A.qso + i2 * A.qsi + tap * A.qst] = (TS)v;
    }
}

// transpose of the build: gradient of the quaternion filter -> gradient of the algebra filter
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) blade_filter_fold_kernel(const BladeFilterArgs A) {
    TS* w = static_cast<TS*>(const_cast<void*>(A.w));
    const TS* q = static_cast<const TS*>(A.q);
    const int H = A.m.halves;
    const long total = (long)A.m.dims * A.Co * A.Cig * A.taps;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int tap = (int)(idx % A.taps);
        long r = idx / A.taps;
        const int i = (int)(r % A.Cig);
        r /= A.Cig;
        const int o = (int)(r % A.Co);
        const int b = (int)(r / A.Co);
        const int s = A.m.slot[b], part = s >> 2, p = s & 3;
        const int g = o / A.Cog, oin = o - g * A.Cog;
        auto at = [&](int ho, int hi) {
            return (float)q[p * A.qcs + (long)((g * H + ho) * A.Cog + oin) * A.qso + (long)(hi * A.Cig + i) * A.qsi + tap * A.qst];
        };
        float v;
        if (H == 1) v = at(0, 0);
        else if (part == 0) v = at(0, 0) + at(1, 1);
        else v = at(1, 0) - at(0, 1);
        w[b * A.wcs + o * A.wso + i * A.wsi + tap * A.wst] = (TS)((float)A.m.sign[s] * v);
    }
}

static int blocks_for(long items) { return (int)std::max<long>(1, std::min<long>((items + WG_THREADS - 1) / WG_THREADS, 1 << 16)); }

template <typename K32, typename K16, typename Args>
static void launch(bool half_storage, K32 k32, K16 k16, long items, const Args& a, hipStream_t st) {
    if (items <= 0) return;
    if (half_storage) hipLaunchKernelGGL(k16, dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL(k32, dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
}

static size_t align256(size_t b) { return (b + 255) / 256 * 256; }

// Buffers of one composed call at the front of the workspace: quaternion forms of the input-side tensor, the
// output-side tensor, the filter and the bias; the quaternion call's own workspace follows.
// Filter element strides (output channel, input channel, tap) of a layout with the given extents
struct FilterStep { long so, si, st; };
static FilterStep conv_filter_step(int layout, long O, long I, long taps) {
    if (layout == PHX_OHWI) return {taps * I, 1, I};
    if (layout == PHX_HWIO) return {1, O, I * O};
    return {I * taps, taps, 1};  // OIHW
}

struct Composition {
    BladeMap m;
    BladeMap bias_map;  // paired form only
    bool packed = false;  // paired form: activations in place, `m` maps the filter
    bool half;
    bool nhwc = false;    // channels-last activations
    int groups = 1;
    int layout = PHX_OIHW;  // filter layout (Dense: phx_dense_layout, see filter_args)
    size_t esize, x_bytes, y_bytes, w_bytes, b_bytes;
    long n;
    int ci, co, taps;
    long hw_in, hw_out;
    size_t buffers() const { return x_bytes + y_bytes + w_bytes + b_bytes; }
    void init(int dtype, long n_, int ci_, int co_, long hw_in_, long hw_out_, int taps_) {
        half = dtype == PHX_F16; esize = half ? 2 : 4;
        n = n_; ci = ci_; co = co_; hw_in = hw_in_; hw_out = hw_out_; taps = taps_;
        const size_t H = m.halves;
        x_bytes = packed ? 0 : align256(4 * n * H * ci * hw_in * esize);
        y_bytes = packed ? 0 : align256(4 * n * H * co * hw_out * esize);
        w_bytes = align256(4 * H * co * H * (ci / groups) * taps * esize);
        b_bytes = align256(4 * H * co * esize);
    }
    // Activations [blade][rows][C][hw] (or [blade][rows][hw][C], channels-last) -> quaternion form.  With channel
    // groups the two halves interleave per group, [g][half][C / groups]: in the channels-first layout that is the
    // ungrouped map on rows * groups "images" of C / groups channels.
    void gather(const void* src, void* dst, long rows, int C, long hw, hipStream_t st, const BladeMap* map = nullptr,
                bool grouped = true) const {
        const int G = grouped ? groups : 1;
        if (nhwc && hw > 1) {
            BladeLastArgs a{src, dst, map ? *map : m, rows, hw, C / G, G};
            launch(half, blade_gather_last_kernel<float>, blade_gather_last_kernel<_Float16>, 4 * rows * hw * m.halves * C, a, st);
            return;
        }
        rows *= G; C /= G;
        BladeArgs a{src, dst, map ? *map : m, rows, C, hw};
        const int V = half ? 8 : 4;
        const long blocks = 4 * rows * m.halves, chw = C * hw;
        if (chw % V == 0) launch(half, blade_gather_kernel<float, 4>, blade_gather_kernel<_Float16, 8>, blocks * (chw / V), a, st);
        else launch(half, blade_gather_kernel<float, 1>, blade_gather_kernel<_Float16, 1>, blocks * chw, a, st);
    }
    void scatter(const void* src, void* dst, long rows, int C, long hw, hipStream_t st) const {
        if (nhwc && hw > 1) {
            BladeLastArgs a{src, dst, m, rows, hw, C / groups, groups};
            launch(half, blade_scatter_last_kernel<float>, blade_scatter_last_kernel<_Float16>, (long)m.dims * rows * hw * C, a, st);
            return;
        }
        rows *= groups; C /= groups;
        BladeArgs a{src, dst, m, rows, C, hw};
        const int V = half ? 8 : 4;
        const long blocks = (long)m.dims * rows, chw = C * hw;
        if (chw % V == 0) launch(half, blade_scatter_kernel<float, 4>, blade_scatter_kernel<_Float16, 8>, blocks * (chw / V), a, st);
        else launch(half, blade_scatter_kernel<float, 1>, blade_scatter_kernel<_Float16, 1>, blocks * chw, a, st);
    }
    // dense filters are [blade][in][out] (IO) or [blade][out][in] (OI), convolution filters [blade] x the layout's axes;
    // the quaternion filter is built in the same layout with halves * the channel counts
    BladeFilterArgs filter_args(const void* w, void* q, bool dense) const {
        BladeFilterArgs a;
        a.w = w; a.q = q; a.m = m; a.Co = co; a.Cog = co / groups; a.Cig = ci / groups; a.taps = taps;
        const long H = m.halves, O = co, I = ci / groups;
        a.wcs = O * I * taps; a.qcs = H * O * H * I * taps;
        FilterStep ws, qs;
        if (dense) {
            ws = layout == PHX_OI ? FilterStep{I, 1, 1} : FilterStep{1, O, 1};
            qs = layout == PHX_OI ? FilterStep{H * I, 1, 1} : FilterStep{1, H * O, 1};
        } else {
            ws = conv_filter_step(layout, O, I, taps);
            qs = conv_filter_step(layout, H * O, H * I, taps);
        }
        a.wso = ws.so; a.wsi = ws.si; a.wst = ws.st;
        a.qso = qs.so; a.qsi = qs.si; a.qst = qs.st;
        return a;
    }
    void build_filter(const void* w, void* q, bool dense, hipStream_t st) const {
        launch(half, blade_filter_build_kernel<float>, blade_filter_build_kernel<_Float16>,
               4L * m.halves * co * m.halves * (ci / groups) * taps, filter_args(w, q, dense), st);
    }
    void fold_filter(const void* q, void* w, bool dense, hipStream_t st) const {
        launch(half, blade_filter_fold_kernel<float>, blade_filter_fold_kernel<_Float16>, (long)m.dims * co * (ci / groups) * taps,
               filter_args(w, const_cast<void*>(q), dense), st);
    }
};

static int conv_composition(const phx_qconv_desc* d, Composition& c, phx_qconv_desc& inner) {
    if (!d || !blade_map(d->algebra, c.m)) return PHX_ERR_INVALID_ARGUMENT;
    // (the reference's generic path is algebra-agnostic in layouts and groups, src/conv2d.hpp:237-275; a real-valued
    // input is taken by the quaternion algebra only here)
    if (d->real_input) return PHX_ERR_NOT_SUPPORTED;
    const int groups = d->groups > 1 ? d->groups : 1;
    if (d->ci % groups || d->co % groups) return PHX_ERR_INVALID_ARGUMENT;
    c.groups = groups; c.layout = d->filter_layout; c.nhwc = d->data_format == PHX_NHWC;
    inner = *d;
    inner.algebra = PHX_QUATERNION;
    int images = 1;
    BladeMap fm, bm;
    if (packed_maps(d->algebra, fm, bm, images) && d->n > 0 && d->n % images == 0) {
        c.packed = true; c.m = fm; c.bias_map = bm;
        inner.n = d->n / images;
    }
    inner.ci = d->ci * c.m.halves;
    inner.co = d->co * c.m.halves;
    int32_t ho = 0, wo = 0;
    const int rc = phx_qconv2d_output_hw(&inner, &ho, &wo);
    if (rc != PHX_OK) return rc;
    c.init(d->dtype, inner.n, d->ci, d->co, (long)d->h * d->w, (long)ho * wo, d->kh * d->kw);
    return PHX_OK;
}

static int dense_composition(const phx_qdense_desc* d, Composition& c, phx_qdense_desc& inner) {
    if (!d || !blade_map(d->algebra, c.m)) return PHX_ERR_INVALID_ARGUMENT;
    c.layout = d->filter_layout;
    if (d->n < 0 || d->ni <= 0 || d->no <= 0 || (d->dtype != PHX_F32 && d->dtype != PHX_F16)) return PHX_ERR_INVALID_ARGUMENT;
    inner = *d;
    inner.algebra = PHX_QUATERNION;
    int images = 1;
    BladeMap fm, bm;
    if (packed_maps(d->algebra, fm, bm, images) && d->n > 0 && d->n % images == 0) {
        c.packed = true; c.m = fm; c.bias_map = bm;
        inner.n = d->n / images;
    }
    inner.ni = d->ni * c.m.halves;
    inner.no = d->no * c.m.halves;
    c.init(d->dtype, inner.n, d->ni, d->no, 1, 1, 1);
    return PHX_OK;
}

// One composed pass.  `pass` picks which tensors are rearranged in and out; `run` is the quaternion call on the
// buffers (x, y, w, bias, inner workspace).
template <typename Run>
static int composed_pass(const Composition& c, int pass, bool dense, hipStream_t st, const void* a, const void* b,
                         const void* bias, void* out, void* ws, size_t ws_bytes, Run run) {
    if (ws_bytes < c.buffers() || !ws) return PHX_ERR_WORKSPACE;
    char* base = static_cast<char*>(ws);
    void* xq = base;
    void* yq = base + c.x_bytes;
    void* wq = base + c.x_bytes + c.y_bytes;
    void* bq = base + c.x_bytes + c.y_bytes + c.w_bytes;
    void* inner_ws = base + c.buffers();
    const size_t inner_bytes = ws_bytes - c.buffers();
    int rc;
    if (c.packed) {  // activations and gradients are used where they lie
        if (pass == PHX_PASS_FWD) {
            c.build_filter(b, wq, dense, st);
            if (bias) c.gather(bias, bq, 1, c.co, 1, st, &c.bias_map);
            rc = run(a, wq, bias ? bq : nullptr, out, inner_ws, inner_bytes);
        } else if (pass == PHX_PASS_BWD_DATA) {
            c.build_filter(b, wq, dense, st);
            rc = run(a, wq, nullptr, out, inner_ws, inner_bytes);
        } else {
            rc = run(a, b, nullptr, wq, inner_ws, inner_bytes);
            if (rc == PHX_OK) c.fold_filter(wq, out, dense, st);
        }
    } else if (pass == PHX_PASS_FWD) {  // a = x, b = w
        c.gather(a, xq, c.n, c.ci, c.hw_in, st);
        c.build_filter(b, wq, dense, st);
        if (bias) c.gather(bias, bq, 1, c.co, 1, st);
        rc = run(xq, wq, bias ? bq : nullptr, yq, inner_ws, inner_bytes);
        if (rc == PHX_OK) c.scatter(yq, out, c.n, c.co, c.hw_out, st);
    } else if (pass == PHX_PASS_BWD_DATA) {  // a = grad, b = w
        c.gather(a, yq, c.n, c.co, c.hw_out, st);
        c.build_filter(b, wq, dense, st);
        rc = run(yq, wq, nullptr, xq, inner_ws, inner_bytes);
        if (rc == PHX_OK) c.scatter(xq, out, c.n, c.ci, c.hw_in, st);
    } else {  // a = x, b = grad
        c.gather(a, xq, c.n, c.ci, c.hw_in, st);
        c.gather(b, yq, c.n, c.co, c.hw_out, st);
        rc = run(xq, yq, nullptr, wq, inner_ws, inner_bytes);
        if (rc == PHX_OK) c.fold_filter(wq, out, dense, st);
    }
    if (rc != PHX_OK) return rc;
    return hipGetLastError() == hipSuccess ? PHX_OK : PHX_ERR_RUNTIME;
}

size_t algebra_conv_workspace_bytes(const phx_qconv_desc* d, int pass) {
    Composition c;
    phx_qconv_desc inner;
    if (conv_composition(d, c, inner) != PHX_OK) return 0;
    return c.buffers() + phx_qconv2d_workspace_bytes(&inner, pass);
}

size_t algebra_dense_workspace_bytes(const phx_qdense_desc* d, int pass) {
    Composition c;
    phx_qdense_desc inner;
    if (dense_composition(d, c, inner) != PHX_OK) return 0;
    return c.buffers() + phx_qdense_workspace_bytes(&inner, pass);
}

int algebra_conv_pass(const phx_qconv_desc* d, int pass, phx_stream_t stream, const void* a, const void* b, const void* bias,
                      void* out, void* ws, size_t ws_bytes) {
    Composition c;
    phx_qconv_desc inner;
    const int rc = conv_composition(d, c, inner);
    if (rc != PHX_OK) return rc;
    if (pass == PHX_PASS_FWD && d->has_bias && !bias) return PHX_ERR_INVALID_ARGUMENT;
    if (pass != PHX_PASS_FWD || !d->has_bias) bias = nullptr;
    return composed_pass(c, pass, false, static_cast<hipStream_t>(stream), a, b, bias, out, ws, ws_bytes,
                         [&](const void* p0, const void* p1, const void* pb, void* po, void* iw, size_t ib) {
                             if (pass == PHX_PASS_FWD) return phx_qconv2d_fwd(&inner, stream, p0, p1, pb, po, iw, ib);
                             if (pass == PHX_PASS_BWD_DATA) return phx_qconv2d_bwd_data(&inner, stream, p0, p1, po, iw, ib);
                             return phx_qconv2d_bwd_weights(&inner, stream, p0, p1, po, iw, ib);
                         });
}

int algebra_dense_pass(const phx_qdense_desc* d, int pass, phx_stream_t stream, const void* a, const void* b, const void* bias,
                       void* out, void* ws, size_t ws_bytes) {
    Composition c;
    phx_qdense_desc inner;
    const int rc = dense_composition(d, c, inner);
    if (rc != PHX_OK) return rc;
    if (pass == PHX_PASS_FWD && d->has_bias && !bias) return PHX_ERR_INVALID_ARGUMENT;
    if (pass != PHX_PASS_FWD || !d->has_bias) bias = nullptr;
    return composed_pass(c, pass, true, static_cast<hipStream_t>(stream), a, b, bias, out, ws, ws_bytes,
                         [&](const void* p0, const void* p1, const void* pb, void* po, void* iw, size_t ib) {
                             if (pass == PHX_PASS_FWD) return phx_qdense_fwd(&inner, stream, p0, p1, pb, po, iw, ib);
                             if (pass == PHX_PASS_BWD_DATA) return phx_qdense_bwd_data(&inner, stream, p0, p1, po, iw, ib);
                             return phx_qdense_bwd_weights(&inner, stream, p0, p1, po, iw, ib);
                         });
}

}  // namespace phx

extern "C" int phx_algebra_map(int algebra, int32_t* dims, int32_t* halves, int32_t* blade, int32_t* sign) {
    phx::BladeMap m;
    if (algebra == PHX_QUATERNION) {
        if (dims) *dims = 4;
        if (halves) *halves = 1;
        for (int s = 0; s < 8; ++s) {
            if (blade) blade[s] = s < 4 ? s : -1;
            if (sign) sign[s] = s < 4 ? 1 : 0;
        }
        return PHX_OK;
    }
    if (!phx::blade_map(algebra, m)) return PHX_ERR_INVALID_ARGUMENT;
    if (dims) *dims = m.dims;
    if (halves) *halves = m.halves;
    for (int s = 0; s < 8; ++s) {
        if (blade) blade[s] = m.blade[s];
        if (sign) sign[s] = m.sign[s];
    }
    return PHX_OK;
}
