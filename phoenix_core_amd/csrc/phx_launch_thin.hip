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

#include <algorithm>
#include <type_traits>

namespace phx {

// Forward and input gradient: grid row = one channel of the written tensor, so the filter entries a workgroup needs
// (other-side channels of the group x taps, four components each) are the same for all its threads and sit in LDS;
// consecutive threads take consecutive pixels of a row, i.e. consecutive addresses of every plane they read.
template <typename TS, bool DGRAD>
__global__ void __launch_bounds__(WG_THREADS) qconv_thin_kernel(const ThinArgs P) {
    extern __shared__ float4 thin_filter[];  // [other-side channel of the chunk][tap]
    const int taps = P.Kh * P.Kw;
    const int c = blockIdx.y;  // channel of the written tensor, over all groups
    const int cside = DGRAD ? P.cig : P.cog, K = DGRAD ? P.cog : P.cig;
    const int g = c / cside, c_in_group = c - g * cside;
    const TS* W = static_cast<const TS*>(P.w);
    const int Hin = DGRAD ? P.Ho : P.H, Win = DGRAD ? P.Wo : P.W;    // the tensor read
    const int Hout = DGRAD ? P.H : P.Ho, Wout = DGRAD ? P.W : P.Wo;  // the tensor written
    const long opix = (long)Hout * Wout, ipix = (long)Hin * Win;
    const long idx_all = (long)blockIdx.x * WG_THREADS + threadIdx.x;
    const bool live = idx_all < P.N * opix;
    const long idx = live ? idx_all : 0;  // (a thread past the end computes the first output again and stores nothing)
    const int n = (int)(idx / opix), rem = (int)(idx - n * opix);
    const int oh = rem / Wout, ow = rem - oh * Wout;
    const long Cin_all = (long)P.groups * K, Cout_all = (long)P.groups * cside;
    // (real-valued input: one stored component; the loads of the absent ones go to the stored one and count as zero)
    const bool real_x = !DGRAD && P.real_x;
    const long in_cs = real_x ? 0 : P.N * Cin_all * ipix, out_cs = P.N * Cout_all * opix;
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
            v[p] = (ok && !(p && real_x)) ? f : 0.f;
        }
        const float4 w4 = thin_filter[e];
        const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += (qneg(p, q) ? -v[p] : v[p]) * wv[p ^ q];
    };
    // exact division by multiplication: m = ceil(2^32 / s) (0: s == 1)
    const auto divide = [](int t, int s, unsigned int m, int& quotient) {
        quotient = m ? (int)__umulhi((unsigned int)t, m) : t;
        return t >= 0 && quotient * s == t;
    };
    // the other side's channels go through LDS in chunks of P.kchunk filters (all of them at once for thin groups)
    for (int k0 = 0; k0 < K; k0 += P.kchunk) {
        const int kn = K - k0 < P.kchunk ? K - k0 : P.kchunk;
        if (k0) __syncthreads();  // (everyone has read the previous chunk)
        for (int e = threadIdx.x; e < kn * taps; e += WG_THREADS) {
            const int k = e / taps, t = e - k * taps, kh = t / P.Kw, kw = t - kh * P.Kw;
            const long co = DGRAD ? g * P.cog + k0 + k : c, ci = DGRAD ? c_in_group : k0 + k;
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
        if (!DGRAD || (P.sh == 1 && P.sw == 1)) {
            // no branches around the loads: a tap outside the image reads the plane's first element and counts as zero,
            // so the loads of several taps are in flight together
            for (int k = 0; k < kn; ++k, in += ipix) {
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
            // ((h + pt - kh dh) / sh, (w + pl - kw dw) / sw) where both divisions leave no remainder; one entry in
            // sh * sw does, the others are skipped
            for (int k = 0; k < kn; ++k, in += ipix) {
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
    }
    if (!live) return;
    TS* out = static_cast<TS*>(P.out) + (n * Cout_all + c) * opix + rem;
#pragma unroll
    for (int q = 0; q < 4; ++q) out[q * out_cs] = (TS)acc[q];
}

// ---- the same two passes from a window tile in LDS ----
// Forward (any stride and dilation) and the unit-stride input gradient where an output row is at most 1024 wide: a
// workgroup writes R rows of J images of one channel (J > 1 only where a whole image is less than its 1024 outputs)
// and first copies the window of those rows -- every element once, zeros where the window leaves the image -- into
// LDS, four components side by side per position.  A tap is then one LDS read per output (and one broadcast read of
// the filter entry per four outputs) with no address arithmetic beyond an add, against four global loads before.
// fp16 tensors keep their halves in LDS, paired (x0,x1) (x2,x3), and the filter entry as the eight pairs
// (s(0,q) w[q], s(1,q) w[1^q]), (s(2,q) w[2^q], s(3,q) w[3^q]): a tap is eight v_dot2_f32_f16 -- two products and
// their sum into an fp32 accumulator each -- instead of sixteen FMAs and four conversions.
typedef _Float16 thin_half2 __attribute__((ext_vector_type(2)));

template <typename TS>
struct ThinTile;
template <>
struct ThinTile<float> {
    using Entry = float4;
    using Filter = float4;
    static __device__ __forceinline__ Entry entry(const float v[4]) { return make_float4(v[0], v[1], v[2], v[3]); }
    static __device__ __forceinline__ Filter filter(const float w[4]) { return make_float4(w[0], w[1], w[2], w[3]); }
    static __device__ __forceinline__ void mac(float acc[4], const Entry& x, const Filter& f) {
        const float v[4] = {x.x, x.y, x.z, x.w}, wv[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += (qneg(p, q) ? -v[p] : v[p]) * wv[p ^ q];
    }
};
template <>
struct ThinTile<_Float16> {
    struct __align__(8) Entry { thin_half2 lo, hi; };
    struct __align__(16) Filter { thin_half2 lo[4], hi[4]; };
    static __device__ __forceinline__ Entry entry(const float v[4]) {
        Entry e;
        e.lo = thin_half2{(_Float16)v[0], (_Float16)v[1]};  // (values that came from halves: exact)
        e.hi = thin_half2{(_Float16)v[2], (_Float16)v[3]};
        return e;
    }
    static __device__ __forceinline__ Filter filter(const float w[4]) {
        Filter f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            f.lo[q] = thin_half2{(_Float16)(qneg(0, q) ? -w[q] : w[q]), (_Float16)(qneg(1, q) ? -w[1 ^ q] : w[1 ^ q])};
            f.hi[q] = thin_half2{(_Float16)(qneg(2, q) ? -w[2 ^ q] : w[2 ^ q]), (_Float16)(qneg(3, q) ? -w[3 ^ q] : w[3 ^ q])};
        }
        return f;
    }
    static __device__ __forceinline__ void mac(float acc[4], const Entry& x, const Filter& f) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc[q] = __builtin_amdgcn_fdot2(x.lo, f.lo[q], acc[q], false);
            acc[q] = __builtin_amdgcn_fdot2(x.hi, f.hi[q], acc[q], false);
        }
    }
};

constexpr int THIN_TILE_THREADS = 256;  // workgroup of the forward / unit-stride input-gradient tile kernel (64 / 128 measured 10-25 % slower at 3x3)
constexpr int THIN_PXT = 4;                          // outputs per thread
constexpr int THIN_TILE_PIXELS = THIN_PXT * THIN_TILE_THREADS;
constexpr size_t THIN_TILE_LDS = 64 * 1024;
constexpr size_t THIN_FILTER_LDS = 32 * 1024;  // the per-tap kernel's filter chunk

__device__ __forceinline__ int thin_div(int t, const ThinDiv& d) { return (int)(__umulhi((unsigned int)t, d.m) + ((unsigned int)t & d.one)); }

// Loads and stores of the tiled kernels: buffer instructions, i.e. a base that is the same for the whole workgroup
// (scalar registers) + a 32-bit byte offset per lane, so that the lanes do no 64-bit address arithmetic; an offset of
// ~0 is out of the buffer's range and reads as zero (how positions outside the image are skipped).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t thin_buffer(const void* base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}
constexpr unsigned int THIN_NOWHERE = ~0u;
template <typename TS>
__device__ __forceinline__ float thin_load(__amdgpu_buffer_rsrc_t buffer, unsigned int bytes);
template <>
__device__ __forceinline__ float thin_load<_Float16>(__amdgpu_buffer_rsrc_t buffer, unsigned int bytes) {
    return (float)__builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(buffer, bytes, 0, 0));
}
template <>
__device__ __forceinline__ float thin_load<float>(__amdgpu_buffer_rsrc_t buffer, unsigned int bytes) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(buffer, bytes, 0, 0));
}
__device__ __forceinline__ void thin_store(__amdgpu_buffer_rsrc_t buffer, unsigned int bytes, _Float16 v) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), buffer, bytes, 0, 0);
}
__device__ __forceinline__ void thin_store(__amdgpu_buffer_rsrc_t buffer, unsigned int bytes, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), buffer, bytes, 0, 0);
}

// body(integral_constant<N>) for N == slots, 0 <= slots <= MAX
template <int MAX, typename Body>
__device__ __forceinline__ void thin_dispatch_slots(int slots, const Body& body) {
    if constexpr (MAX == 0) {
        body(std::integral_constant<int, 0>());
    } else {
        if (slots >= MAX) body(std::integral_constant<int, MAX>());
        else thin_dispatch_slots<MAX - 1>(slots, body);
    }
}

template <typename TS, bool DGRAD>
__global__ void __launch_bounds__(THIN_TILE_THREADS) qconv_thin_tile_kernel(const ThinArgs P) {
    using T = ThinTile<TS>;
    using Entry = typename T::Entry;
    using Filter = typename T::Filter;
    extern __shared__ __align__(16) unsigned char thin_lds[];
    const int taps = P.Kh * P.Kw;
    const int c = blockIdx.y;  // channel of the written tensor, over all groups
    const int cside = DGRAD ? P.cig : P.cog, K = DGRAD ? P.cog : P.cig;
    const int g = c / cside, c_in_group = c - g * cside;
    Filter* filt = reinterpret_cast<Filter*>(thin_lds);                          // [other-side channel][tap]
    Entry* tile = reinterpret_cast<Entry*>(thin_lds + (size_t)K * taps * sizeof(Filter));  // [image][window row][window column]
    const TS* W = static_cast<const TS*>(P.w);
    for (int e = threadIdx.x; e < K * taps; e += THIN_TILE_THREADS) {
        const int k = e / taps, t = e - k * taps, kh = t / P.Kw, kw = t - kh * P.Kw;
        const long co = DGRAD ? g * P.cog + k : c, ci = DGRAD ? c_in_group : k;
        const TS* at = W + co * P.so + ci * P.si + kh * P.skh + kw * P.skw;
        float w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = ldf<TS>(at + r * P.wcs);
            w[r] = (DGRAD && r) ? -v : v;  // conjugate
        }
        filt[e] = T::filter(w);
    }
    const int Hin = DGRAD ? P.Ho : P.H, Win = DGRAD ? P.Wo : P.W;    // the tensor read
    const int Hout = DGRAD ? P.H : P.Ho, Wout = DGRAD ? P.W : P.Wo;  // the tensor written
    const int rstep = DGRAD ? 1 : P.sh, cstep = DGRAD ? 1 : P.sw;    // window rows / columns per output row / column
    const long opix = (long)Hout * Wout, ipix = (long)Hin * Win;
    const long Cin_all = (long)P.groups * K, Cout_all = (long)P.groups * cside;
    const bool real_x = !DGRAD && P.real_x;  // real-valued input: one stored component, the others read as zero
    const long in_cs = real_x ? 0 : P.N * Cin_all * ipix, out_cs = P.N * Cout_all * opix;
    const int ng = blockIdx.x / P.tile_bands, band = blockIdx.x - ng * P.tile_bands;
    const int n0 = ng * P.tile_J, r0 = band * P.tile_R;
    // the tile's first row and column in the tensor read
    const int ih0 = DGRAD ? r0 + P.pt - (P.Kh - 1) * P.dh : r0 * P.sh - P.pt;
    const int iw0 = DGRAD ? P.pl - (P.Kw - 1) * P.dw : -P.pl;
    const int entries = P.tile_J * P.tile_rows * P.tile_cols;
    const int image_in = (int)(Cin_all * ipix), image_out = (int)(Cout_all * opix);  // elements from an image to the next

    // this thread's outputs: numbers tid, tid + 256, .. of the workgroup's J x R x Wout
    int tbase[THIN_PXT];
    unsigned int oaddr[THIN_PXT];  // (32-bit offsets from bases that are the same for the whole workgroup: see thin_tile_plan)
    bool live[THIN_PXT];
    float acc[THIN_PXT][4];
#pragma unroll
    for (int s = 0; s < THIN_PXT; ++s) {
        const int pix = threadIdx.x + s * THIN_TILE_THREADS;
        const int prow = thin_div(pix, P.d_wout), ow = pix - prow * Wout;
        const int j = thin_div(prow, P.d_R), r = prow - j * P.tile_R;
        live[s] = j < P.tile_J && n0 + j < P.N && r0 + r < Hout;
        tbase[s] = live[s] ? (j * P.tile_rows + r * rstep) * P.tile_cols + ow * cstep : 0;
        oaddr[s] = (unsigned int)(j * image_out + r * Wout + ow);
#pragma unroll
        for (int q = 0; q < 4; ++q)
            acc[s][q] = (!DGRAD && P.bias) ? ldf<TS>(static_cast<const TS*>(P.bias) + q * Cout_all + c) : 0.f;
    }
    // outputs in flight per wave: whole slots of 256 beyond the workgroup's last output are skipped by the waves they
    // would leave idle (784 outputs of a 28 x 28 image: the fourth slot is run by the first wave alone)
    const int wave_first = __builtin_amdgcn_readfirstlane(threadIdx.x & ~63);
    const int total = P.tile_J * P.tile_R * Wout;
    const int wave_slots = total <= wave_first ? 0 : std::min(THIN_PXT, (total - wave_first + THIN_TILE_THREADS - 1) / THIN_TILE_THREADS);

    const TS* in = static_cast<const TS*>(P.in) + ((long)n0 * Cin_all + (long)g * K) * ipix;
    for (int k = 0; k < K; ++k, in += ipix) {
        if (k) __syncthreads();  // (everyone has read the previous channel's tile)
        const __amdgpu_buffer_rsrc_t planes[4] = {thin_buffer(in), thin_buffer(in + in_cs), thin_buffer(in + 2 * in_cs),
                                                  thin_buffer(in + 3 * in_cs)};
#pragma unroll 2
        for (int e = threadIdx.x; e < entries; e += THIN_TILE_THREADS) {
            const int row = thin_div(e, P.d_cols), tc = e - row * P.tile_cols;
            const int j = thin_div(row, P.d_rows), tr = row - j * P.tile_rows;
            const int ih = ih0 + tr, iw = iw0 + tc;
            const bool ok = n0 + j < P.N && (unsigned)ih < (unsigned)Hin && (unsigned)iw < (unsigned)Win;
            const unsigned int at = ok ? (unsigned int)(j * image_in + ih * Win + iw) * (unsigned int)sizeof(TS) : THIN_NOWHERE;
            float v[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) v[p] = thin_load<TS>(planes[p], (p && real_x) ? THIN_NOWHERE : at);
            tile[e] = T::entry(v);
        }
        __syncthreads();
        // (one instance of the tap loop per number of slots, so that a tap's reads are issued together)
        const auto run_taps = [&](auto slots) {
            constexpr int NS = decltype(slots)::value;
            int kh = 0, kw = 0;
#pragma unroll 3
            for (int t = 0; t < taps; ++t) {
                const int toff = DGRAD ? (P.Kh - 1 - kh) * P.dh * P.tile_cols + (P.Kw - 1 - kw) * P.dw
                                       : kh * P.dh * P.tile_cols + kw * P.dw;
                const Filter f = filt[k * taps + t];
                Entry x[NS > 0 ? NS : 1];
#pragma unroll
                for (int s = 0; s < NS; ++s) x[s] = tile[tbase[s] + toff];
#pragma unroll
                for (int s = 0; s < NS; ++s) T::mac(acc[s], x[s], f);
                if (++kw == P.Kw) { kw = 0; ++kh; }
            }
        };
        thin_dispatch_slots<THIN_PXT>(wave_slots, run_taps);
    }
    TS* out = static_cast<TS*>(P.out) + ((long)n0 * Cout_all + c) * opix + (long)r0 * Wout;
    const __amdgpu_buffer_rsrc_t oplanes[4] = {thin_buffer(out), thin_buffer(out + out_cs), thin_buffer(out + 2 * out_cs),
                                               thin_buffer(out + 3 * out_cs)};
#pragma unroll
    for (int s = 0; s < THIN_PXT; ++s)
        if (live[s]) {
#pragma unroll
            for (int q = 0; q < 4; ++q) thin_store(oplanes[q], oaddr[s] * (unsigned int)sizeof(TS), (TS)acc[s][q]);
        }
}

// The input gradient of a convolution with stride 2 (along either axis or both) from window tiles: a window entry
// (kh, kw) reaches the input positions of ONE phase (h mod sh, w mod sw) only -- ph(kh) = (kh dh - pt) mod sh -- and
// there it reads the gradient at block row + (ph + pt - kh dh) / sh.  So a thread takes whole sh x sw blocks of input
// positions (two of them), a tile holds the gradient window of R block rows, and every entry is applied once, to the
// accumulators of its phase: no divisibility tests and none of the entries that do not apply (three in four at
// stride 2 x 2) are touched.  The per-entry tile offset and phase are tabled in LDS next to the filter.
constexpr int THIN_PH_SLOTS = 2;  // blocks of input positions per thread

template <int N, typename Body>
__device__ __forceinline__ void thin_dispatch_phase(int phase, const Body& body) {
    if constexpr (N == 1) {
        body(std::integral_constant<int, 0>());
    } else {
        if (phase == N - 1) body(std::integral_constant<int, N - 1>());
        else thin_dispatch_phase<N - 1>(phase, body);
    }
}

template <typename TS, int SH, int SW>
__global__ void __launch_bounds__(WG_THREADS) qconv_thin_dgrad_phase_kernel(const ThinArgs P) {
    using T = ThinTile<TS>;
    using Entry = typename T::Entry;
    using Filter = typename T::Filter;
    constexpr int PHASES = SH * SW;
    extern __shared__ __align__(16) unsigned char thin_lds[];
    const int taps = P.Kh * P.Kw;
    const int c = blockIdx.y;  // input channel, over all groups
    const int K = P.cog, g = c / P.cig, c_in_group = c - g * P.cig;
    Filter* filt = reinterpret_cast<Filter*>(thin_lds);                                    // [output channel of the group][entry]
    int2* table = reinterpret_cast<int2*>(thin_lds + (size_t)K * taps * sizeof(Filter));   // [entry]: tile offset, phase
    Entry* tile = reinterpret_cast<Entry*>(thin_lds + (size_t)K * taps * sizeof(Filter) + (size_t)((taps + 1) & ~1) * sizeof(int2));
    const TS* W = static_cast<const TS*>(P.w);
    for (int e = threadIdx.x; e < K * taps; e += WG_THREADS) {
        const int k = e / taps, t = e - k * taps, kh = t / P.Kw, kw = t - kh * P.Kw;
        const TS* at = W + ((long)g * P.cog + k) * P.so + c_in_group * P.si + kh * P.skh + kw * P.skw;
        float w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = ldf<TS>(at + r * P.wcs);
            w[r] = r ? -v : v;  // conjugate
        }
        filt[e] = T::filter(w);
        if (k == 0) {
            const int ph = ((kh * P.dh - P.pt) % SH + SH) % SH, pw = ((kw * P.dw - P.pl) % SW + SW) % SW;
            const int oh = (ph + P.pt - kh * P.dh) / SH, ow = (pw + P.pl - kw * P.dw) / SW;  // (exact divisions)
            table[t] = make_int2((oh - P.tile_row0) * P.tile_cols + (ow - P.tile_col0), ph * SW + pw);
        }
    }
    const int Hb = (P.H + SH - 1) / SH, Wb = (P.W + SW - 1) / SW;  // blocks of input positions
    const long opix = (long)P.H * P.W, ipix = (long)P.Ho * P.Wo;
    const long Cin_all = (long)P.groups * K, Cout_all = (long)P.groups * P.cig;
    const long in_cs = P.N * Cin_all * ipix, out_cs = P.N * Cout_all * opix;
    const int ng = blockIdx.x / P.tile_bands, band = blockIdx.x - ng * P.tile_bands;
    const int n0 = ng * P.tile_J, r0 = band * P.tile_R;
    const int ih0 = r0 + P.tile_row0, iw0 = P.tile_col0;
    const int entries = P.tile_J * P.tile_rows * P.tile_cols;
    const int image_in = (int)(Cin_all * ipix), image_out = (int)(Cout_all * opix);

    int tbase[THIN_PH_SLOTS], oh0[THIN_PH_SLOTS], ow0[THIN_PH_SLOTS];
    unsigned int oaddr[THIN_PH_SLOTS];
    bool live[THIN_PH_SLOTS];
    float acc[THIN_PH_SLOTS][PHASES][4];
#pragma unroll
    for (int s = 0; s < THIN_PH_SLOTS; ++s) {
        const int pix = threadIdx.x + s * WG_THREADS;
        const int prow = thin_div(pix, P.d_wout), bw = pix - prow * Wb;
        const int j = thin_div(prow, P.d_R), r = prow - j * P.tile_R;
        live[s] = j < P.tile_J && n0 + j < P.N && r0 + r < Hb;
        tbase[s] = live[s] ? (j * P.tile_rows + r) * P.tile_cols + bw : 0;
        oh0[s] = (r0 + r) * SH;
        ow0[s] = bw * SW;
        oaddr[s] = (unsigned int)(j * image_out + r * SH * P.W + bw * SW);
#pragma unroll
        for (int ph = 0; ph < PHASES; ++ph)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[s][ph][q] = 0.f;
    }
    const int wave_first = __builtin_amdgcn_readfirstlane(threadIdx.x & ~63);
    const int total = P.tile_J * P.tile_R * Wb;
    const int wave_slots = total <= wave_first ? 0 : std::min(THIN_PH_SLOTS, (total - wave_first + WG_THREADS - 1) / WG_THREADS);

    const TS* in = static_cast<const TS*>(P.in) + ((long)n0 * Cin_all + (long)g * K) * ipix;
    for (int k = 0; k < K; ++k, in += ipix) {
        if (k) __syncthreads();
        const __amdgpu_buffer_rsrc_t planes[4] = {thin_buffer(in), thin_buffer(in + in_cs), thin_buffer(in + 2 * in_cs),
                                                  thin_buffer(in + 3 * in_cs)};
#pragma unroll 2
        for (int e = threadIdx.x; e < entries; e += WG_THREADS) {
            const int row = thin_div(e, P.d_cols), tc = e - row * P.tile_cols;
            const int j = thin_div(row, P.d_rows), tr = row - j * P.tile_rows;
            const int ih = ih0 + tr, iw = iw0 + tc;
            const bool ok = n0 + j < P.N && (unsigned)ih < (unsigned)P.Ho && (unsigned)iw < (unsigned)P.Wo;
            const unsigned int at = ok ? (unsigned int)(j * image_in + ih * P.Wo + iw) * (unsigned int)sizeof(TS) : THIN_NOWHERE;
            float v[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) v[p] = thin_load<TS>(planes[p], at);
            tile[e] = T::entry(v);
        }
        __syncthreads();
        const auto run_taps = [&](auto slots) {
            constexpr int NS = decltype(slots)::value;
            for (int t = 0; t < taps; ++t) {
                const int2 where = table[t];
                const int toff = __builtin_amdgcn_readfirstlane(where.x), phase = __builtin_amdgcn_readfirstlane(where.y);
                const Filter f = filt[k * taps + t];
                Entry x[NS > 0 ? NS : 1];
#pragma unroll
                for (int s = 0; s < NS; ++s) x[s] = tile[tbase[s] + toff];
                thin_dispatch_phase<PHASES>(phase, [&](auto which) {
                    constexpr int PH = decltype(which)::value;
#pragma unroll
                    for (int s = 0; s < NS; ++s) T::mac(acc[s][PH], x[s], f);
                    // (keeps the phases' instances apart: merged, they would index the accumulators by a variable,
                    // which puts them into scratch memory)
                    asm volatile("; phase %0" ::"n"(PH));
                });
            }
        };
        thin_dispatch_slots<THIN_PH_SLOTS>(wave_slots, run_taps);
    }
    TS* out = static_cast<TS*>(P.out) + ((long)n0 * Cout_all + c) * opix + (long)r0 * SH * P.W;
    const __amdgpu_buffer_rsrc_t oplanes[4] = {thin_buffer(out), thin_buffer(out + out_cs), thin_buffer(out + 2 * out_cs),
                                               thin_buffer(out + 3 * out_cs)};
#pragma unroll
    for (int s = 0; s < THIN_PH_SLOTS; ++s)
#pragma unroll
        for (int ph = 0; ph < SH; ++ph)
#pragma unroll
            for (int pw = 0; pw < SW; ++pw)
                if (live[s] && oh0[s] + ph < P.H && ow0[s] + pw < P.W) {
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        thin_store(oplanes[q], (oaddr[s] + ph * P.W + pw) * (unsigned int)sizeof(TS), (TS)acc[s][ph * SW + pw][q]);
                }
}

static ThinDiv thin_magic(int d) { return d > 1 ? ThinDiv{(unsigned int)(((1ULL << 32) + d - 1) / d), 0u} : ThinDiv{0u, ~0u}; }

// Fills the tile fields of `a` for the forward pass / unit-stride input gradient; false where the tiled kernel does not
// apply (a strided input gradient, rows wider than a workgroup's outputs, a window that does not fit LDS).
static bool thin_tile_plan(bool half_storage, bool dgrad, int filter_entries, int tile_pixels, ThinArgs& a, size_t& lds) {
    if (dgrad && (a.sh != 1 || a.sw != 1)) return false;
    const int Hout = dgrad ? a.H : a.Ho, Wout = dgrad ? a.W : a.Wo;
    const int rstep = dgrad ? 1 : a.sh, cstep = dgrad ? 1 : a.sw;
    if (Wout > tile_pixels) return false;
    const size_t entry = half_storage ? 8 : 16, filter = (size_t)filter_entries * (half_storage ? 32 : 16);
    const long cols = (long)(Wout - 1) * cstep + (long)(a.Kw - 1) * a.dw + 1;
    int R = std::min(Hout, std::max(1, tile_pixels / Wout));
    int J = R == Hout ? std::min(a.N, std::max(1, tile_pixels / (Hout * Wout))) : 1;
    const auto rows_of = [&](int r) { return (long)(r - 1) * rstep + (long)(a.Kh - 1) * a.dh + 1; };
    const auto bytes_of = [&](int r, int j) { return filter + (size_t)j * rows_of(r) * cols * entry; };
    while (J > 1 && bytes_of(R, J) > THIN_TILE_LDS) --J;
    while (R > 1 && bytes_of(R, J) > THIN_TILE_LDS) R = (R + 1) / 2;
    if (bytes_of(R, J) > THIN_TILE_LDS) return false;
    // (the kernels address a tile's J images by 32-bit byte offsets from the first one)
    const long image = (long)a.groups * std::max((long)a.cig * a.H * a.W, (long)a.cog * a.Ho * a.Wo);
    if ((J + 1) * image * (half_storage ? 2 : 4) >= (1L << 32)) return false;
    a.tile_R = R; a.tile_J = J; a.tile_rows = (int)rows_of(R); a.tile_cols = (int)cols;
    a.tile_bands = (Hout + R - 1) / R;
    a.d_cols = thin_magic(a.tile_cols); a.d_rows = thin_magic(a.tile_rows); a.d_wout = thin_magic(Wout); a.d_R = thin_magic(R);
    lds = bytes_of(R, J);
    return true;
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
    const long x_cs = P.real_x ? 0 : P.N * Ci_all * xpix, g_cs = P.N * Co_all * gpix;  // (real-valued x: one stored component)
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
                cx[p] = (!ok || (p && P.real_x)) ? 0.f : p ? -v : v;  // conjugate
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

// The filter gradient from the same window tiles (forward geometry): a workgroup walks over its share of the
// (image group, row band) tiles of one channel pair; per tile it copies the CONJUGATED window of x into LDS, each
// thread takes its (up to four) output positions' gradient values straight from global memory, turns them into the
// filter form of ThinTile -- dw[q] = sum_p s(p,q) conj(x)[p] g[p^q] is the forward product with g in the filter's
// place -- and accumulates TB taps from LDS.  Partial sums per slice of the tiles, as in the kernel above.
constexpr int THIN_WG_PXT = 2;  // output positions per thread and tile of the tiled filter gradient

template <typename TS, int TB>
__global__ void __launch_bounds__(WG_THREADS) qconv_thin_wgrad_tile_kernel(const ThinArgs P) {
    using T = ThinTile<TS>;
    using Entry = typename T::Entry;
    using Filter = typename T::Filter;
    extern __shared__ __align__(16) unsigned char thin_lds[];
    __shared__ float red[WG_THREADS / 64][TB * 4];
    Entry* tile = reinterpret_cast<Entry*>(thin_lds);
    const int pair = blockIdx.x;
    const int co = pair / P.cig, i = pair - co * P.cig, g = co / P.cog;
    const int taps = P.Kh * P.Kw, tap0 = blockIdx.y * TB;
    const long Ci_all = (long)P.groups * P.cig, Co_all = (long)P.groups * P.cog;
    const long xpix = (long)P.H * P.W, gpix = (long)P.Ho * P.Wo;
    const long x_cs = P.real_x ? 0 : P.N * Ci_all * xpix, g_cs = P.N * Co_all * gpix;  // (real-valued x: one stored component)
    const TS* x = static_cast<const TS*>(P.in) + ((long)g * P.cig + i) * xpix;
    const TS* gr = static_cast<const TS*>(P.grad) + (long)co * gpix;
    int toff[TB];  // tile offsets of this workgroup's taps
#pragma unroll
    for (int j = 0; j < TB; ++j) {
        const int t = tap0 + j < taps ? tap0 + j : tap0;  // (a tap beyond the last repeats the first: its sums are dropped)
        toff[j] = (t / P.Kw) * P.dh * P.tile_cols + (t % P.Kw) * P.dw;
    }
    // this thread's output positions inside a tile: numbers tid, tid + 256, .. of J x R x Wo
    const int image_x = (int)(Ci_all * xpix), image_g = (int)(Co_all * gpix);  // elements from an image to the next
    int tbase[THIN_WG_PXT], pj[THIN_WG_PXT], pr[THIN_WG_PXT];
    unsigned int goff[THIN_WG_PXT];  // (32-bit offsets from a tile's first gradient element: see thin_tile_plan)
#pragma unroll
    for (int s = 0; s < THIN_WG_PXT; ++s) {
        const int pix = threadIdx.x + s * WG_THREADS;
        const int prow = thin_div(pix, P.d_wout), pw = pix - prow * P.Wo;
        pj[s] = thin_div(prow, P.d_R);
        pr[s] = prow - pj[s] * P.tile_R;
        tbase[s] = pj[s] < P.tile_J ? (pj[s] * P.tile_rows + pr[s] * P.sh) * P.tile_cols + pw * P.sw : 0;
        goff[s] = (unsigned int)(pj[s] * image_g + pr[s] * P.Wo + pw);
    }
    const int wave_first = __builtin_amdgcn_readfirstlane(threadIdx.x & ~63);
    const int total = P.tile_J * P.tile_R * P.Wo;
    const int wave_slots = total <= wave_first ? 0 : std::min(THIN_WG_PXT, (total - wave_first + WG_THREADS - 1) / WG_THREADS);
    const int entries = P.tile_J * P.tile_rows * P.tile_cols;
    const int ntiles = ((P.N + P.tile_J - 1) / P.tile_J) * P.tile_bands;
    const int t0 = (int)((long)blockIdx.z * ntiles / P.Z), t1 = (int)((long)(blockIdx.z + 1) * ntiles / P.Z);
    float acc[TB][4];
#pragma unroll
    for (int j = 0; j < TB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[j][q] = 0.f;

    const auto run_tiles = [&](auto slots) {
        constexpr int NS = decltype(slots)::value;
        int ng = t0 / P.tile_bands, band = t0 - ng * P.tile_bands;
        for (int tile_idx = t0; tile_idx < t1; ++tile_idx) {
            const int n0 = ng * P.tile_J, r0 = band * P.tile_R;
            const TS* gtile = gr + (long)n0 * Co_all * gpix + (long)r0 * P.Wo;
            const __amdgpu_buffer_rsrc_t gplanes[4] = {thin_buffer(gtile), thin_buffer(gtile + g_cs), thin_buffer(gtile + 2 * g_cs),
                                                       thin_buffer(gtile + 3 * g_cs)};
            float gv[NS > 0 ? NS : 1][4];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const bool live = pj[s] < P.tile_J && n0 + pj[s] < P.N && r0 + pr[s] < P.Ho;
                const unsigned int at = live ? goff[s] * (unsigned int)sizeof(TS) : THIN_NOWHERE;
#pragma unroll
                for (int q = 0; q < 4; ++q) gv[s][q] = thin_load<TS>(gplanes[q], at);
            }
            if (tile_idx != t0) __syncthreads();  // (everyone has read the previous tile)
            const int ih0 = r0 * P.sh - P.pt, iw0 = -P.pl;
            const TS* xin = x + (long)n0 * Ci_all * xpix;
            const __amdgpu_buffer_rsrc_t xplanes[4] = {thin_buffer(xin), thin_buffer(xin + x_cs), thin_buffer(xin + 2 * x_cs),
                                                       thin_buffer(xin + 3 * x_cs)};
#pragma unroll 2
            for (int e = threadIdx.x; e < entries; e += WG_THREADS) {
                const int row = thin_div(e, P.d_cols), tc = e - row * P.tile_cols;
                const int j = thin_div(row, P.d_rows), tr = row - j * P.tile_rows;
                const int ih = ih0 + tr, iw = iw0 + tc;
                const bool ok = n0 + j < P.N && (unsigned)ih < (unsigned)P.H && (unsigned)iw < (unsigned)P.W;
                const unsigned int at = ok ? (unsigned int)(j * image_x + ih * P.W + iw) * (unsigned int)sizeof(TS) : THIN_NOWHERE;
                float v[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const float f = thin_load<TS>(xplanes[p], (p && P.real_x) ? THIN_NOWHERE : at);
                    v[p] = p ? -f : f;  // conjugate
                }
                tile[e] = T::entry(v);
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const Filter f = T::filter(gv[s]);
                Entry xv[TB];
#pragma unroll
                for (int j = 0; j < TB; ++j) xv[j] = tile[tbase[s] + toff[j]];
#pragma unroll
                for (int j = 0; j < TB; ++j) T::mac(acc[j], xv[j], f);
            }
            if (++band == P.tile_bands) { band = 0; ++ng; }
        }
    };
    thin_dispatch_slots<THIN_WG_PXT>(wave_slots, run_tiles);  // (a wave without outputs still fills and meets the barriers)
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

// The plan of the strided input gradient by phases (strides 1 or 2 per axis): blocks of sh x sw input positions play
// the part of the outputs, the tile is the gradient window of R block rows.
static bool thin_phase_plan(bool half_storage, ThinArgs& a, size_t& lds) {
    if (a.sh > 2 || a.sw > 2 || (a.sh == 1 && a.sw == 1)) return false;
    const int Hb = (a.H + a.sh - 1) / a.sh, Wb = (a.W + a.sw - 1) / a.sw, taps = a.Kh * a.Kw;
    const int tile_pixels = THIN_PH_SLOTS * WG_THREADS;
    if (Wb > tile_pixels) return false;
    const auto span = [](int k, int d, int pad, int s, int& lo, int& hi) {  // block offsets that the window entries read
        lo = 1 << 30; hi = -(1 << 30);
        for (int i = 0; i < k; ++i) {
            const int ph = ((i * d - pad) % s + s) % s, o = (ph + pad - i * d) / s;
            lo = std::min(lo, o); hi = std::max(hi, o);
        }
    };
    int rlo, rhi, clo, chi;
    span(a.Kh, a.dh, a.pt, a.sh, rlo, rhi);
    span(a.Kw, a.dw, a.pl, a.sw, clo, chi);
    const size_t entry = half_storage ? 8 : 16;
    const size_t fixed = (size_t)a.cog * taps * (half_storage ? 32 : 16) + (size_t)((taps + 1) & ~1) * 8;
    const long cols = (long)Wb + chi - clo;
    int R = std::min(Hb, std::max(1, tile_pixels / Wb));
    int J = R == Hb ? std::min(a.N, std::max(1, tile_pixels / (Hb * Wb))) : 1;
    const auto bytes_of = [&](int r, int j) { return fixed + (size_t)j * (r + rhi - rlo) * cols * entry; };
    while (J > 1 && bytes_of(R, J) > THIN_TILE_LDS) --J;
    while (R > 1 && bytes_of(R, J) > THIN_TILE_LDS) R = (R + 1) / 2;
    if (bytes_of(R, J) > THIN_TILE_LDS) return false;
    const long image = (long)a.groups * std::max((long)a.cig * a.H * a.W, (long)a.cog * a.Ho * a.Wo);
    if ((J + 1) * image * (half_storage ? 2 : 4) >= (1L << 32)) return false;
    a.tile_R = R; a.tile_J = J; a.tile_rows = R + rhi - rlo; a.tile_cols = (int)cols;
    a.tile_bands = (Hb + R - 1) / R;
    a.tile_row0 = rlo; a.tile_col0 = clo;
    a.d_cols = thin_magic(a.tile_cols); a.d_rows = thin_magic(a.tile_rows); a.d_wout = thin_magic(Wb); a.d_R = thin_magic(R);
    lds = bytes_of(R, J);
    return true;
}

static int thin_wgrad_taps_per_block(int taps) { return taps == 1 ? 1 : 9; }

// The filter gradient's plan: tiled kernel or not (tile fields of `a`, LDS bytes), and the number of slices Z of the
// images (tiles) whose partial sums separate workgroups make -- enough workgroups to fill the GPU, each with work
// worth its prologue.
static bool thin_wgrad_plan(bool half_storage, ThinArgs& a, size_t& lds) {
    const int taps = a.Kh * a.Kw, TB = thin_wgrad_taps_per_block(taps);
    const long columns = (long)a.groups * a.cog * a.cig * ((taps + TB - 1) / TB);
    const long want = (2048 + columns - 1) / columns;
    if (!tuning_thin_notile() && thin_tile_plan(half_storage, false, 0, THIN_WG_PXT * WG_THREADS, a, lds)) {
        const long ntiles = (long)((a.N + a.tile_J - 1) / a.tile_J) * a.tile_bands;
        a.Z = (int)std::max(1L, std::min({want, ntiles, 65535L}));
        return true;
    }
    const long fit = std::max(1L, (long)a.N * a.Ho * a.Wo / (4 * WG_THREADS));
    a.Z = (int)std::max(1L, std::min({want, fit, (long)a.N, 65535L}));
    return false;
}

int thin_wgrad_slices(bool half_storage, const ThinArgs& a) {
    ThinArgs t = a;
    size_t lds = 0;
    thin_wgrad_plan(half_storage, t, lds);
    return t.Z;
}

int launch_thin(bool half_storage, int pass, const ThinArgs& a, hipStream_t st) {
    const int taps = a.Kh * a.Kw;
    if (pass == PHX_PASS_BWD_WEIGHTS) {
        const long pairs = (long)a.groups * a.cog * a.cig;
        const int TB = thin_wgrad_taps_per_block(taps);
        ThinArgs t = a;
        size_t lds = 0;
        const bool tiled = thin_wgrad_plan(half_storage, t, lds);
        if (pairs >= (1L << 31) || t.Z != a.Z || !a.partial) return -1;  // (the caller sized `partial` for thin_wgrad_slices())
        const dim3 grid((unsigned int)pairs, (unsigned int)((taps + TB - 1) / TB), (unsigned int)t.Z), block(WG_THREADS);
        if (tiled) {
            if (TB == 1) {
                if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_tile_kernel<_Float16, 1>), grid, block, lds, st, t);
                else hipLaunchKernelGGL((qconv_thin_wgrad_tile_kernel<float, 1>), grid, block, lds, st, t);
            } else {
                if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_tile_kernel<_Float16, 9>), grid, block, lds, st, t);
                else hipLaunchKernelGGL((qconv_thin_wgrad_tile_kernel<float, 9>), grid, block, lds, st, t);
            }
        } else if (TB == 1) {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_kernel<_Float16, 1>), grid, block, 0, st, t);
            else hipLaunchKernelGGL((qconv_thin_wgrad_kernel<float, 1>), grid, block, 0, st, t);
        } else {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_wgrad_kernel<_Float16, 9>), grid, block, 0, st, t);
            else hipLaunchKernelGGL((qconv_thin_wgrad_kernel<float, 9>), grid, block, 0, st, t);
        }
        const dim3 rgrid((unsigned int)((pairs * taps * 4 + WG_THREADS - 1) / WG_THREADS));
        if (half_storage) hipLaunchKernelGGL(thin_wgrad_reduce_kernel<_Float16>, rgrid, block, 0, st, t);
        else hipLaunchKernelGGL(thin_wgrad_reduce_kernel<float>, rgrid, block, 0, st, t);
        return tiled ? 1 : 0;
    }
    const bool dgrad = pass == PHX_PASS_BWD_DATA;
    if (dgrad && (a.sh > 1 || a.sw > 1) && (long)std::max(a.H + a.pt, a.W + a.pl) * std::max(a.sh, a.sw) >= (1L << 31)) return -1;
    const long channels = (long)a.groups * (dgrad ? a.cig : a.cog);
    if (channels > 65535) return -1;
    ThinArgs t = a;
    size_t tile_lds = 0;
    if (!tuning_thin_notile() && thin_tile_plan(half_storage, dgrad, (dgrad ? a.cog : a.cig) * taps, THIN_TILE_PIXELS, t, tile_lds)) {
        const long blocks = (long)((a.N + t.tile_J - 1) / t.tile_J) * t.tile_bands;
        if (blocks >= (1L << 31)) return -1;
        const dim3 grid((unsigned int)blocks, (unsigned int)channels), block(THIN_TILE_THREADS);
        if (dgrad) {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_tile_kernel<_Float16, true>), grid, block, tile_lds, st, t);
            else hipLaunchKernelGGL((qconv_thin_tile_kernel<float, true>), grid, block, tile_lds, st, t);
        } else {
            if (half_storage) hipLaunchKernelGGL((qconv_thin_tile_kernel<_Float16, false>), grid, block, tile_lds, st, t);
            else hipLaunchKernelGGL((qconv_thin_tile_kernel<float, false>), grid, block, tile_lds, st, t);
        }
        return 1;
    }
    if (!tuning_thin_notile() && dgrad && thin_phase_plan(half_storage, t, tile_lds)) {
        const long blocks = (long)((a.N + t.tile_J - 1) / t.tile_J) * t.tile_bands;
        if (blocks >= (1L << 31)) return -1;
        const dim3 grid((unsigned int)blocks, (unsigned int)channels), block(WG_THREADS);
        const int key = t.sh * 10 + t.sw;
        if (half_storage) {
            if (key == 22) hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<_Float16, 2, 2>), grid, block, tile_lds, st, t);
            else if (key == 21) hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<_Float16, 2, 1>), grid, block, tile_lds, st, t);
            else hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<_Float16, 1, 2>), grid, block, tile_lds, st, t);
        } else {
            if (key == 22) hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<float, 2, 2>), grid, block, tile_lds, st, t);
            else if (key == 21) hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<float, 2, 1>), grid, block, tile_lds, st, t);
            else hipLaunchKernelGGL((qconv_thin_dgrad_phase_kernel<float, 1, 2>), grid, block, tile_lds, st, t);
        }
        return 2;
    }
    const long pixels = (long)a.N * (dgrad ? (long)a.H * a.W : (long)a.Ho * a.Wo);
    const long blocks = (pixels + WG_THREADS - 1) / WG_THREADS;
    const int K = dgrad ? a.cog : a.cig;
    t.kchunk = std::min(K, (int)(THIN_FILTER_LDS / (taps * sizeof(float4))));
    if (blocks >= (1L << 31) || t.kchunk < 1) return -1;
    const size_t lds = (size_t)t.kchunk * taps * sizeof(float4);
    const dim3 grid((unsigned int)blocks, (unsigned int)channels), block(WG_THREADS);
    if (dgrad) {
        if (half_storage) hipLaunchKernelGGL((qconv_thin_kernel<_Float16, true>), grid, block, lds, st, t);
        else hipLaunchKernelGGL((qconv_thin_kernel<float, true>), grid, block, lds, st, t);
    } else {
        if (half_storage) hipLaunchKernelGGL((qconv_thin_kernel<_Float16, false>), grid, block, lds, st, t);
        else hipLaunchKernelGGL((qconv_thin_kernel<float, false>), grid, block, lds, st, t);
    }
    return 0;
}

}  // namespace phx
