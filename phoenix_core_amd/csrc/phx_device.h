// Shared device-side helpers of the gfx950 quaternion kernels: vector types, storage<->compute
// conversions, the Hamilton sign table, the lane maps of the factorized product and the generic
// global->LDS tile loader.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace phx {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
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

// -v for eight packed halves: flip the sign bits with four integer XORs (the generic vector negate
// lowers to three instructions per register)
__device__ __forceinline__ f16x8 neg8(const f16x8 v) {
    const u32x4 m = {0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
    return __builtin_bit_cast(f16x8, __builtin_bit_cast(u32x4, v) ^ m);
}

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

// The same lane maps on eight packed halves.  The compiler expands a vector subtraction of halves
// into scalar operations (three instructions per register); a - b is written as a + (-b) with the
// sign flipped by an integer XOR, which it cannot fold back into a subtraction: two instructions.
__device__ __forceinline__ f16x8 sub8(const f16x8 a, const f16x8 b) { return a + neg8(b); }

// Single-instruction forms, a + b and a - b as one packed add (second operand negated).  The
// instruction scheduler and the hazard logic of the compiler do not see through these: use them only
// where the result is consumed many instructions later (lane_step in the LDS forward kernel), and
// they then stay exactly where they are written, between the matrix instructions they overlap with.
__device__ __forceinline__ f16x8 add8_pinned(const f16x8 a, const f16x8 b) {
    const u32x4 ua = __builtin_bit_cast(u32x4, a), ub = __builtin_bit_cast(u32x4, b);
    u32x4 r;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        unsigned int t;
        asm("v_pk_add_f16 %0, %1, %2" : "=v"(t) : "v"(ua[m]), "v"(ub[m]));
        r[m] = t;
    }
    return __builtin_bit_cast(f16x8, r);
}

__device__ __forceinline__ f16x8 sub8_pinned(const f16x8 a, const f16x8 b) {
    const u32x4 ua = __builtin_bit_cast(u32x4, a), ub = __builtin_bit_cast(u32x4, b);
    u32x4 r;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        unsigned int t;
        asm("v_pk_add_f16 %0, %1, %2 neg_lo:[0,1] neg_hi:[0,1]" : "=v"(t) : "v"(ua[m]), "v"(ub[m]));
        r[m] = t;
    }
    return __builtin_bit_cast(f16x8, r);
}

__device__ __forceinline__ void lanes_left(const f16x8 (&x)[4], f16x8 (&L)[8]) {
    const f16x8 n1 = neg8(x[1]), n2 = neg8(x[2]);
    L[0] = x[3] + x[1];
    L[1] = x[0] + n2;
    L[2] = x[0] + x[2];
    L[3] = x[3] + n1;
    L[4] = x[3] + n2;
    L[5] = x[1] + x[0];
    L[6] = x[0] + n1;
    L[7] = x[3] + x[2];
}

// lanes_grad without the factor 1/2 on lanes 0..3 (the caller folds it into the other operand)
__device__ __forceinline__ void lanes_grad_unscaled(const f16x8 (&g)[4], f16x8 (&G)[8]) {
    const f16x8 t1 = g[0] + g[1], t3 = g[0] + neg8(g[1]), t2 = g[2] + g[3], t4 = g[2] + neg8(g[3]);
    G[0] = t2 + neg8(t1);
    G[1] = t3 + neg8(t4);
    G[2] = t3 + t4;
    G[3] = t1 + t2;
    G[4] = g[0];
    G[5] = g[1];
    G[6] = g[2];
    G[7] = g[3];
}

__device__ __forceinline__ void lanes_grad(const f16x8 (&g)[4], f16x8 (&G)[8], _Float16 half) {
    lanes_grad_unscaled(g, G);
#pragma unroll
    for (int i = 0; i < 4; ++i) G[i] = G[i] * half;
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

// 16- and 4-byte global loads from addresses with only 2-byte alignment (one instruction each).
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef unsigned int u32_a2 __attribute__((aligned(2)));

__device__ __forceinline__ u32x4 load16_a2(const _Float16* p) {
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a2*>(
        (const __attribute__((address_space(1))) _Float16*)p);
}
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
__device__ __forceinline__ u32x2 load8_a2(const _Float16* p) {
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x2_a2*>(
        (const __attribute__((address_space(1))) _Float16*)p);
}
__device__ __forceinline__ unsigned int load4_a2(const _Float16* p) {
    return *reinterpret_cast<const __attribute__((address_space(1))) u32_a2*>(
        (const __attribute__((address_space(1))) _Float16*)p);
}

// Bit masks over the eight fp16 values of a 16-byte chunk.
// bit i of `bits` set <=> half i of the chunk is kept
__device__ __forceinline__ u32x4 expand_half_mask(unsigned int bits) {
    u32x4 mk;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const unsigned int lo = (unsigned int)((int)(bits << (31 - 2 * d)) >> 31);
        const unsigned int hi = (unsigned int)((int)(bits << (30 - 2 * d)) >> 31);
        mk[d] = (lo & 0x0000FFFFu) | (hi & 0xFFFF0000u);
    }
    return mk;
}

// bits [lo, hi) set, both clamped to [0, MAXB]
template <int MAXB = 8>
__device__ __forceinline__ unsigned int interval_bits(int lo, int hi) {
    lo = lo < 0 ? 0 : lo;
    hi = hi > MAXB ? MAXB : hi;
    return hi > lo ? ((1u << hi) - (1u << lo)) : 0u;
}

// Developer option -DPHX_PHASE_TIMING: a kernel brackets its phases with PHX_STAMP(i); the shader
// clocks spent in each phase (at most six) are summed per wave and printed by lane 0 of every 97th workgroup.
// Without the option the macros expand to nothing.
#ifdef PHX_PHASE_TIMING
#define PHX_PHASES_BEGIN(n) long long phx_tph[6] = {}; long long phx_tlast = clock64();
#define PHX_STAMP(i)                                             \
    {                                                            \
        __builtin_amdgcn_sched_barrier(0);                       \
        const long long phx_now = clock64();                     \
        phx_tph[i] += phx_now - phx_tlast;                       \
        phx_tlast = phx_now;                                     \
        __builtin_amdgcn_sched_barrier(0);                       \
    }
#define PHX_PHASES_REPORT(what, n)                                                                           \
    if ((blockIdx.x % 97) == 0 && (threadIdx.x & 63) == 0)                                                   \
        printf("%s | wg %d wave %d: %lld %lld %lld %lld %lld %lld\n", what, (int)blockIdx.x,                 \
               (int)(threadIdx.x >> 6), phx_tph[0], phx_tph[1], phx_tph[2], phx_tph[3], phx_tph[4], phx_tph[5]);
#else
#define PHX_PHASES_BEGIN(n)
#define PHX_STAMP(i)
#define PHX_PHASES_REPORT(what, n)
#endif

// Sixty-four zero bytes in device memory: out-of-tensor staging positions load from here, which
// keeps the staging loads unconditional and free of selects.
static __device__ __attribute__((aligned(16))) const unsigned int phx_zero_block[16] = {};

template <typename T>
__device__ __forceinline__ const T* zero_ptr() {
    return reinterpret_cast<const T*>(phx_zero_block);
}

// A rectangular window of a component-stacked NCHW tensor t[4][N][C][Hd][Wd], seen through an
// optional zero-insertion (virtual coordinate v maps to stored v/u when v % u == 0, else zero).
// One launch for all groups of a grouped convolution: the workgroups of grid row blockIdx.y work on group blockIdx.y,
// whose tensors lie blockIdx.y times a byte step behind group 0's (a grid of one row, i.e. no shift, otherwise).
__device__ __forceinline__ const void* group_shift(const void* p, long step) {
    return p ? static_cast<const char*>(p) + (long)blockIdx.y * step : nullptr;
}
__device__ __forceinline__ void* group_shift(void* p, long step) {
    return p ? static_cast<char*>(p) + (long)blockIdx.y * step : nullptr;
}

struct TileSrc {
    const void* base;
    long comp_stride;  // elements between components
    int N, C, Hd, Wd;  // stored dims per component
    int Cs;            // channels per image in memory (>= C: a grouped convolution sees a slice of C channels from base on)
    int uh, uw;        // zero-insertion factors (1 = none)
    int ncomp;         // components present in memory: 4, or 1 for a real-valued tensor (components 1..3 read as zero)
    int pw;            // pointwise trick: window row r holds channels (chunk*pw + r)*16.. of the single image row (0 = off)
    int tall;          // flat tiling: the images are rows [n*tall, n*tall + Hd) of one tall image, zero rows between them (0 = off)
    int nhwc;          // channels-last memory, t[4][N][Hd][Wd][Cs] (chunk staging of the fp16 LDS kernels only; 0 = planes)
};

// Window staging, split so that global loads can be in flight while the previous chunk is being
// multiplied: each thread owns ONE position of the window [n0, n0+NB) x [h0, h0+HTH) x [w0, w0+HTW)
// (decoded once, it does not depend on the channel) and walks over the (component, channel) planes
// of a chunk.  The 256 threads form G = 256 >> P2LOG groups of 2^P2LOG positions; group g loads
// planes g, g+G, ...  Loads are unconditional (out-of-tensor positions read a block of zeros) so
// that the staged values stay plain registers.
struct StagePos {
    long goff;   // offset of this thread's position from the start of component 0, channel 0
    int pos;     // position inside the window, < 2^P2LOG
    int group;   // which plane subset this thread loads
    bool valid;  // position lies inside the tensor (otherwise it is staged as zero)
};

template <int P2LOG>
__device__ __forceinline__ StagePos make_stage_pos(const TileSrc& s, int n0, int h0, int w0, int NB, int HTH, int HTW) {
    StagePos sp;
    sp.pos = threadIdx.x & ((1 << P2LOG) - 1);
    sp.group = threadIdx.x >> P2LOG;
    const int hw = HTH * HTW;
    const int nb = sp.pos / hw, rem = sp.pos - nb * hw;
    const int hr = rem / HTW, hc = rem - hr * HTW;
    int vh = h0 + hr, vw = w0 + hc;
    bool ok = nb < NB && (n0 + nb) < s.N && vh >= 0 && vw >= 0;
    if (s.uh > 1) { ok = ok && (vh % s.uh == 0); vh /= s.uh; }
    if (s.uw > 1) { ok = ok && (vw % s.uw == 0); vw /= s.uw; }
    ok = ok && vh < s.Hd && vw < s.Wd;
    sp.valid = ok;
    sp.goff = ok ? ((long)(n0 + nb) * s.Cs * s.Hd + vh) * s.Wd + vw : 0;
    return sp;
}

// Issues the loads of one chunk: NCH channels starting at c0, all four components.
// v[e] receives plane pc = e*G + group, pc = p*NCH + c.
template <typename TS, int NCH, int P2LOG>
__device__ __forceinline__ void stage_load(float (&v)[(4 * NCH) >> (8 - P2LOG)], const TileSrc& s, const StagePos& sp,
                                           int c0) {
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = (4 * NCH) / G;
    const TS* origin = static_cast<const TS*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int pc = e * G + sp.group;
        const int p = pc / NCH, c = pc % NCH;
        const bool ok = sp.valid && (c0 + c) < s.C && p < s.ncomp;
        const TS* ptr = ok ? origin + sp.goff + p * s.comp_stride + (long)(c0 + c) * plane : zero_ptr<TS>();
        v[e] = ldf<TS>(ptr);
    }
}

// Writes the staged chunk as dst[pc*pitch + pos]
template <int NCH, int P2LOG, typename TD>
__device__ __forceinline__ void stage_store(TD* dst, const float (&v)[(4 * NCH) >> (8 - P2LOG)], const StagePos& sp,
                                            int HP, int pitch) {
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = (4 * NCH) / G;
    if (sp.pos < HP) {
#pragma unroll
        for (int e = 0; e < E; ++e) dst[(e * G + sp.group) * pitch + sp.pos] = (TD)v[e];
    }
}

}  // namespace phx
