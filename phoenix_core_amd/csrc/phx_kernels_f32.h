// fp32-MFMA kernels (v_mfma_f32_32x32x2_f32): quaternion convolution forward / input-gradient
// (one kernel, two lane maps) and filter-gradient, in the 16-product and the factorized 8-product
// formulation.  Storage type TS is float or _Float16 (operands widened while staged into LDS).
#pragma once

#include "phx_device.h"

namespace phx {

enum { MAP_FWD = 0, MAP_DGRAD = 1 };

constexpr int F32_CK = 8;   // fp32 MFMA: input channels per K chunk (4 MFMA k-pairs)
constexpr int F16_CK = 16;  // fp16 MFMA: input channels per K chunk = one MFMA K step (two 8-channel packs)
constexpr int F16_TG = 3;   // fp16 MFMA, LDS-staged filters: taps per filter group
constexpr int F16_XPITCH = 256;  // fp16 LDS kernels with chunk staging: entries per unit of the staged window

struct ConvArgs {
    TileSrc in;         // x (forward) or the output gradient (input-gradient pass)
    const void* wpk;    // packed filters (see the pack_filters kernels), in the MFMA operand type
    const void* bias;   // [4][Cout] in storage type or null
    void* out;
    long out_cs;        // elements between output components
    int Cout, Hout, Wout;
    int CoutS;          // output channels per image in memory (>= Cout: grouped convolutions write a slice); also the bias stride
    int taps, Kw;       // filter taps (Kh*Kw) and filter width
    int dh, dw, sh, sw; // dilation and stride of the correlation
    int pt, pl;         // virtual input row of output row 0, tap 0, is -pt (same for columns)
    int NB, TH, TW;     // output pixels per workgroup tile: images x rows x columns
    int HTH, HTW, HP, HPp;  // halo window, its size and the LDS pitch per staged channel
    int tiles_n, tiles_h, tiles_w, co_tiles;
    int nchunks;        // ceil(Cin / CK) for the kernel's chunk size CK
    int vec;            // output pixels a lane stores at once (4, 2 or 1): divides TW and Wout
    int nhwc;           // the output is channels-last, out[4][N][Hout][Wout][CoutS] (fp16 chunk-staging kernel only)
    int groups;         // grid rows: the groups of a grouped convolution run by this one launch (1 otherwise)
    long g_in, g_w, g_bias, g_out;  // bytes from one group's input / packed filters / bias / output to the next group's
};

// the arguments as group blockIdx.y sees them
__device__ __forceinline__ ConvArgs group_view(const ConvArgs& P0) {
    ConvArgs P = P0;
    P.in.base = group_shift(P0.in.base, P0.g_in);
    P.wpk = group_shift(P0.wpk, P0.g_w);
    P.bias = group_shift(P0.bias, P0.g_bias);
    P.out = group_shift(P0.out, P0.g_out);
    return P;
}

// ---------------------------------------------------------------------------------------------
// Epilogue shared by the forward / input-gradient kernels (32x32 MFMA tiles: a lane holds one pixel
// column, register e the channel row 8*(e/4) + 4*(lane/32) + e%4).  Vector memory instructions are
// accepted at a fixed rate per wave whatever their width, so 64 scalar stores per column tile are
// the expensive way out.  Each group of four registers (four consecutive channels) is transposed
// across the four lanes of a quad (four consecutive pixels) with DPP moves; a lane then owns one
// channel x four pixels and stores them as one 8- or 16-byte word.  P.vec == 2 does the same with
// lane pairs, P.vec == 1 is the scalar form for tiles whose rows do not divide.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
}

// a[k] = row k at this lane's column -> o[m] = row (lane & 1) + 2*h at columns (pair base + m), h = 0, 1
__device__ __forceinline__ void pair_transpose(const float (&a)[4], float (&b)[2], float (&d)[2], bool odd) {
    const float n0 = dpp_quad_xor1(a[0]), n1 = dpp_quad_xor1(a[1]), n2 = dpp_quad_xor1(a[2]), n3 = dpp_quad_xor1(a[3]);
    b[0] = odd ? n1 : a[0];  b[1] = odd ? a[1] : n0;   // rows 0 / 1
    d[0] = odd ? n3 : a[2];  d[1] = odd ? a[3] : n2;   // rows 2 / 3
}

// a[k] = row k at this lane's column -> o[m] = row (lane & 3) at columns (quad base + m)
__device__ __forceinline__ void quad_transpose(const float (&a)[4], float (&o)[4], int ql) {
    float b[2], d[2];
    pair_transpose(a, b, d, ql & 1);
    const bool hi = ql & 2;
    const float s0 = hi ? b[0] : d[0], s1 = hi ? b[1] : d[1];
    const float r0 = dpp_quad_xor2(s0), r1 = dpp_quad_xor2(s1);
    o[0] = hi ? r0 : b[0];  o[1] = hi ? r1 : b[1];
    o[2] = hi ? d[0] : r0;  o[3] = hi ? d[1] : r1;
}

template <typename TS, int V>
__device__ __forceinline__ void store_pixels(TS* ptr, const float (&v)[V]) {
    if constexpr (sizeof(TS) == 4) {
        typedef float fv __attribute__((ext_vector_type(V), aligned(4)));
        fv w;
#pragma unroll
        for (int i = 0; i < V; ++i) w[i] = v[i];
        *reinterpret_cast<fv*>(ptr) = w;
    } else {
        typedef _Float16 hv __attribute__((ext_vector_type(V), aligned(2)));
        hv w;
#pragma unroll
        for (int i = 0; i < V; ++i) w[i] = (_Float16)v[i];
        *reinterpret_cast<hv*>(ptr) = w;
    }
}

template <typename TS, int MODE, int NTW, int NACC>
__device__ __forceinline__ void conv_epilogue(const ConvArgs& P, const f32x16 (&acc)[NTW][NACC], int co_base,
                                              const long (&oaddr)[NTW], const bool (&pvalid)[NTW]) {
    TS* out = static_cast<TS*>(P.out);
    const TS* bias = static_cast<const TS*>(P.bias);
    const long plane = (long)P.Hout * P.Wout;
    const int ql = threadIdx.x & 3;
    auto component_rows = [&](int t, int e, float (&y)[4]) {  // the four output components of register e
        if constexpr (MODE == 16) {
#pragma unroll
            for (int q = 0; q < 4; ++q) y[q] = acc[t][q][e];
        } else {
            float l[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) l[i] = acc[t][i][e];
            merge_output(l, y);
        }
    };
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        if (!pvalid[t]) continue;  // uniform over a quad / pair when P.vec > 1
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            float y[4][4];  // [row in group][component]
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                component_rows(t, rq * 4 + k, y[k]);
                const int co = co_base + 8 * rq + k;
                if (bias && co < P.Cout) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) y[k][q] += ldf<TS>(bias + q * P.CoutS + co);
                }
            }
            if (P.vec == 4) {
                const int co = co_base + 8 * rq + ql;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float a[4] = {y[0][q], y[1][q], y[2][q], y[3][q]};
                    float o[4];
                    quad_transpose(a, o, ql);
                    if (co < P.Cout) store_pixels<TS, 4>(out + q * P.out_cs + (oaddr[t] - ql) + co * plane, o);
                }
            } else if (P.vec == 2) {
                const int odd = ql & 1;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float a[4] = {y[0][q], y[1][q], y[2][q], y[3][q]};
                    float b[2], d[2];
                    pair_transpose(a, b, d, odd);
                    const int co = co_base + 8 * rq + odd;
                    TS* dst = out + q * P.out_cs + (oaddr[t] - odd);
                    if (co < P.Cout) store_pixels<TS, 2>(dst + co * plane, b);
                    if (co + 2 < P.Cout) store_pixels<TS, 2>(dst + (co + 2) * plane, d);
                }
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int co = co_base + 8 * rq + k;
                    if (co < P.Cout) {
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            stf<TS>(out + q * P.out_cs + oaddr[t] + co * plane, y[k][q]);
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Vector staging of the activation window for the fp32-MFMA kernels (VSTG): the LDS layout
// [component][channel][position] is position-contiguous like NCHW itself, so staging is a plain
// copy.  A thread owns one group of 4 consecutive positions of a window row (HTW is a multiple of 4)
// and walks over the (component, channel) planes: one 16-byte (fp32) or 8-byte (fp16 storage) load
// and one 16-byte LDS store per plane, a quarter of the instructions of the per-position form.
// Positions outside the image are cleared with a mask that is fixed per thread; threads whose
// loads could leave the tensor load nothing and fill their positions element by element.
// 2^(P2LOG-2) position groups x (1024 >> P2LOG) thread groups; thread group g takes planes g, g+G4, ...
// ---------------------------------------------------------------------------------------------
struct StageVec {
    long goff;           // element offset of the group's first position from component 0, channel 0
    long tbase;          // goff + the offset of the thread group's own (component, channel) plane
    int lpos;            // first window position of the group
    int group;
    int c_room, p_room;  // channels / components from the thread group's own plane to the end of the tensor
    unsigned int bits;   // positions inside the image
    bool live, careful;
    bool fast;           // live and every vector load stays inside the tensor
};

// What a thread's position group is, apart from the window's origin: decoded once per kernel.
struct StageVecLane {
    int lpos, group, nb, hr, col;
    bool inside;  // the group lies inside the window
};

template <int P2LOG>
__device__ __forceinline__ StageVecLane make_stage_vec_lane(int NB, int HTH, int HTW, int HP) {
    StageVecLane L;
    constexpr int NPC = 1 << (P2LOG - 2);
    const int pc = threadIdx.x & (NPC - 1);
    L.group = threadIdx.x >> (P2LOG - 2);
    L.lpos = pc * 4;
    const int row = L.lpos / HTW;
    L.col = L.lpos - row * HTW;
    L.nb = row / HTH;
    L.hr = row - L.nb * HTH;
    L.inside = L.lpos < HP && L.nb < NB;
    return L;
}

// NCH channels per chunk: thread group g takes planes g, g + G4, ... of the chunk's 4*NCH (component, channel)
// planes; plane pc is (component pc / NCH, channel pc % NCH).  With G4 and NCH powers of two, the plane of load e
// is (p_group + pe(e), c_group + ce(e)) with pe, ce the same for every thread.
// vector loads per thread and chunk
constexpr int stage_loads(int nch, int p2log, int nt) { return (4 * nch) / (nt >> (p2log - 2)); }

template <int NCH, int P2LOG, int NT = WG_THREADS>
struct StagePlanes {
    static constexpr int G4 = NT >> (P2LOG - 2);   // thread groups
    static constexpr int E = stage_loads(NCH, P2LOG, NT);
    static __device__ __forceinline__ int p_group(int group) { return G4 >= NCH ? group / NCH : 0; }
    static __device__ __forceinline__ int c_group(int group) { return G4 >= NCH ? group % NCH : group; }
    static __device__ __forceinline__ int pe(int e) { return G4 >= NCH ? e * (G4 / NCH) : (e * G4) / NCH; }
    static __device__ __forceinline__ int ce(int e) { return G4 >= NCH ? 0 : (e * G4) % NCH; }
};

template <typename TS, int NCH, int P2LOG, int NT = WG_THREADS>
__device__ __forceinline__ StageVec place_stage_vec(const TileSrc& s, const StageVecLane& L, int n0, int h0, int w0) {
    typedef StagePlanes<NCH, P2LOG, NT> PL;
    StageVec sv;
    sv.group = L.group;
    sv.lpos = L.lpos;
    const int vh = h0 + L.hr, vw0 = w0 + L.col;
    sv.live = L.inside && (n0 + L.nb) < s.N && vh >= 0 && vh < s.Hd;
    sv.bits = sv.live ? interval_bits<4>(-vw0, s.Wd - vw0) : 0u;
    sv.goff = ((long)(n0 + L.nb) * s.Cs * s.Hd + vh) * s.Wd + vw0;
    const long plane = (long)s.Hd * s.Wd;
    const long last = (long)(s.ncomp - 1) * s.comp_stride;  // offset of the last component in memory
    const long total = last + ((long)(s.N - 1) * s.Cs + s.C) * plane;
    sv.careful = sv.live && (sv.goff < 0 || sv.goff + last + (long)(s.C - 1) * plane + 4 > total);
    sv.fast = sv.live && !sv.careful;
    const int pg = PL::p_group(L.group), cg = PL::c_group(L.group);
    sv.tbase = sv.goff + pg * s.comp_stride + cg * plane;
    sv.c_room = s.C - cg;
    sv.p_room = s.ncomp - pg;
    return sv;
}

template <typename TS, int NCH, int P2LOG>
__device__ __forceinline__ StageVec make_stage_vec(const TileSrc& s, int n0, int h0, int w0, int NB, int HTH, int HTW,
                                                   int HP) {
    return place_stage_vec<TS, NCH, P2LOG>(s, make_stage_vec_lane<P2LOG>(NB, HTH, HTW, HP), n0, h0, w0);
}

// load e of the chunk that starts at channel c0
template <typename TS, int NCH, int P2LOG, int NT = WG_THREADS>
__device__ __forceinline__ void stage_vec_load(f32x4 (&v)[stage_loads(NCH, P2LOG, NT)], const TileSrc& s,
                                               const StageVec& sv, int c0, int e) {
    typedef StagePlanes<NCH, P2LOG, NT> PL;
    const TS* origin = static_cast<const TS*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
    // the same for every thread: scalar arithmetic, one 64-bit add per load and thread
    const long uoff = (long)PL::pe(e) * s.comp_stride + (long)(c0 + PL::ce(e)) * plane;
    // channels past the tensor meet zero filters: any finite value will do, the tensor's first bytes are safe
    // (components a real-valued tensor does not have are masked to zero by the store)
    const bool ok = sv.fast && (c0 + PL::ce(e)) < sv.c_room && PL::pe(e) < sv.p_room;
    const TS* ptr = ok ? origin + (sv.tbase + uoff) : origin;
    if constexpr (sizeof(TS) == 4) {
        typedef f32x4 f32x4_a4 __attribute__((aligned(4)));
        v[e] = *reinterpret_cast<const f32x4_a4*>(ptr);
    } else {
        // kept as loaded (8 bytes in the first two registers) and widened by staged_values() when it is stored:
        // a conversion here would wait for the load where it is issued
        typedef _Float16 f16x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
        typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f16x4 h = *reinterpret_cast<const f16x4_a2*>(ptr);
        const f32x2 bits = __builtin_bit_cast(f32x2, h);
        v[e] = f32x4{bits[0], bits[1], 0.f, 0.f};
    }
}

// the four fp32 values of a staged group
template <typename TS>
__device__ __forceinline__ f32x4 staged_values(const f32x4& raw) {
    if constexpr (sizeof(TS) == 4) {
        return raw;
    } else {
        // (the elements are copied out first: __builtin_bit_cast applied to a vector element reads element 0)
        const float lo = raw[0], hi = raw[1];
        const unsigned int a = __builtin_bit_cast(unsigned int, lo), b = __builtin_bit_cast(unsigned int, hi);
        auto half_of = [](unsigned int bits) { return (float)__builtin_bit_cast(_Float16, (unsigned short)bits); };
        return f32x4{half_of(a), half_of(a >> 16), half_of(b), half_of(b >> 16)};
    }
}

template <typename TS, int NCH, int P2LOG, int NT = WG_THREADS>
__device__ __forceinline__ void stage_vec_store(float* lds, const f32x4 (&v)[stage_loads(NCH, P2LOG, NT)],
                                                const TileSrc& s, const StageVec& sv, int c0, int HP, int HPp) {
    constexpr int G4 = StagePlanes<NCH, P2LOG, NT>::G4;
    constexpr int E = StagePlanes<NCH, P2LOG, NT>::E;
    if (sv.lpos >= HP) return;
    const unsigned int keep = sv.careful ? 0u : sv.bits;
    u32x4 mk;
#pragma unroll
    for (int i = 0; i < 4; ++i) mk[i] = (unsigned int)((int)(keep << (31 - i)) >> 31);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const bool present = (e * G4 + sv.group) / NCH < s.ncomp;
        const u32x4 w = present ? (__builtin_bit_cast(u32x4, staged_values<TS>(v[e])) & mk) : u32x4{0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4*>(lds + (e * G4 + sv.group) * HPp + sv.lpos) = w;
    }
    if (sv.careful) {
        const TS* origin = static_cast<const TS*>(s.base);
        const long plane = (long)s.Hd * s.Wd;
#pragma unroll 2
        for (int e = 0; e < E; ++e) {
            const int pc = e * G4 + sv.group;
            const int p = pc / NCH, c = c0 + pc % NCH;
            float t[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                t[i] = (c < s.C && p < s.ncomp && ((sv.bits >> i) & 1))
                           ? ldf<TS>(origin + sv.goff + p * s.comp_stride + c * plane + i)
                           : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) lds[pc * HPp + sv.lpos + i] = t[i];
        }
    }
}

// same, for LDS rows with an odd pitch (bank-conflict-free 4-byte reads down a column of rows): four 4-byte stores
template <typename TS, int NCH, int P2LOG, int NT = WG_THREADS>
__device__ __forceinline__ void stage_vec_store_scalar(float* lds, const f32x4 (&v)[stage_loads(NCH, P2LOG, NT)],
                                                       const TileSrc& s, const StageVec& sv, int c0, int HP, int pitch) {
    constexpr int G4 = StagePlanes<NCH, P2LOG, NT>::G4;
    constexpr int E = StagePlanes<NCH, P2LOG, NT>::E;
    if (sv.lpos >= HP) return;
    const unsigned int keep = sv.careful ? 0u : sv.bits;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        float* dst = lds + (e * G4 + sv.group) * pitch + sv.lpos;
        const bool present = (e * G4 + sv.group) / NCH < s.ncomp;
        const f32x4 val = staged_values<TS>(v[e]);
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = (present && ((keep >> i) & 1)) ? val[i] : 0.f;
    }
    if (sv.careful) {
        const TS* origin = static_cast<const TS*>(s.base);
        const long plane = (long)s.Hd * s.Wd;
#pragma unroll 2
        for (int e = 0; e < E; ++e) {
            const int pc = e * G4 + sv.group;
            const int p = pc / NCH, c = c0 + pc % NCH;
            float t[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                t[i] = (c < s.C && p < s.ncomp && ((sv.bits >> i) & 1))
                           ? ldf<TS>(origin + sv.goff + p * s.comp_stride + c * plane + i)
                           : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) lds[pc * pitch + sv.lpos + i] = t[i];
        }
    }
}

// Forward / input-gradient kernel.
//   workgroup = 4 waves = WCO filter sub-tiles (32 output channels each) x 4/WCO pixel ranges,
//   each wave owns NTW MFMA column tiles of 32 output pixels and all four output components.
//   A operand = packed filters straight from global memory (L2 resident, one 16/32-byte load per
//   lane and K step, prefetched one step ahead); B operand = activations from the LDS halo window.
//   MODE 16: acc[q] += W_{p^q} * (+-x_p), 16 MFMAs per K step, filters reused across the 4x4 block.
//   MODE 8 : acc[i] += R_i * L_i with the 8 lanes L_i formed in registers, 8 MFMAs per K step.
template <typename TS, int MODE, int WCO, int NTW, int CK, int P2LOG, bool VSTG>
__global__ void __launch_bounds__(WG_THREADS, (MODE == 8 || NTW == 1) ? 2 : 1) qconv_fwd_f32_kernel(const ConvArgs P0) {
    const ConvArgs P = group_view(P0);
    constexpr int NACC = (MODE == 16) ? 4 : 8;
    constexpr int WC = (MODE == 16) ? 4 : 8;  // packed filter values per lane and K step
    extern __shared__ float lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wco = wave % WCO, wpx = wave / WCO;
    const int j = lane & 31, kk = lane >> 5;

    int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int ct = bid % P.co_tiles;
    bid /= P.co_tiles;
    const int tw = bid % P.tiles_w;
    bid /= P.tiles_w;
    const int th = bid % P.tiles_h;
    const int tn = bid / P.tiles_h;
    const int n0 = tn * P.NB, ho0 = th * P.TH, wo0 = tw * P.TW;
    const int h0 = ho0 * P.sh - P.pt, w0 = wo0 * P.sw - P.pl;

    int poff[NTW];
    long oaddr[NTW];
    bool pvalid[NTW];
    const int thw = P.TH * P.TW;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        const int pix = (wpx * NTW + t) * 32 + j;
        const int nb = pix / thw, rem = pix - nb * thw;
        const int r = rem / P.TW, c = rem - r * P.TW;
        pvalid[t] = nb < P.NB && (n0 + nb) < P.in.N && (ho0 + r) < P.Hout && (wo0 + c) < P.Wout;
        poff[t] = pvalid[t] ? (nb * P.HTH + r * P.sh) * P.HTW + c * P.sw : 0;
        oaddr[t] = ((long)(n0 + nb) * P.CoutS * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c);
    }

    f32x16 acc[NTW][NACC];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][a][r] = 0.f;

    const int steps_per_chunk = P.taps * (CK / 2);
    const long nsteps = (long)P.nchunks * steps_per_chunk;
    const float* wptr = static_cast<const float*>(P.wpk) + ((long)(ct * WCO + wco) * nsteps * 64 + lane) * WC;
    // packed filters: register pipeline two K steps deep (an L2 hit takes longer than one step's MFMAs)
    f32x4 wcur[WC / 4], wnext[WC / 4], wnext2[WC / 4];
#pragma unroll
    for (int v = 0; v < WC / 4; ++v) {
        wcur[v] = *reinterpret_cast<const f32x4*>(wptr + 4 * v);
        wnext[v] = *reinterpret_cast<const f32x4*>(wptr + (nsteps > 1 ? 1 : 0) * (64 * WC) + 4 * v);
    }

    long step = 0;
    const long cpitch = (long)CK * P.HPp;  // LDS floats between components
    // 2^P2LOG window positions, 256 >> P2LOG thread groups sharing the 4*CK planes of a chunk
    const StagePos sp = make_stage_pos<P2LOG>(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW);
    const StageVec sv = make_stage_vec<TS, CK, P2LOG>(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW, P.HP);
    constexpr int EV = (CK << P2LOG) >> 8;  // vector loads per thread and chunk
    float stage[VSTG ? 1 : ((4 * CK) >> (8 - P2LOG))];
    f32x4 stagev[VSTG ? EV : 1];
    if constexpr (VSTG) {
#pragma unroll
        for (int e = 0; e < EV; ++e) stage_vec_load<TS, CK, P2LOG>(stagev, P.in, sv, 0, e);
    } else {
        stage_load<TS, CK, P2LOG>(stage, P.in, sp, 0);
    }
    PHX_PHASES_BEGIN(6)
    for (int chunk = 0; chunk < P.nchunks; ++chunk) {
        __syncthreads();
        PHX_STAMP(0)
        if constexpr (VSTG) stage_vec_store<TS, CK, P2LOG>(lds, stagev, P.in, sv, chunk * CK, P.HP, P.HPp);
        else stage_store<CK, P2LOG, float>(lds, stage, sp, P.HP, P.HPp);
        PHX_STAMP(1)
        __syncthreads();
        PHX_STAMP(2)
        // next chunk's global loads fly while this chunk is multiplied; the vector form deals them out over
        // the K steps of the first tap (a wave that issues them back to back stalls until all are taken)
        const bool more = chunk + 1 < P.nchunks;
        if constexpr (!VSTG) {
            if (more) stage_load<TS, CK, P2LOG>(stage, P.in, sp, (chunk + 1) * CK);
        }
        PHX_STAMP(3)
        int kh = 0, kw = 0;
        for (int tap = 0; tap < P.taps; ++tap) {
            const int tapoff = kh * P.dh * P.HTW + kw * P.dw;
#pragma unroll
            for (int cp = 0; cp < CK / 2; ++cp) {
                if constexpr (VSTG) {
                    constexpr int LPS = (EV + CK / 2 - 1) / (CK / 2);  // loads per K step
                    if (more && tap == 0) {
#pragma unroll
                        for (int e = cp * LPS; e < (cp + 1) * LPS && e < EV; ++e)
                            stage_vec_load<TS, CK, P2LOG>(stagev, P.in, sv, (chunk + 1) * CK, e);
                    }
                }
                const long nxt = (step + 2 < nsteps) ? step + 2 : nsteps - 1;
#pragma unroll
                for (int v = 0; v < WC / 4; ++v)
                    wnext2[v] = *reinterpret_cast<const f32x4*>(wptr + nxt * (64 * WC) + 4 * v);
                const float* xb = lds + (2 * cp + kk) * P.HPp + tapoff;
#pragma unroll
                for (int t = 0; t < NTW; ++t) {
                    float x[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) x[p] = xb[p * cpitch + poff[t]];
                    if constexpr (MODE == 16) {
                        float nx[4];
#pragma unroll
                        for (int p = 0; p < 4; ++p) nx[p] = -x[p];
#pragma unroll
                        for (int p = 0; p < 4; ++p)
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                                acc[t][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(wcur[0][p ^ q], qneg(p, q) ? nx[p] : x[p],
                                                                                 acc[t][q], 0, 0, 0);
                    } else {
                        float L[8];
                        lanes_left(x, L);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(wcur[i >> 2][i & 3], L[i], acc[t][i], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int v = 0; v < WC / 4; ++v) {
                    wcur[v] = wnext[v];
                    wnext[v] = wnext2[v];
                }
                ++step;
            }
            if (++kw == P.Kw) { kw = 0; ++kh; }
        }
        PHX_STAMP(4)
    }

    // epilogue: fold lanes (8-product), add bias, store NCHW with components on the batch axis
    conv_epilogue<TS, MODE, NTW, NACC>(P, acc, (ct * WCO + wco) * 32 + 4 * kk, oaddr, pvalid);
    PHX_STAMP(5)
    PHX_PHASES_REPORT("fwd_f32: barrier / store / barrier / load issue / mfma / epilogue", 6)
}

// Filter packing for the kernel above.  One value group per (32-channel filter tile, K step, lane):
//   lane = (row = lane % 32, kk = lane / 32), output channel = tile*32 + row,
//   K step = ((chunk * taps) + tap) * 4 + cp, input channel = chunk*8 + 2*cp + kk.
//   MODE 16: the four filter components; MODE 8: the eight right-operand lanes R_i.
//   MAP_DGRAD swaps the channel roles, mirrors the taps and conjugates the filter (MODE 8: before its
//   lanes are formed), so that dx = g (x) conj(w) runs through the forward kernel.
// Filter element (r, o, i, kh, kw) lives at r*wcs + o*so + i*si + kh*skh + kw*skw.
struct PackArgs {
    const void* w;
    void* out;
    long wcs, so, si, skh, skw;
    int Co, Ci;       // filter dims of the convolution (not of the correlation being run)
    int Kh, Kw;       // taps of the correlation being run
    int khm, khs, kwm, kws;  // input gradient: tap (u, v) of the correlation is filter tap (khm - u*khs, kwm - v*kws)
    int rows, red;    // correlation: output channels (rows) and reduced channels
    int row_tiles, nchunks;
    int groups;       // grid rows: the groups packed by this one launch (1 otherwise)
    long g_w, g_out;  // bytes from one group's filter / packed image to the next group's
};

__device__ __forceinline__ PackArgs group_view(const PackArgs& P0) {
    PackArgs P = P0;
    P.w = group_shift(P0.w, P0.g_w);
    P.out = group_shift(P0.out, P0.g_out);
    return P;
}

// (the packing bodies take the thread's first index and the stride of its loop, so that one launch can also pack
// several filter images side by side: pack_jobs_kernel)
template <typename TS, int MODE, int MAP>
__device__ __forceinline__ void pack_filters_f32_body(const PackArgs& P, long first, long stride) {
    constexpr int WC = (MODE == 16) ? 4 : 8;
    const int taps = P.Kh * P.Kw;
    const long total = (long)P.row_tiles * P.nchunks * taps * 4 * 64;
    const TS* w = static_cast<const TS*>(P.w);
    for (long idx = first; idx < total; idx += stride) {
        const int lane = idx & 63;
        long s = idx >> 6;
        const int cp = s & 3;
        s >>= 2;
        const int tap = s % taps;
        s /= taps;
        const int chunk = s % P.nchunks;
        const int tile = s / P.nchunks;
        const int row = tile * 32 + (lane & 31);
        const int red = chunk * F32_CK + 2 * cp + (lane >> 5);
        int kh = tap / P.Kw, kw = tap - kh * P.Kw;
        float wv[4] = {0.f, 0.f, 0.f, 0.f};
        if (row < P.rows && red < P.red) {
            int o = row, i = red;
            if (MAP == MAP_DGRAD) {
                o = red;
                i = row;
                kh = P.khm - kh * P.khs;
                kw = P.kwm - kw * P.kws;
            }
            const long off = o * P.so + i * P.si + kh * P.skh + kw * P.skw;
#pragma unroll
            for (int r = 0; r < 4; ++r) wv[r] = ldf<TS>(w + r * P.wcs + off);
        }
        float* dst = static_cast<float*>(P.out) + idx * WC;
        if (MAP == MAP_DGRAD) {
#pragma unroll
            for (int r = 1; r < 4; ++r) wv[r] = -wv[r];
        }
        if constexpr (MODE == 16) {
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[r] = wv[r];
        } else {
            float R[8];
            lanes_right(wv, R);
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[i] = R[i];
        }
    }
}

template <typename TS, int MODE, int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_f32_kernel(const PackArgs P0) {
    const PackArgs P = group_view(P0);
    pack_filters_f32_body<TS, MODE, MAP>(P, (long)blockIdx.x * blockDim.x + threadIdx.x, (long)gridDim.x * blockDim.x);
}

// ---------------------------------------------------------------------------------------------
// Filter gradient.  GEMM view: rows = output channels (A operand = output gradient), columns =
// input channels (B operand = shifted input), reduction over batch and output pixels.
//   grid.x = (64-channel row tile, 64-channel column tile), grid.y = tap group (one filter row kh
//   and up to TPW adjacent kw), grid.z = split of the reduction; each workgroup walks its share of
//   the pixel tiles, stages gradient and input windows in LDS and accumulates in registers.
//   wave = (32 rows) x (32 columns) x TPW taps x 4 components (MODE 16) or 8 lanes (MODE 8).
//   Partial sums go to workspace[z] and are summed in a fixed order by reduce_wgrad_kernel.
// ---------------------------------------------------------------------------------------------
struct WgradArgs {
    TileSrc x, g;
    float* partial;     // [Z][taps][4][CoP][CiP]
    int Kh, Kw, sh, sw, dh, dw, pt, pl;
    int NB, TH, TW;     // reduction tile: images x output rows x output columns
    int KP, KPp, HPp;   // pixels per tile (even), LDS pitches (odd) of gradient / input windows
    int HTH, HTWmax;
    int HPx;            // input window size for a full tap group (<= 32, like KP)
    int tiles_n, tiles_h, tiles_w;
    int co_tiles, ci_tiles, CoP, CiP;
    int groups_per_row; // tap groups per filter row
    int cpr, nchunks, ntiles, zsplit;  // fp16 kernel: 8-pixel chunks per output row / in total, pixel tiles, reduction slices
    int flat, rows;                    // fp16 kernel: chunk list over whole planes (rows = 1) or over the rows of an image
    int groups;                        // grid rows: the groups of a grouped convolution run by this one launch (1 otherwise)
    long g_x, g_g, g_partial;          // bytes from one group's input / gradient / partial sums to the next group's
};

__device__ __forceinline__ WgradArgs group_view(const WgradArgs& P0) {
    WgradArgs P = P0;
    P.x.base = group_shift(P0.x.base, P0.g_x);
    P.g.base = group_shift(P0.g.base, P0.g_g);
    P.partial = static_cast<float*>(group_shift(static_cast<void*>(P0.partial), P0.g_partial));
    return P;
}

//   KSETS = 2: eight waves, two per SIMD (while one forms lanes or waits for LDS, the other's matrix
//   instructions run); the second set of four takes the odd K steps of every tile into accumulators of its
//   own, which go to a reduction slice of their own (slice z*KSETS + set).  Every thread stages half as much.
template <typename TS, int MODE, int TPW, bool VEC, int KSETS>
__global__ void __launch_bounds__(WG_THREADS * KSETS) qconv_wgrad_f32_kernel(const WgradArgs P0) {
    const WgradArgs P = group_view(P0);
    constexpr int CT = 64;
    constexpr int NT = WG_THREADS * KSETS;
    constexpr int EV = 8 / KSETS;  // vector loads per thread, tile and operand
    static_assert(KSETS == 1 || VEC, "the K split is written for the vector staging");
    constexpr int NACC = (MODE == 16) ? 4 : 8;
    extern __shared__ float lds[];
    float* gl = lds;                           // [4][CT][KPp]
    float* xl = lds + 4 * CT * P.KPp;          // [4][CT][HPp]
    int* poff = reinterpret_cast<int*>(xl + 4 * CT * P.HPp);  // [KP]

    const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, kset = tid >> 8;
    const int wco = wave & 1, wci = wave >> 1;
    const int m = lane & 31, kk = lane >> 5;
    // workgroups that share a reduction slice read the same gradient / input tiles: keep them on one XCD
    int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int cot = bid % P.co_tiles;  bid /= P.co_tiles;
    const int cit = bid % P.ci_tiles;  bid /= P.ci_tiles;
    const int ngroups = P.groups_per_row * P.Kh;
    const int grp = bid % ngroups;
    const int zi = bid / ngroups;
    const int kh = grp / P.groups_per_row;
    const int kw0 = (grp % P.groups_per_row) * TPW;
    const int nkw = (P.Kw - kw0 < TPW) ? P.Kw - kw0 : TPW;
    const int HTWx = (P.TW - 1) * P.sw + (nkw - 1) * P.dw + 1;
    const int HTW = VEC ? ((HTWx + 3) & ~3) : HTWx;  // vector staging: whole groups of 4 positions per window row

    const int thw = P.TH * P.TW;
    for (int k = tid; k < P.KP; k += NT) {
        const int nb = k / thw, rem = k - nb * thw;
        const int r = rem / P.TW, c = rem - r * P.TW;
        poff[k] = (nb < P.NB) ? (nb * P.HTH + r * P.sh) * HTW + c * P.sw : 0;
    }

    f32x16 acc[TPW][NACC];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][a][r] = 0.f;

    const int ntiles = P.tiles_n * P.tiles_h * P.tiles_w;
    const long gcp = (long)CT * P.KPp, xcp = (long)CT * P.HPp;
    constexpr int P2LOG = 5;  // 32 window positions x 8 plane groups (vector form: 8 groups of 4 x 32 plane groups)
    float sg[VEC ? 1 : 32], sx[VEC ? 1 : 32];
    f32x4 vg[VEC ? EV : 1], vx[VEC ? EV : 1];
    StagePos spg, spx;
    StageVec svg, svx;
    // tiles zi, zi + zsplit, ... as (image group, row tile, column tile): stepped with carries, no division per tile
    int tw = zi % P.tiles_w, th = (zi / P.tiles_w) % P.tiles_h, tn = zi / (P.tiles_w * P.tiles_h);
    const int step_w = P.zsplit % P.tiles_w, step_h = (P.zsplit / P.tiles_w) % P.tiles_h;
    const int step_n = P.zsplit / (P.tiles_w * P.tiles_h);
    const StageVecLane lane_g = make_stage_vec_lane<P2LOG>(P.NB, P.TH, P.TW, P.NB * thw);
    const StageVecLane lane_x = make_stage_vec_lane<P2LOG>(P.NB, P.HTH, HTW, P.NB * P.HTH * HTW);
    auto locate = [&]() {  // the staging positions of tile (tn, th, tw); then steps to the workgroup's next tile
        const int n0 = tn * P.NB, ho0 = th * P.TH, wo0 = tw * P.TW;
        const int h0x = ho0 * P.sh - P.pt + kh * P.dh, w0x = wo0 * P.sw - P.pl + kw0 * P.dw;
        // gradient window: TH x TW output pixels, no halo; pixels beyond the tensor are zero and
        // therefore contribute nothing whatever the input window holds there
        if constexpr (VEC) {
            svg = place_stage_vec<TS, CT, P2LOG, NT>(P.g, lane_g, n0, ho0, wo0);
            svx = place_stage_vec<TS, CT, P2LOG, NT>(P.x, lane_x, n0, h0x, w0x);
        } else {
            spg = make_stage_pos<P2LOG>(P.g, n0, ho0, wo0, P.NB, P.TH, P.TW);
            spx = make_stage_pos<P2LOG>(P.x, n0, h0x, w0x, P.NB, P.HTH, HTW);
        }
        tw += step_w;
        if (tw >= P.tiles_w) { tw -= P.tiles_w; ++th; }
        th += step_h;
        if (th >= P.tiles_h) { th -= P.tiles_h; ++tn; }
        tn += step_n;
    };
    auto issue = [&]() {
        locate();
        if constexpr (VEC) {
#pragma unroll
            for (int e = 0; e < EV; ++e) {
                stage_vec_load<TS, CT, P2LOG, NT>(vg, P.g, svg, cot * CT, e);
                stage_vec_load<TS, CT, P2LOG, NT>(vx, P.x, svx, cit * CT, e);
            }
        } else {
            stage_load<TS, CT, P2LOG>(sg, P.g, spg, cot * CT);
            stage_load<TS, CT, P2LOG>(sx, P.x, spx, cit * CT);
        }
    };
    const int HPx = P.NB * P.HTH * HTW;
    if (zi < ntiles) issue();
    PHX_PHASES_BEGIN(5)
    for (int tile = zi; tile < ntiles; tile += P.zsplit) {
        PHX_STAMP(4)
        __syncthreads();
        PHX_STAMP(0)
        if constexpr (VEC) {
            stage_vec_store_scalar<TS, CT, P2LOG, NT>(gl, vg, P.g, svg, cot * CT, P.NB * thw, P.KPp);
            stage_vec_store_scalar<TS, CT, P2LOG, NT>(xl, vx, P.x, svx, cit * CT, HPx, P.HPp);
        } else {
            stage_store<CT, P2LOG, float>(gl, sg, spg, P.NB * thw, P.KPp);
            stage_store<CT, P2LOG, float>(xl, sx, spx, HPx, P.HPp);
        }
        if (P.KP != P.NB * thw)  // odd pixel count: the padding column of the gradient window must be zero
            for (int c = tid; c < 4 * CT; c += NT) gl[c * P.KPp + P.KP - 1] = 0.f;
        // Threads without a window position skip the stores and, with them, the waits for their loads.  Stated
        // here for every path, it lets the next tile's loads be issued below without a wait in front of each
        // (they reuse the staging registers).
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        PHX_STAMP(1)
        __syncthreads();
        PHX_STAMP(2)
        const bool more = tile + P.zsplit < ntiles;
        if constexpr (VEC) {
            if (more) locate();
        } else {
            if (more) issue();
        }
        PHX_STAMP(3)
        const float* ga = gl + (wco * 32 + m) * P.KPp + kk;
        const float* xb = xl + (wci * 32 + m) * P.HPp;
        // one K step (two pixels): gradient values g of the wave's 32 output channels, input values x[t] of its
        // 32 input channels under each tap
        auto products = [&](const float (&g)[4], const float (&xs)[TPW][4]) {
            float G[8];
            if constexpr (MODE == 8) lanes_grad(g, G, 0.5f);
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
                if (t < nkw) {
                    const float(&x)[4] = xs[t];
                    if constexpr (MODE == 16) {
                        float nx[4];
#pragma unroll
                        for (int p = 0; p < 4; ++p) nx[p] = -x[p];
#pragma unroll
                        for (int p = 0; p < 4; ++p)
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                                acc[t][p ^ q] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[q], qneg(p, q) ? nx[p] : x[p],
                                                                                     acc[t][p ^ q], 0, 0, 0);
                    } else {
                        float L[8];
                        lanes_left(x, L);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(G[i], L[i], acc[t][i], 0, 0, 0);
                    }
                }
            }
        };
        if constexpr (VEC) {
            // At most 16 K steps, unrolled: the next tile's global loads are dealt over the first eight (a wave
            // that issues them back to back stalls until the memory pipeline has taken them all), and each step's
            // LDS reads (the pixel's window offset, then the values) are issued one step ahead of the matrix
            // products that use them.
            // (a wave of set s takes the steps s, s + KSETS, ...)
            constexpr int NJ = 16 / KSETS;
            auto fetch = [&](int j, float (&g)[4], float (&xs)[TPW][4]) {
                const int ksi = j * KSETS + kset;
                const int ks = (2 * ksi < P.KP) ? 2 * ksi : P.KP - 2;
#pragma unroll
                for (int q = 0; q < 4; ++q) g[q] = ga[q * gcp + ks];
                const int pk = poff[ks + kk];
#pragma unroll
                for (int t = 0; t < TPW; ++t) {
                    const int tt = (t < nkw) ? t : 0;
#pragma unroll
                    for (int p = 0; p < 4; ++p) xs[t][p] = xb[p * xcp + pk + tt * P.dw];
                }
            };
            float gc[4], xc[TPW][4];
            fetch(0, gc, xc);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (j == NJ / 2) { PHX_STAMP(5) }
                if (more && j < EV) {
                    stage_vec_load<TS, CT, P2LOG, NT>(vg, P.g, svg, cot * CT, j);
                    stage_vec_load<TS, CT, P2LOG, NT>(vx, P.x, svx, cit * CT, j);
                }
                float gn[4], xn[TPW][4];
                if (j + 1 < NJ) fetch(j + 1, gn, xn);
                if (2 * (j * KSETS + kset) < P.KP) products(gc, xc);
                if (j + 1 < NJ) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) gc[q] = gn[q];
#pragma unroll
                    for (int t = 0; t < TPW; ++t)
#pragma unroll
                        for (int q = 0; q < 4; ++q) xc[t][q] = xn[t][q];
                }
            }
        } else {
            for (int ks = 0; ks < P.KP; ks += 2) {
                float g[4], xs[TPW][4];
#pragma unroll
                for (int q = 0; q < 4; ++q) g[q] = ga[q * gcp + ks];
                const int pk = poff[ks + kk];
#pragma unroll
                for (int t = 0; t < TPW; ++t) {
                    const int tt = (t < nkw) ? t : 0;
#pragma unroll
                    for (int p = 0; p < 4; ++p) xs[t][p] = xb[p * xcp + pk + tt * P.dw];
                }
                products(g, xs);
            }
        }
    }

    PHX_STAMP(4)
    PHX_PHASES_REPORT("wgrad_f32: barrier / store / barrier / locate / products, second half / products, first half", 6)
    // partial[z][tap][r][co][ci]
    const int taps = P.Kh * P.Kw;
    const long tap_stride = 4L * P.CoP * P.CiP;
    float* dst = P.partial + ((long)zi * KSETS + kset) * taps * tap_stride;
    const int ci = cit * CT + wci * 32 + m;
    const int co_base = cot * CT + wco * 32 + 4 * kk;
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        if (t >= nkw) continue;
        float* d = dst + (long)(kh * P.Kw + kw0 + t) * tap_stride;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int co = co_base + 8 * (e >> 2) + (e & 3);
            float y[4];
            if constexpr (MODE == 16) {
#pragma unroll
                for (int r = 0; r < 4; ++r) y[r] = acc[t][r][e];
            } else {
                float l[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) l[i] = acc[t][i][e];
                merge_right_grad(l, y);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) d[((long)r * P.CoP + co) * P.CiP + ci] = y[r];
        }
    }
}

struct ReduceArgs {
    const float* partial;
    void* dw;
    long wcs, so, si, skh, skw;
    int Z, Co, Ci, Kh, Kw, CoP, CiP;
    int groups;              // grid rows: the groups reduced by this one launch (1 otherwise)
    long g_partial, g_dw;    // bytes from one group's partial sums / filter gradient to the next group's
};

__device__ __forceinline__ ReduceArgs group_view(const ReduceArgs& P0) {
    ReduceArgs P = P0;
    P.partial = static_cast<const float*>(group_shift(static_cast<const void*>(P0.partial), P0.g_partial));
    P.dw = group_shift(P0.dw, P0.g_dw);
    return P;
}

// dw(r, co, ci, kh, kw) = sum_z partial[z][tap][r][co][ci].  A thread owns four consecutive input channels of
// one (tap, component, output channel) -- 16-byte loads, the padded row length CiP is a multiple of 4.  The
// threads of a workgroup form nsl z-slices (8 where there are that many partials, else 4, 2 or 1) over
// WG_THREADS / nsl such groups; slice s adds partials s, s + nsl, ..., then the slices are added in a fixed
// order, so the result does not depend on scheduling.
__host__ __device__ inline int reduce_slices(int Z) { return Z >= 7 ? 8 : Z >= 4 ? 4 : Z >= 2 ? 2 : 1; }

template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) reduce_wgrad_kernel(const ReduceArgs P0) {
    const ReduceArgs P = group_view(P0);
    __shared__ f32x4 part[WG_THREADS];
    const int taps = P.Kh * P.Kw;
    const int ci4s = (P.Ci + 3) >> 2;
    const long total = 4L * taps * P.Co * ci4s;
    const long zstride = 4L * taps * P.CoP * P.CiP;
    TS* dw = static_cast<TS*>(P.dw);
    const int nsl = reduce_slices(P.Z), groups = WG_THREADS / nsl;
    const int lane = threadIdx.x % groups, slice = threadIdx.x / groups;
    const long idx = (long)blockIdx.x * groups + lane;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    int ci = 0, co = 0, r = 0, tap = 0;
    if (idx < total) {
        ci = (int)(idx % ci4s) * 4;
        long t = idx / ci4s;
        co = t % P.Co;
        t /= P.Co;
        r = t & 3;
        tap = t >> 2;
        const float* src = P.partial + (((long)tap * 4 + r) * P.CoP + co) * P.CiP + ci;
        f32x4 s0 = sum, s1 = sum, s2 = sum, s3 = sum;
        int z = slice;
        for (; z + 3 * nsl < P.Z; z += 4 * nsl) {
            s0 += *reinterpret_cast<const f32x4*>(src + (long)z * zstride);
            s1 += *reinterpret_cast<const f32x4*>(src + (long)(z + nsl) * zstride);
            s2 += *reinterpret_cast<const f32x4*>(src + (long)(z + 2 * nsl) * zstride);
            s3 += *reinterpret_cast<const f32x4*>(src + (long)(z + 3 * nsl) * zstride);
        }
        for (; z < P.Z; z += nsl) s0 += *reinterpret_cast<const f32x4*>(src + (long)z * zstride);
        sum = (s0 + s1) + (s2 + s3);
    }
    part[threadIdx.x] = sum;
    __syncthreads();
    if (slice == 0 && idx < total) {
        f32x4 v = part[lane];
        for (int k = 1; k < nsl; ++k) v += part[k * groups + lane];
        const int kh = tap / P.Kw, kw = tap - kh * P.Kw;
        TS* dst = dw + r * P.wcs + co * P.so + ci * P.si + kh * P.skh + kw * P.skw;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (ci + e < P.Ci) stf<TS>(dst + e * P.si, v[e]);
    }
}

}  // namespace phx
