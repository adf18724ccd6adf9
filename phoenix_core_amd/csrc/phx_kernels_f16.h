// fp16-MFMA kernels (v_mfma_f32_32x32x16_f16, fp32 accumulation) for fp16 tensors: quaternion
// convolution forward / input-gradient in the 16-product and the factorized 8-product formulation.
#pragma once

#include "phx_kernels_f32.h"

namespace phx {

// Staged layout: unit u = p*2 + kp (component p, 8-channel pack kp) holds one 16-byte entry per
// window position, lds[u*pitch + pos] = {x_p[c0 + kp*8 + 0..7]} at that position.  NCHW keeps the
// channels of one pixel HW elements apart, so the transposition happens here: every thread gathers
// the 8 channels of a pack for its own position and writes them with one 16-byte LDS store; the
// MFMA B operand (lane = pixel, 8 consecutive K values) is then a single aligned 16-byte LDS read.
template <int P2LOG>
__device__ __forceinline__ void stage_load16(f16x8 (&v)[8 >> (8 - P2LOG)], const TileSrc& s, const StagePos& sp,
                                             int c0) {
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = 8 / G;
    const _Float16* origin = static_cast<const _Float16*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int u = e * G + sp.group;
        const int p = u >> 1, kp = u & 1;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = c0 + kp * 8 + i;
            const bool ok = sp.valid && c < s.C;
            const _Float16* ptr = ok ? origin + sp.goff + p * s.comp_stride + (long)c * plane : zero_ptr<_Float16>();
            v[e][i] = *ptr;
        }
    }
}

template <int P2LOG>
__device__ __forceinline__ void stage_store16(f16x8* dst, const f16x8 (&v)[8 >> (8 - P2LOG)], const StagePos& sp,
                                              int HP, int pitch) {
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = 8 / G;
    if (sp.pos < HP) {
#pragma unroll
        for (int e = 0; e < E; ++e) dst[(e * G + sp.group) * pitch + sp.pos] = v[e];
    }
}

// Pair staging: when image rows have an even length (and no zero insertion is in play) the window
// is widened to start at an even column, so that two horizontally adjacent positions are one aligned
// 32-bit word in every channel plane.  A thread then gathers the 8 channels of a pack for TWO
// positions with 8 dword loads, splits low/high halves with 8 byte-permutes and writes two 16-byte
// LDS entries: half the load instructions, each twice as wide.  128 pair positions x 2 thread
// groups; a group walks 4 of the 8 (component, pack) units.
struct StagePairPos {
    long goff;   // element offset of the pair's first position (even)
    int pos;     // window position of the pair's first element
    int group;
    bool valid, inwin;
};

__device__ __forceinline__ StagePairPos make_stage_pairpos(const TileSrc& s, int n0, int h0, int w0e, int NB, int HTH,
                                                           int HTWe) {
    StagePairPos sp;
    const int pp = threadIdx.x & 127;
    sp.group = threadIdx.x >> 7;
    const int rowpairs = HTWe >> 1;
    const int hw = HTH * rowpairs;
    const int nb = pp / hw, rem = pp - nb * hw;
    const int hr = rem / rowpairs, hcp = rem - hr * rowpairs;
    const int vh = h0 + hr, vw = w0e + 2 * hcp;
    sp.inwin = nb < NB;
    sp.pos = (nb * HTH + hr) * HTWe + 2 * hcp;
    const bool ok = sp.inwin && (n0 + nb) < s.N && vh >= 0 && vh < s.Hd && vw >= 0 && vw + 1 < s.Wd;
    sp.valid = ok;
    sp.goff = ok ? ((long)(n0 + nb) * s.C * s.Hd + vh) * s.Wd + vw : 0;
    return sp;
}

__device__ __forceinline__ void stage_load16_pairs(unsigned int (&d)[4][8], const TileSrc& s, const StagePairPos& sp,
                                                   int c0) {
    const _Float16* origin = static_cast<const _Float16*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int u = e * 2 + sp.group;
        const int p = u >> 1, kp = u & 1;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = c0 + kp * 8 + i;
            const bool ok = sp.valid && c < s.C;
            const _Float16* ptr = ok ? origin + sp.goff + p * s.comp_stride + (long)c * plane : zero_ptr<_Float16>();
            d[e][i] = *reinterpret_cast<const unsigned int*>(ptr);
        }
    }
}

__device__ __forceinline__ void stage_store16_pairs(f16x8* dst, const unsigned int (&d)[4][8], const StagePairPos& sp,
                                                    int pitch) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    if (sp.inwin) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            u32x4 lo, hi;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                lo[m] = __builtin_amdgcn_perm(d[e][2 * m + 1], d[e][2 * m], 0x05040100u);
                hi[m] = __builtin_amdgcn_perm(d[e][2 * m + 1], d[e][2 * m], 0x07060302u);
            }
            f16x8* q = dst + (e * 2 + sp.group) * pitch + sp.pos;
            q[0] = __builtin_bit_cast(f16x8, lo);
            q[1] = __builtin_bit_cast(f16x8, hi);
        }
    }
}

// Same tiling as qconv_fwd_f32_kernel: 4 waves = WCO filter sub-tiles (32 output channels) x
// 4/WCO pixel ranges, NTW column tiles of 32 pixels per wave, all four output components per wave.
// One K step is a whole 16-channel chunk at one filter tap.
//   MODE 16: 16 MFMAs per step and column tile, the four filter components reused across the
//            4x4 block, negative entries by flipping the sign bits of the activation operand.
//   MODE 8 : 8 MFMAs per step and column tile on lanes formed with packed fp16 adds.
template <int MODE, int MAP, int WCO, int NTW, int P2LOG>
__global__ void __launch_bounds__(WG_THREADS, (MODE == 8 || NTW == 1) ? 2 : 1) qconv_fwd_f16_kernel(const ConvArgs P) {
    constexpr int CK = F16_CK;
    constexpr int WPX = 4 / WCO;
    constexpr int NACC = (MODE == 16) ? 4 : 8;
    constexpr int WC = (MODE == 16) ? 4 : 8;  // packed 16-byte filter vectors per lane and K step
    extern __shared__ f16x8 lds16[];

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
        oaddr[t] = ((long)(n0 + nb) * P.Cout * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c);
    }

    f32x16 acc[NTW][NACC];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][a][r] = 0.f;

    const long nsteps = (long)P.nchunks * P.taps;
    const f16x8* wptr = static_cast<const f16x8*>(P.wpk) + ((long)(ct * WCO + wco) * nsteps * 64 + lane) * WC;
    f16x8 wcur[WC], wnext[WC];
#pragma unroll
    for (int v = 0; v < WC; ++v) wcur[v] = wptr[v];

    long step = 0;
    const StagePos sp = make_stage_pos<P2LOG>(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW);
    f16x8 stage[8 >> (8 - P2LOG)];
    stage_load16<P2LOG>(stage, P.in, sp, 0);
    for (int chunk = 0; chunk < P.nchunks; ++chunk) {
        __syncthreads();
        stage_store16<P2LOG>(lds16, stage, sp, P.HP, P.HPp);
        __syncthreads();
        if (chunk + 1 < P.nchunks) stage_load16<P2LOG>(stage, P.in, sp, (chunk + 1) * CK);
        int kh = 0, kw = 0;
        for (int tap = 0; tap < P.taps; ++tap) {
            const int tapoff = kh * P.dh * P.HTW + kw * P.dw;
            const long nxt = (step + 1 < nsteps) ? step + 1 : step;
#pragma unroll
            for (int v = 0; v < WC; ++v) wnext[v] = wptr[nxt * (64 * WC) + v];
            const f16x8* xb = lds16 + kk * P.HPp + tapoff;
#pragma unroll
            for (int t = 0; t < NTW; ++t) {
                f16x8 x[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) x[p] = xb[p * 2 * P.HPp + poff[t]];
                if constexpr (MODE == 16) {
                    f16x8 nx[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) nx[p] = neg8(x[p]);
#pragma unroll
                    for (int p = 0; p < 4; ++p)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            acc[t][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wcur[p ^ q], qneg(p, q) ? nx[p] : x[p],
                                                                               acc[t][q], 0, 0, 0);
                } else {
                    f16x8 L[8];
                    if constexpr (MAP == MAP_FWD) lanes_left(x, L);
                    else lanes_grad(x, L, (_Float16)0.5f);
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wcur[i], L[i], acc[t][i], 0, 0, 0);
                }
            }
#pragma unroll
            for (int v = 0; v < WC; ++v) wcur[v] = wnext[v];
            ++step;
            if (++kw == P.Kw) { kw = 0; ++kh; }
        }
    }

    _Float16* out = static_cast<_Float16*>(P.out);
    const _Float16* bias = static_cast<const _Float16*>(P.bias);
    const long plane = (long)P.Hout * P.Wout;
    const int co_base = (ct * WCO + wco) * 32 + 4 * kk;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        if (!pvalid[t]) continue;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int co = co_base + 8 * (r >> 2) + (r & 3);
            float y[4];
            if constexpr (MODE == 16) {
#pragma unroll
                for (int q = 0; q < 4; ++q) y[q] = acc[t][q][r];
            } else {
                float l[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) l[i] = acc[t][i][r];
                if constexpr (MAP == MAP_FWD) merge_output(l, y);
                else merge_left_grad(l, y);
            }
            if (co < P.Cout) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float v = y[q];
                    if (bias) v += (float)bias[q * P.Cout + co];
                    out[q * P.out_cs + oaddr[t] + co * plane] = (_Float16)v;
                }
            }
        }
    }
}

// Filter packing for the kernel above: one group of WC 16-byte vectors per (32-channel filter
// tile, K step, lane); lane = (row = lane % 32, kk = lane / 32), K step = chunk*taps + tap,
// vector element i = reduced channel chunk*16 + kk*8 + i.  MODE 16: the four filter components
// (conjugated for MAP_DGRAD); MODE 8: the eight right-operand lanes, formed in fp32 and rounded once.
template <int MODE, int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_f16_kernel(const PackArgs P) {
    constexpr int WC = (MODE == 16) ? 4 : 8;
    const int taps = P.Kh * P.Kw;
    const long total = (long)P.row_tiles * P.nchunks * taps * 64;
    const _Float16* w = static_cast<const _Float16*>(P.w);
    f16x8* outv = reinterpret_cast<f16x8*>(P.out);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int lane = idx & 63;
        long s = idx >> 6;
        const int tap = s % taps;
        s /= taps;
        const int chunk = s % P.nchunks;
        const int tile = s / P.nchunks;
        const int row = tile * 32 + (lane & 31);
        int kh = tap / P.Kw, kw = tap - kh * P.Kw;
        if (MAP == MAP_DGRAD) {
            kh = P.Kh - 1 - kh;
            kw = P.Kw - 1 - kw;
        }
        f16x8 vec[WC];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int red = chunk * F16_CK + (lane >> 5) * 8 + i;
            float wv[4] = {0.f, 0.f, 0.f, 0.f};
            if (row < P.rows && red < P.red) {
                const int o = (MAP == MAP_DGRAD) ? red : row;
                const int in = (MAP == MAP_DGRAD) ? row : red;
                const long off = o * P.so + in * P.si + kh * P.skh + kw * P.skw;
#pragma unroll
                for (int r = 0; r < 4; ++r) wv[r] = (float)w[r * P.wcs + off];
            }
            if constexpr (MODE == 16) {
                const float sgn = (MAP == MAP_DGRAD) ? -1.f : 1.f;
                vec[0][i] = (_Float16)wv[0];
                vec[1][i] = (_Float16)(sgn * wv[1]);
                vec[2][i] = (_Float16)(sgn * wv[2]);
                vec[3][i] = (_Float16)(sgn * wv[3]);
            } else {
                float R[8];
                lanes_right(wv, R);
#pragma unroll
                for (int l = 0; l < 8; ++l) vec[l][i] = (_Float16)R[l];
            }
        }
#pragma unroll
        for (int v = 0; v < WC; ++v) outv[idx * WC + v] = vec[v];
    }
}

// ---------------------------------------------------------------------------------------------
// Forward / input-gradient, 16-product, both operands through LDS.
// The K loop runs over steps (16-channel chunk, tap).  Filters are packed per call into the exact
// LDS image of a group of TG consecutive steps of one chunk and copied global->LDS by the direct
// (register-less) load path, double buffered: the copy of group i+1 is issued before group i is
// multiplied.  Activations are staged per chunk as in qconv_fwd_f16_kernel, their global loads
// issued one chunk ahead into registers.  The inner loop therefore holds only LDS reads and MFMAs.
//   packed filters: [filter tile of WCO*32 channels][group][tap in group][wco][component][lane] x 16 bytes
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void lds_dma_16(const void* gsrc, void* ldst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)ldst, 16, 0, 0);
}

__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0)

template <int WCO, int NTW, int P2LOG, bool PAIRS>
__global__ void __launch_bounds__(WG_THREADS, 2) qconv_fwd_f16_lds_kernel(const ConvArgs P) {
    constexpr int CK = F16_CK;
    constexpr int WPX = 4 / WCO;
    constexpr int TG = F16_TG;
    constexpr int WIMG = TG * WCO * 4 * 64;  // 16-byte vectors per filter group image
    extern __shared__ f16x8 lds16[];
    f16x8* xl = lds16;                    // [8 units][HPp]
    f16x8* wl = lds16 + 8 * P.HPp;        // [2][WIMG]

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
    const int w0e = PAIRS ? (w0 & ~1) : w0;  // pair staging starts the window at an even column
    const int colshift = w0 - w0e;

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
        poff[t] = pvalid[t] ? (nb * P.HTH + r * P.sh) * P.HTW + c * P.sw + colshift : colshift;
        oaddr[t] = ((long)(n0 + nb) * P.Cout * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c);
    }

    f32x16 acc[NTW][4];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][a][r] = 0.f;

    const int ngroups = (P.taps + TG - 1) / TG;          // per chunk
    const int total_groups = P.nchunks * ngroups;
    const f16x8* wsrc = static_cast<const f16x8*>(P.wpk) + (long)ct * total_groups * WIMG;
    // filter group image -> LDS buffer: TG*WCO*4 slices of 64 vectors, dealt round-robin to the waves
    auto copy_group = [&](int gs) {
        const f16x8* src = wsrc + (long)gs * WIMG;
        f16x8* dst = wl + (gs & 1) * WIMG;
#pragma unroll
        for (int s = 0; s < TG * WCO; ++s) {
            const int slice = s * 4 + wave;
            lds_dma_16(src + slice * 64 + lane, dst + slice * 64);
        }
    };

    const StagePos sp = make_stage_pos<P2LOG>(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW);
    const StagePairPos spp = make_stage_pairpos(P.in, n0, h0, w0e, P.NB, P.HTH, P.HTW);
    f16x8 stage[PAIRS ? 1 : (8 >> (8 - P2LOG))];
    unsigned int stagep[PAIRS ? 4 : 1][8];
    auto load_chunk = [&](int c0) {
        if constexpr (PAIRS) stage_load16_pairs(stagep, P.in, spp, c0);
        else stage_load16<P2LOG>(stage, P.in, sp, c0);
    };
    auto store_chunk = [&]() {
        if constexpr (PAIRS) stage_store16_pairs(xl, stagep, spp, P.HPp);
        else stage_store16<P2LOG>(xl, stage, sp, P.HP, P.HPp);
    };
    load_chunk(0);
    copy_group(0);

    int gs = 0;
    for (int chunk = 0; chunk < P.nchunks; ++chunk) {
        __syncthreads();  // every wave is done reading the previous chunk's activations
        store_chunk();
        int tap = 0, kh = 0, kw = 0;
        for (int g = 0; g < ngroups; ++g, ++gs) {
            wait_vmem_all();   // this group's filters have landed in LDS
            __syncthreads();   // ... for every wave; activations of this chunk are visible
            if (gs + 1 < total_groups) copy_group(gs + 1);
            if (g == 0 && chunk + 1 < P.nchunks) load_chunk((chunk + 1) * CK);
            const f16x8* wb = wl + (gs & 1) * WIMG + wco * 256 + lane;
#pragma unroll
            for (int tg = 0; tg < TG; ++tg) {
                if (tap < P.taps) {
                    const int tapoff = kh * P.dh * P.HTW + kw * P.dw;
                    // negative blocks of the Hamilton matrix only ever use -w1, -w2, -w3: flip the
                    // filter operand once per step instead of the activation operand per column tile
                    f16x8 w[4], nw[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        w[r] = wb[(tg * WCO * 4 + r) * 64];
                        nw[r] = neg8(w[r]);
                    }
                    const f16x8* xb = xl + kk * P.HPp + tapoff;
#pragma unroll
                    for (int t = 0; t < NTW; ++t) {
                        f16x8 x[4];
#pragma unroll
                        for (int p = 0; p < 4; ++p) x[p] = xb[p * 2 * P.HPp + poff[t]];
#pragma unroll
                        for (int p = 0; p < 4; ++p)
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                                acc[t][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qneg(p, q) ? nw[p ^ q] : w[p ^ q], x[p],
                                                                                   acc[t][q], 0, 0, 0);
                    }
                    ++tap;
                    if (++kw == P.Kw) { kw = 0; ++kh; }
                }
            }
        }
    }

    _Float16* out = static_cast<_Float16*>(P.out);
    const _Float16* bias = static_cast<const _Float16*>(P.bias);
    const long plane = (long)P.Hout * P.Wout;
    const int co_base = (ct * WCO + wco) * 32 + 4 * kk;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        if (!pvalid[t]) continue;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int co = co_base + 8 * (r >> 2) + (r & 3);
            if (co < P.Cout) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float v = acc[t][q][r];
                    if (bias) v += (float)bias[q * P.Cout + co];
                    out[q * P.out_cs + oaddr[t] + co * plane] = (_Float16)v;
                }
            }
        }
    }
}

// Filter packing for qconv_fwd_f16_lds_kernel (16-product only; conjugated / mirrored / transposed
// for MAP_DGRAD).  One thread per 16-byte vector of the image described above; taps beyond the
// filter (last group of a chunk) and channels beyond the tensor are zero.
struct PackLdsArgs {
    PackArgs base;
    int WCO;       // filter sub-tiles per workgroup tile
    int ngroups;   // tap groups per chunk
};

template <int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_f16_lds_kernel(const PackLdsArgs A) {
    const PackArgs& P = A.base;
    constexpr int TG = F16_TG;
    const int taps = P.Kh * P.Kw;
    // index = ((((tile*nchunks + chunk)*ngroups + g)*TG + tg)*WCO + wco)*4 + r)*64 + lane
    const long total = (long)P.row_tiles * P.nchunks * A.ngroups * TG * A.WCO * 4 * 64;
    const _Float16* w = static_cast<const _Float16*>(P.w);
    f16x8* outv = reinterpret_cast<f16x8*>(P.out);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int lane = idx & 63;
        long s = idx >> 6;
        const int r = s & 3; s >>= 2;
        const int wco = s % A.WCO; s /= A.WCO;
        const int tg = s % TG; s /= TG;
        const int g = s % A.ngroups; s /= A.ngroups;
        const int chunk = s % P.nchunks;
        const int tile = s / P.nchunks;
        const int tap = g * TG + tg;
        const int row = (tile * A.WCO + wco) * 32 + (lane & 31);
        f16x8 vec;
#pragma unroll
        for (int i = 0; i < 8; ++i) vec[i] = (_Float16)0;
        if (tap < taps && row < P.rows) {
            int kh = tap / P.Kw, kw = tap - kh * P.Kw;
            if (MAP == MAP_DGRAD) { kh = P.Kh - 1 - kh; kw = P.Kw - 1 - kw; }
            const float sgn = (MAP == MAP_DGRAD && r > 0) ? -1.f : 1.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int red = chunk * F16_CK + (lane >> 5) * 8 + i;
                if (red < P.red) {
                    const int o = (MAP == MAP_DGRAD) ? red : row;
                    const int in = (MAP == MAP_DGRAD) ? row : red;
                    vec[i] = (_Float16)(sgn * (float)w[r * P.wcs + o * P.so + in * P.si + kh * P.skh + kw * P.skw]);
                }
            }
        }
        outv[idx] = vec;
    }
}

// ---------------------------------------------------------------------------------------------
// Filter gradient on fp16 MFMA.  Same decomposition as qconv_wgrad_f32_kernel (64x64 channel tile,
// tap group = one filter row with up to TPW taps, split-K over pixel tiles, fp32 partial sums
// reduced by reduce_wgrad_kernel); the reduction index (pixels) is contiguous in NCHW, so both
// windows are staged as they lie.  One K step = 16 pixels = two 8-pixel packs:
//   A operand (output gradient): 8 consecutive tile pixels = one aligned 16-byte LDS read;
//   B operand (input, shifted by the tap): the 8 pixels' window offsets come from a per-tile
//   table, the 8 halves are gathered with 16-bit LDS reads (any stride / dilation / padding).
// ---------------------------------------------------------------------------------------------
template <int P2LOG>
__device__ __forceinline__ void stage_load_h2(f16x2 (&v)[(128) >> (8 - P2LOG)], const TileSrc& s, const StagePos& sp,
                                              int c0) {
    // 256 planes (4 components x 64 channels), G = 256 >> P2LOG groups, 256/G planes per thread, two per register
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = 256 / G;
    const _Float16* origin = static_cast<const _Float16*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int pc = e * G + sp.group;
        const int p = pc >> 6, c = pc & 63;
        const bool ok = sp.valid && (c0 + c) < s.C;
        const _Float16* ptr = ok ? origin + sp.goff + p * s.comp_stride + (long)(c0 + c) * plane : zero_ptr<_Float16>();
        v[e >> 1][e & 1] = *ptr;
    }
}

template <int P2LOG>
__device__ __forceinline__ void stage_store_h2(_Float16* dst, const f16x2 (&v)[(128) >> (8 - P2LOG)],
                                               const StagePos& sp, int HP, int pitch) {
    constexpr int G = WG_THREADS >> P2LOG;
    constexpr int E = 256 / G;
    if (sp.pos < HP) {
#pragma unroll
        for (int e = 0; e < E; ++e) dst[(e * G + sp.group) * pitch + sp.pos] = v[e >> 1][e & 1];
    }
}

template <int MODE, int TPW>
__global__ void __launch_bounds__(WG_THREADS) qconv_wgrad_f16_kernel(const WgradArgs P) {
    constexpr int CT = 64;
    constexpr int NACC = (MODE == 16) ? 4 : 8;
    constexpr int P2LOG = 6;  // 64 window positions x 4 plane groups
    extern __shared__ f16x8 lds16[];
    _Float16* gl = reinterpret_cast<_Float16*>(lds16);   // [4][CT][KPp], KPp multiple of 8 (16-byte rows)
    _Float16* xl = gl + 4 * CT * P.KPp;                    // [4][CT][HPp]
    int* poff = reinterpret_cast<int*>(xl + 4 * CT * P.HPp);  // [KP], 16-byte aligned

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wco = wave & 1, wci = wave >> 1;
    const int m = lane & 31, kk = lane >> 5;
    const int cot = blockIdx.x % P.co_tiles, cit = blockIdx.x / P.co_tiles;
    const int kh = blockIdx.y / P.groups_per_row;
    const int kw0 = (blockIdx.y % P.groups_per_row) * TPW;
    const int nkw = (P.Kw - kw0 < TPW) ? P.Kw - kw0 : TPW;
    const int HTW = (P.TW - 1) * P.sw + (nkw - 1) * P.dw + 1;
    const int thw = P.TH * P.TW;
    const int npix = P.NB * thw;

    for (int k = tid; k < P.KP; k += WG_THREADS) {
        const int nb = k / thw, rem = k - nb * thw;
        const int r = rem / P.TW, c = rem - r * P.TW;
        poff[k] = (k < npix) ? (nb * P.HTH + r * P.sh) * HTW + c * P.sw : 0;
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
    f16x2 sg[32], sx[32];
    StagePos spg, spx;
    auto issue = [&](int tile) {
        const int tw = tile % P.tiles_w;
        const int th = (tile / P.tiles_w) % P.tiles_h;
        const int tn = tile / (P.tiles_w * P.tiles_h);
        const int n0 = tn * P.NB, ho0 = th * P.TH, wo0 = tw * P.TW;
        spg = make_stage_pos<P2LOG>(P.g, n0, ho0, wo0, P.NB, P.TH, P.TW);
        spx = make_stage_pos<P2LOG>(P.x, n0, ho0 * P.sh - P.pt + kh * P.dh, wo0 * P.sw - P.pl + kw0 * P.dw, P.NB, P.HTH,
                                    HTW);
        stage_load_h2<P2LOG>(sg, P.g, spg, cot * CT);
        stage_load_h2<P2LOG>(sx, P.x, spx, cit * CT);
    };
    const int HPx = P.NB * P.HTH * HTW;
    if ((int)blockIdx.z < ntiles) issue(blockIdx.z);
    for (int tile = blockIdx.z; tile < ntiles; tile += gridDim.z) {
        __syncthreads();
        stage_store_h2<P2LOG>(gl, sg, spg, npix, P.KPp);
        stage_store_h2<P2LOG>(xl, sx, spx, HPx, P.HPp);
        // reduction indices beyond the tile's pixels must contribute zero
        for (int i = tid; i < 4 * CT * (P.KP - npix); i += WG_THREADS) {
            const int c = i / (P.KP - npix), k = npix + i % (P.KP - npix);
            gl[c * P.KPp + k] = (_Float16)0;
        }
        __syncthreads();
        if (tile + (int)gridDim.z < ntiles) issue(tile + gridDim.z);

        const _Float16* ga = gl + (wco * 32 + m) * P.KPp + kk * 8;
        const _Float16* xb = xl + (wci * 32 + m) * P.HPp;
        for (int ks = 0; ks < P.KP; ks += 16) {
            f16x8 g[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) g[q] = *reinterpret_cast<const f16x8*>(ga + q * gcp + ks);
            int po[8];
            {
                const int4 a = *reinterpret_cast<const int4*>(poff + ks + kk * 8);
                const int4 b = *reinterpret_cast<const int4*>(poff + ks + kk * 8 + 4);
                po[0] = a.x; po[1] = a.y; po[2] = a.z; po[3] = a.w;
                po[4] = b.x; po[5] = b.y; po[6] = b.z; po[7] = b.w;
            }
            f16x8 G[8];
            if constexpr (MODE == 8) lanes_grad(g, G, (_Float16)0.5f);
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
                if (t < nkw) {
                    f16x8 x[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p)
#pragma unroll
                        for (int i = 0; i < 8; ++i) x[p][i] = xb[p * xcp + po[i] + t * P.dw];
                    if constexpr (MODE == 16) {
                        f16x8 nx[4];
#pragma unroll
                        for (int p = 0; p < 4; ++p) nx[p] = neg8(x[p]);
#pragma unroll
                        for (int p = 0; p < 4; ++p)
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                                acc[t][p ^ q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(g[q], qneg(p, q) ? nx[p] : x[p],
                                                                                       acc[t][p ^ q], 0, 0, 0);
                    } else {
                        f16x8 L[8];
                        lanes_left(x, L);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(G[i], L[i], acc[t][i], 0, 0, 0);
                    }
                }
            }
        }
    }

    const int taps = P.Kh * P.Kw;
    const long tap_stride = 4L * P.CoP * P.CiP;
    float* dst = P.partial + (long)blockIdx.z * taps * tap_stride;
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

}  // namespace phx
