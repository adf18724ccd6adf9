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
            const bool ok = sp.valid && c < s.C && p < s.ncomp;
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
    sp.goff = ok ? ((long)(n0 + nb) * s.Cs * s.Hd + vh) * s.Wd + vw : 0;
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
            const bool ok = sp.valid && c < s.C && p < s.ncomp;
            const _Float16* ptr = ok ? origin + sp.goff + p * s.comp_stride + (long)c * plane : zero_ptr<_Float16>();
            d[e][i] = *reinterpret_cast<const unsigned int*>(ptr);
        }
    }
}

__device__ __forceinline__ void stage_store16_pairs(f16x8* dst, const unsigned int (&d)[4][8], const StagePairPos& sp,
                                                    int pitch) {
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
template <int MODE, int WCO, int NTW, int P2LOG, bool PAIRS>
__global__ void __launch_bounds__(WG_THREADS, (MODE == 8 || NTW == 1) ? 2 : 1) qconv_fwd_f16_kernel(const ConvArgs P0) {
    const ConvArgs P = group_view(P0);
    constexpr int CK = F16_CK;
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
        oaddr[t] = ((long)(n0 + nb) * P.CoutS * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c);
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
    const StagePairPos spp = make_stage_pairpos(P.in, n0, h0, w0e, P.NB, P.HTH, P.HTW);
    f16x8 stage[PAIRS ? 1 : (8 >> (8 - P2LOG))];
    unsigned int stagep[PAIRS ? 4 : 1][8];
    auto load_chunk = [&](int c0) {
        if constexpr (PAIRS) stage_load16_pairs(stagep, P.in, spp, c0);
        else stage_load16<P2LOG>(stage, P.in, sp, c0);
    };
    auto store_chunk = [&]() {
        if constexpr (PAIRS) stage_store16_pairs(lds16, stagep, spp, P.HPp);
        else stage_store16<P2LOG>(lds16, stage, sp, P.HP, P.HPp);
    };
    load_chunk(0);
    for (int chunk = 0; chunk < P.nchunks; ++chunk) {
        __syncthreads();
        store_chunk();
        __syncthreads();
        if (chunk + 1 < P.nchunks) load_chunk((chunk + 1) * CK);
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
                    lanes_left(x, L);
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

    conv_epilogue<_Float16, MODE, NTW, NACC>(P, acc, (ct * WCO + wco) * 32 + 4 * kk, oaddr, pvalid);
}

// Filter packing for the kernel above: one group of WC 16-byte vectors per (32-channel filter
// tile, K step, lane); lane = (row = lane % 32, kk = lane / 32), K step = chunk*taps + tap,
// vector element i = reduced channel chunk*16 + kk*8 + i.  MODE 16: the four filter components
// MODE 8: the eight right-operand lanes, formed in fp32 and rounded once (both of the conjugated filter for
// MAP_DGRAD: dx = g (x) conj(w) is a forward product, and the forward kernel runs it).
template <int MODE, int MAP>
__device__ __forceinline__ void pack_filters_f16_body(const PackArgs& P, long first, long stride) {
    constexpr int WC = (MODE == 16) ? 4 : 8;
    const int taps = P.Kh * P.Kw;
    const long total = (long)P.row_tiles * P.nchunks * taps * 64;
    const _Float16* w = static_cast<const _Float16*>(P.w);
    f16x8* outv = reinterpret_cast<f16x8*>(P.out);
    for (long idx = first; idx < total; idx += stride) {
        const int lane = idx & 63;
        long s = idx >> 6;
        const int tap = s % taps;
        s /= taps;
        const int chunk = s % P.nchunks;
        const int tile = s / P.nchunks;
        const int row = tile * 32 + (lane & 31);
        int kh = tap / P.Kw, kw = tap - kh * P.Kw;
        if (MAP == MAP_DGRAD) {
            kh = P.khm - kh * P.khs;
            kw = P.kwm - kw * P.kws;
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
                for (int r = 0; r < 4; ++r) wv[r] = ((MAP == MAP_DGRAD && r > 0) ? -1.f : 1.f) * (float)w[r * P.wcs + off];
            }
            if constexpr (MODE == 16) {
#pragma unroll
                for (int r = 0; r < 4; ++r) vec[r][i] = (_Float16)wv[r];
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

template <int MODE, int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_f16_kernel(const PackArgs P0) {
    const PackArgs P = group_view(P0);
    pack_filters_f16_body<MODE, MAP>(P, (long)blockIdx.x * blockDim.x + threadIdx.x, (long)gridDim.x * blockDim.x);
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

// The copies into LDS and the workgroup barrier of the kernels that keep copies in flight across barriers, kept out of the compiler's memory model.
// __syncthreads() carries workgroup-scope fences, in front of which the compiler waits for EVERY outstanding
// vector memory operation (s_waitcnt vmcnt(0)), and it puts the same wait in front of LDS reads that may alias an
// LDS write by a global_load_lds it knows of -- either way the copies of the steps ahead, which a ring of stages
// exists to keep in flight across the barrier, would be drained at every step.  So the copy is issued from inline
// assembly (the compiler then counts nothing for it: the kernels wait for their copies with explicit s_waitcnt
// vmcnt(n); the compiler's own waits for the loads it does know of stay correct, extra operations in flight can
// only make them longer), and the barrier is the bare instruction behind a wait for this wave's LDS operations.
__device__ __forceinline__ void lds_dma_16_untracked(const void* gsrc, void* ldst) {
    const unsigned int lds_addr = (unsigned int)(unsigned long)(__attribute__((address_space(3))) void*)ldst;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gsrc), "s"(lds_addr)
                 : "memory");  // (m0 is a reserved register: it cannot be named as clobbered, and nothing else here uses it)
}
__device__ __forceinline__ void wg_barrier_no_vmem_wait() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}


// Chunk staging of the activation window (CHUNKS): the window is NB*HTH rows of HTW positions, HTW a
// multiple of 8.  One task = (component, 8-channel pack, 8 consecutive positions of a row): eight
// 16-byte loads (one per channel, 2-byte aligned), an 8x8 transpose with byte permutes, eight 16-byte
// LDS entries.  A quarter of the load instructions of the pair staging, and no restriction on W.
// Positions outside the image are cleared with a mask that is fixed per task; tasks whose loads
// could leave the tensor (first / last rows of the first / last plane) load nothing and are filled
// element by element.  Entries are swizzled inside aligned groups of 8 (entry ^ (entry/8)%8) so that
// the eight stores of neighbouring tasks spread over all LDS banks.
struct StageChunk {
    const _Float16* ptr;  // channel 0 of the task's component at the task's first position
    int ent;              // unit * pitch + first entry of the task
    int swz;
    unsigned int bits;    // positions inside the image
    int kp;
    int sub;              // pointwise trick: 16-channel sub-chunk this window row stands for
    int cpr;              // channels-last: tasks per window row = positions between two of a task's entries
    bool task, live, careful;
};

__device__ __forceinline__ int swizzle_entry(int e) { return e ^ ((e >> 3) & 7); }

__device__ __forceinline__ StageChunk make_stage_chunk(const TileSrc& s, int n0, int h0, int w0, int NB, int HTH, int HTW,
                                                       int HPp) {
    StageChunk sc;
    const int cpr = HTW >> 3;
    const int hp8 = NB * HTH * cpr;  // tasks per unit
    const int u = threadIdx.x / hp8, ch = threadIdx.x - u * hp8;
    sc.task = u < 8;
    const int row = ch / cpr, cc = ch - row * cpr;
    const int nb = row / HTH, hr = row - nb * HTH;
    // pointwise trick (s.pw > 0): the window rows are not image rows but consecutive 16-channel
    // sub-chunks of the one (flattened) image row, so that a "filter column" of s.pw taps walks over
    // 16*s.pw channels per staged chunk
    sc.sub = s.pw ? hr : 0;
    int vh = s.pw ? 0 : h0 + hr, img = n0 + nb;
    const int vw0 = w0 + cc * 8;
    if (s.tall) {  // h0 counts rows of the tall image; rows above it and between the images are zeros
        img = vh >= 0 ? vh / s.tall : -1;
        vh -= img * s.tall;
    }
    const int p = u >> 1;
    sc.kp = u & 1;
    sc.live = sc.task && p < s.ncomp && nb < NB && img >= 0 && img < s.N && vh >= 0 && vh < s.Hd;
    const _Float16* base = static_cast<const _Float16*>(s.base);
    const long plane = (long)s.Hd * s.Wd;
    sc.cpr = cpr;
    if (s.nhwc) {
        // channels-last: the entry of a position (8 consecutive channels) is 16 contiguous bytes of memory, loaded and
        // stored as it is.  A task takes positions cc, cc + cpr, ... of its window row rather than 8 neighbours:
        // the lanes of a load then read neighbouring positions (Cs elements apart) instead of every eighth -- with a
        // power-of-two channel count those would all sit 4 or 8 KiB apart, on one memory channel.
        const int vw = w0 + cc;
        sc.bits = 0u;
        if (sc.live) {
#pragma unroll
            for (int j = 0; j < 8; ++j) sc.bits |= (unsigned int)(vw + j * cpr >= 0 && vw + j * cpr < s.Wd) << j;
        }
        sc.ptr = base + p * s.comp_stride + (((long)img * s.Hd + vh) * s.Wd + vw) * s.Cs;
        const _Float16* end = base + (long)(s.ncomp - 1) * s.comp_stride + (long)s.N * plane * s.Cs;
        sc.careful = sc.live && (sc.ptr < base || sc.ptr + 7L * cpr * s.Cs + ((s.C + 15) & ~15) > end);
        sc.ent = (sc.task ? u : 0) * HPp;  // unit base; the entries are row * HTW + cc + j * cpr, swizzled one by one
        sc.swz = row * HTW + cc;
        return sc;
    } else {
        sc.bits = sc.live ? interval_bits(-vw0, s.Wd - vw0) : 0u;
        sc.ptr = base + p * s.comp_stride + ((long)img * s.Cs * s.Hd + vh) * s.Wd + vw0;
        const _Float16* end = base + (long)(s.ncomp - 1) * s.comp_stride + ((long)(s.N - 1) * s.Cs + s.C) * plane;
        sc.careful = sc.live && (sc.ptr < base || sc.ptr + (long)(s.C - 1) * plane + 8 > end);
    }
    const int e0 = row * HTW + cc * 8;
    sc.ent = (sc.task ? u : 0) * HPp + e0;
    sc.swz = (e0 >> 3) & 7;
    return sc;
}

__device__ __forceinline__ void stage_chunk_load(u32x4 (&r)[8], const TileSrc& s, const StageChunk& sc, int c0, int i) {
    if (s.nhwc) {  // position i of the task: channels c0 + 8 kp .. + 7
        const int c = c0 + sc.kp * 8;
        const _Float16* ptr = (sc.live && !sc.careful && c < s.C) ? sc.ptr + (long)i * sc.cpr * s.Cs + c : static_cast<const _Float16*>(s.base);
        r[i] = load16_a2(ptr);
        return;
    }
    const long plane = (long)s.Hd * s.Wd;
    const int cv = c0 + sc.kp * 8 + i;
    const int c = s.pw ? ((cv >> 4) * s.pw + sc.sub) * 16 + (cv & 15) : cv;
    // channels past the tensor meet zero filters: any finite value will do, the tensor's first bytes are safe
    const _Float16* ptr =
        (sc.live && !sc.careful && c < s.C) ? sc.ptr + c * plane : static_cast<const _Float16*>(s.base);
    r[i] = load16_a2(ptr);
}

__device__ __forceinline__ void stage_chunk_store(f16x8* xl, const u32x4 (&r)[8], const TileSrc& s, const StageChunk& sc,
                                                  int c0) {
    if (!sc.task) return;
    if (s.nhwc) {
        // entries as loaded (the host takes this path only when C is a multiple of 8: a pack of 8 channels is inside
        // the tensor or outside it as a whole); positions outside the image and packs outside the tensor are cleared
        const int c = c0 + sc.kp * 8;
        const unsigned int bits = (sc.careful || c >= s.C) ? 0u : sc.bits;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const u32x4 v = ((bits >> j) & 1) ? r[j] : u32x4{0u, 0u, 0u, 0u};
            xl[sc.ent + swizzle_entry(sc.swz + j * sc.cpr)] = __builtin_bit_cast(f16x8, v);
        }
        if (sc.careful) {
            _Float16* xh = reinterpret_cast<_Float16*>(xl);
#pragma unroll 2
            for (int j = 0; j < 8; ++j) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    xh[(sc.ent + swizzle_entry(sc.swz + j * sc.cpr)) * 8 + i] =
                        (c + i < s.C && ((sc.bits >> j) & 1)) ? sc.ptr[(long)j * sc.cpr * s.Cs + c + i] : (_Float16)0;
            }
        }
        return;
    }
    const u32x4 mk = expand_half_mask(sc.careful ? 0u : sc.bits);
    u32x4 rm[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) rm[i] = r[i] & mk;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        u32x4 v;
#pragma unroll
        for (int m = 0; m < 4; ++m)
            v[m] = __builtin_amdgcn_perm(rm[2 * m + 1][j >> 1], rm[2 * m][j >> 1], (j & 1) ? 0x07060302u : 0x05040100u);
        xl[sc.ent + (j ^ sc.swz)] = __builtin_bit_cast(f16x8, v);
    }
    if (sc.careful) {
        const long plane = (long)s.Hd * s.Wd;
        _Float16* xh = reinterpret_cast<_Float16*>(xl);
#pragma unroll 2
        for (int i = 0; i < 8; ++i) {
            const int cv = c0 + sc.kp * 8 + i;
            const int c = s.pw ? ((cv >> 4) * s.pw + sc.sub) * 16 + (cv & 15) : cv;
            _Float16 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (c < s.C && ((sc.bits >> j) & 1)) ? sc.ptr[c * plane + j] : (_Float16)0;
#pragma unroll
            for (int j = 0; j < 8; ++j) xh[(sc.ent + (j ^ sc.swz)) * 8 + i] = v[j];
        }
    }
}

// Epilogue for a channels-last output, out[4][N][Hout][Wout][CoutS] with oaddr = pixel index * CoutS.  Register e of an
// accumulator is output channel 8*(e/4) + 4*kk + e%4 of the wave's 32 at this lane's pixel: four groups of 4
// consecutive channels.  One v_permlane32_swap per packed dword between the two lane halves (which hold the same
// pixels) turns them into 16 consecutive channels per lane -- the lower half 0..15, the upper half 16..31 -- stored as
// two 16-byte words.  The host takes this path only when Cout and CoutS are multiples of 8.
template <int MODE, int NTW, int NACC>
__device__ __forceinline__ void conv_epilogue_cl(const ConvArgs& P, const f32x16 (&acc)[NTW][NACC], int co_wave,
                                                 const long (&oaddr)[NTW], const bool (&pvalid)[NTW]) {
    _Float16* out = static_cast<_Float16*>(P.out);
    const _Float16* bias = static_cast<const _Float16*>(P.bias);
    const int kk = (threadIdx.x >> 5) & 1;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        unsigned int d[4][4][2];  // [component][register group][packed pair]
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                float y[2][4];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const int e = 4 * g + 2 * i + k;
                    if constexpr (MODE == 16) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) y[k][q] = acc[t][q][e];
                    } else {
                        float l[8];
#pragma unroll
                        for (int a = 0; a < 8; ++a) l[a] = acc[t][a][e];
                        merge_output(l, y[k]);
                    }
                    const int co = co_wave + 8 * g + 4 * kk + 2 * i + k;
                    if (bias && co < P.Cout) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) y[k][q] += (float)bias[q * P.CoutS + co];
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    f16x2 h;
                    h[0] = (_Float16)y[0][q];
                    h[1] = (_Float16)y[1][q];
                    d[q][g][i] = __builtin_bit_cast(unsigned int, h);
                }
            }
        const int co = co_wave + 16 * kk;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            u32x4 v0, v1;
#pragma unroll
            for (int i = 0; i < 2; ++i) {  // (every lane takes part in the swaps, whatever its pixel)
                const auto s02 = __builtin_amdgcn_permlane32_swap(d[q][0][i], d[q][2][i], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(d[q][1][i], d[q][3][i], false, false);
                v0[i] = s02[0]; v0[2 + i] = s02[1];
                v1[i] = s13[0]; v1[2 + i] = s13[1];
            }
            _Float16* dst = out + q * P.out_cs + oaddr[t] + co;
            if (pvalid[t] && co < P.Cout) *reinterpret_cast<u32x4_a2*>(dst) = v0;
            if (pvalid[t] && co + 8 < P.Cout) *reinterpret_cast<u32x4_a2*>(dst + 8) = v1;
        }
    }
}

// One eighth of the left-operand lane map of the factorized product (lanes_left): step i leaves lane i ready.
__device__ __forceinline__ void lane_step(const f16x8 (&x)[4], f16x8 (&L)[8], int i) {
    switch (i) {
        case 0: L[0] = add8_pinned(x[3], x[1]); break;
        case 1: L[1] = sub8_pinned(x[0], x[2]); break;
        case 2: L[2] = add8_pinned(x[0], x[2]); break;
        case 3: L[3] = sub8_pinned(x[3], x[1]); break;
        case 4: L[4] = sub8_pinned(x[3], x[2]); break;
        case 5: L[5] = add8_pinned(x[1], x[0]); break;
        case 6: L[6] = sub8_pinned(x[0], x[1]); break;
        default: L[7] = add8_pinned(x[3], x[2]); break;
    }
}

// EARLY (chunk staging, problems with one filter group per chunk, i.e. pointwise ones): only the products of one
// group stand between the request for the next chunk's activations and their use, so the request goes out at the
// start of the group, ahead of the filter copy (which the same wait then covers).
// XREAL (16-product, chunk staging): the input holds its real component only (P.in.ncomp == 1); the twelve
// products with the absent components and their operand reads are left out at compile time.
template <int MODE, int WCO, int NTW, int P2LOG, bool CHUNKS, bool EARLY = false, bool XREAL = false>
__global__ void __launch_bounds__(WG_THREADS, (MODE == 16 && NTW == 1) ? 2 : 1) qconv_fwd_f16_lds_kernel(const ConvArgs P0) {
    const ConvArgs P = group_view(P0);
    static_assert(!EARLY || CHUNKS, "early activation requests belong to chunk staging");
    static_assert(!XREAL || (MODE == 16 && CHUNKS), "the real-input variant is a 16-product kernel with chunk staging");
    constexpr int NP = XREAL ? 1 : 4;          // input components that take part
    constexpr int CK = F16_CK;
    constexpr int WPX = 4 / WCO;
    constexpr int TG = F16_TG;
    constexpr int NW = (MODE == 16) ? 4 : 8;   // filter operands per tap and sub-tile: components or right lanes
    constexpr bool PIN = !(MODE == 16 && NTW == 1);  // one workgroup per CU: MFMA in its AGPR form
    constexpr int WIMG = TG * WCO * NW * 64;   // 16-byte vectors per filter group image
    constexpr int NSL = TG * WCO * NW / 4;     // 1 KiB slices of that image per wave
    extern __shared__ f16x8 lds16[];
    // unit pitch of the staged window: fixed with chunk staging, so that the four component reads of an
    // operand differ by immediate offsets only (the host sets HPp to the same value)
    const int XP = CHUNKS ? F16_XPITCH : P.HPp;
    f16x8* xl = lds16;                    // [8 units][XP]
    f16x8* wl = lds16 + 8 * XP;           // [2][WIMG]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wco = wave % WCO, wpx = wave / WCO;
    const int j = lane & 31, kk = lane >> 5;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // (a scalar the compiler can address LDS copies with)

    int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int ct = bid % P.co_tiles;
    bid /= P.co_tiles;
    const int tw = bid % P.tiles_w;
    bid /= P.tiles_w;
    const int th = bid % P.tiles_h;
    const int tn = bid / P.tiles_h;
    const int n0 = tn * P.NB, ho0 = th * P.TH, wo0 = tw * P.TW;
    int h0 = ho0 * P.sh - P.pt;
    const int w0 = wo0 * P.sw - P.pl;
    // Flat tiling (P.in.tall > 0; unit stride, whole rows): the images form one tall image, P.in.tall rows apart
    // with zero rows between them, and workgroup th takes the next WPX*NTW*32 output positions of it in row-major
    // order -- every lane works whatever the image size; the window is every row those positions touch.
    const int q0 = th * (WPX * NTW * 32), R0 = P.in.tall ? q0 / P.Wout : 0;
    if (P.in.tall) h0 = R0 - P.pt;

    int poff[NTW];
    long oaddr[NTW];
    bool pvalid[NTW];
    const int thw = P.TH * P.TW;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        const int pix = (wpx * NTW + t) * 32 + j;
        if (P.in.tall) {
            const int q = q0 + pix, R = q / P.Wout, c = q - R * P.Wout;
            const int n = R / P.in.tall, ho = R - n * P.in.tall;
            pvalid[t] = n < P.in.N && ho < P.Hout;
            poff[t] = pvalid[t] ? (R - R0) * P.HTW + c : 0;
            oaddr[t] = P.nhwc ? (((long)n * P.Hout + ho) * P.Wout + c) * P.CoutS : ((long)n * P.CoutS * P.Hout + ho) * P.Wout + c;
        } else {
            const int nb = pix / thw, rem = pix - nb * thw;
            const int r = rem / P.TW, c = rem - r * P.TW;
            pvalid[t] = nb < P.NB && (n0 + nb) < P.in.N && (ho0 + r) < P.Hout && (wo0 + c) < P.Wout;
            poff[t] = pvalid[t] ? (nb * P.HTH + r * P.sh) * P.HTW + c * P.sw : 0;
            oaddr[t] = P.nhwc ? (((long)(n0 + nb) * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c)) * P.CoutS
                              : ((long)(n0 + nb) * P.CoutS * P.Hout + (ho0 + r)) * P.Wout + (wo0 + c);
        }
    }

    f32x16 acc[NTW][NW];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][a][r] = 0.f;

    const int ngroups = (P.taps + TG - 1) / TG;          // per chunk
    const int total_groups = P.nchunks * ngroups;
    const f16x8* wsrc = static_cast<const f16x8*>(P.wpk) + (long)ct * total_groups * WIMG;

    // activation staging, one chunk ahead in registers
    const StagePos sp = make_stage_pos<P2LOG>(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW);
    const StageChunk sc = make_stage_chunk(P.in, n0, h0, w0, P.NB, P.HTH, P.HTW, XP);
    f16x8 stage[CHUNKS ? 1 : (8 >> (8 - P2LOG))];
    u32x4 stagec[CHUNKS ? 8 : 1];
    constexpr int XLOADS = CHUNKS ? 8 : 0;  // activation load instructions that can be dealt out one by one
    auto store_chunk = [&](int c0) {
        if constexpr (CHUNKS) stage_chunk_store(xl, stagec, P.in, sc, c0);
        else stage_store16<P2LOG>(xl, stage, sp, P.HP, P.HPp);
    };
    if constexpr (CHUNKS) {
#pragma unroll
        for (int i = 0; i < 8; ++i) stage_chunk_load(stagec, P.in, sc, 0, i);
    } else {
        stage_load16<P2LOG>(stage, P.in, sp, 0);
    }
    // filter group image -> LDS buffer: slices of 64 vectors, dealt round-robin to the waves.  Slice
    // s * 4 + wave starts at vector s * 256 + wave * 64: a uniform base plus the thread index on the
    // global side, a scalar address on the LDS side.
    auto copy_slice = [&](const f16x8* src, f16x8* dst, int s) {
        lds_dma_16(src + s * 256 + tid, dst + s * 256 + wave_u * 64);
    };
    {
#pragma unroll
        for (int s = 0; s < NSL; ++s) copy_slice(wsrc, wl, s);
    }

    PHX_PHASES_BEGIN(5)
    bool x_in_flight = false;  // activation loads were issued after the latest filter copy
    int chunk = 0, g = 0, tap = 0, kh = 0, kw = 0;
    // Factorized form: the left lanes of a block are formed from the four staged components while the
    // previous block is being multiplied (one wave per SIMD: nothing else hides that arithmetic), from
    // components requested a block earlier still.  Where the next group works on the same staged chunk
    // that pipeline runs on across the group boundary (CARRY; it needs an even number of blocks per group
    // so that the register double buffers keep their parity).
    constexpr bool CARRY = MODE == 8 && (TG * NTW) % 2 == 0;
    f16x8 xf[2][4], Lf[MODE == 8 ? 2 : 1][8];
    bool carried = false;      // the previous group left this group's first lanes and components in registers
    // one flat loop over (chunk, filter group) steps: a single loop keeps the accumulators in place
    for (int gs = 0; gs < total_groups; ++gs) {
        if (g == 0) {
            __syncthreads();  // every wave is done reading the previous chunk's activations
            PHX_STAMP(0)
            store_chunk(chunk * CK);  // (waits for this chunk's activation loads)
            PHX_STAMP(1)
            tap = 0; kh = 0; kw = 0;
        }
        {
            // this group's filters have landed in LDS; vmcnt counts in order, so activation loads issued
            // after the filter copy may stay in flight
            if (x_in_flight) __builtin_amdgcn_s_waitcnt(0x0F70 | XLOADS);
            else wait_vmem_all();
            __syncthreads();   // ... for every wave; activations of this chunk are visible
            PHX_STAMP(2)
            // The group is a fixed sequence of TG*NTW blocks of 16 MFMAs.  Taps past the end of the filter
            // are packed as zeros, so they are multiplied like the others (against window offset 0).
            // A wave that issues its global loads back to back stalls until the memory pipeline has taken
            // them all; so the LDS copy of the next filter group is dealt out over the first half of the
            // blocks and the activation loads of the next chunk (first group of a chunk) over the second half.
            constexpr int NBLK = TG * NTW;
            constexpr int DBLK = (NBLK + 1) / 2;                    // blocks that carry filter-copy slices
            constexpr int DPB = (NSL + DBLK - 1) / DBLK;
            constexpr int XBLK = NBLK - DBLK;                       // blocks that carry activation loads
            constexpr int XPB = XBLK ? (XLOADS + XBLK - 1) / XBLK : 0;
            const bool more_groups = gs + 1 < total_groups;
            const bool more_chunks = g == 0 && chunk + 1 < P.nchunks;
            // window offsets of this group's taps and (CARRY) of the next group's
            int tapoff[CARRY ? 2 * TG : TG];
#pragma unroll
            for (int tg = 0; tg < TG; ++tg) {
                tapoff[tg] = tap < P.taps ? kh * P.dh * P.HTW + kw * P.dw : 0;
                ++tap;
                if (++kw == P.Kw) { kw = 0; ++kh; }
            }
            if constexpr (CARRY) {
                int tap2 = tap, kh2 = kh, kw2 = kw;
#pragma unroll
                for (int tg = TG; tg < 2 * TG; ++tg) {
                    tapoff[tg] = tap2 < P.taps ? kh2 * P.dh * P.HTW + kw2 * P.dw : 0;
                    ++tap2;
                    if (++kw2 == P.Kw) { kw2 = 0; ++kh2; }
                }
            }
            const bool carry = CARRY && g + 1 < ngroups;  // the next group multiplies the same staged chunk
            const f16x8* wb = wl + (gs & 1) * WIMG + wco * (NW * 64) + lane;
            const f16x8* wsrc_next = wsrc + (long)(gs + 1) * WIMG;
            f16x8* wdst_next = wl + ((gs + 1) & 1) * WIMG;
            f16x8 wf[2][NW];
            auto read_w = [&](f16x8 (&w)[NW], int tg) {
#pragma unroll
                for (int r = 0; r < NW; ++r) w[r] = wb[(tg * WCO * NW + r) * 64];
            };
            auto read_x = [&](f16x8 (&x)[4], int blk) {
                const int pos = tapoff[blk / NTW] + poff[blk % NTW];
                const f16x8* xb = xl + kk * XP + (CHUNKS ? swizzle_entry(pos) : pos);
#pragma unroll
                for (int p = 0; p < NP; ++p) x[p] = xb[p * 2 * XP];
            };
            read_w(wf[0], 0);
            if constexpr (MODE == 16) {
                read_x(xf[0], 0);
            } else {
                if (!carried) {
                    read_x(xf[0], 0);
                    if (NBLK > 1) read_x(xf[1], 1);
#pragma unroll
                    for (int i = 0; i < 8; ++i) lane_step(xf[0], Lf[0], i);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (NBLK > 2) read_x(xf[0], 2);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (!CHUNKS) {
                if (more_chunks) stage_load16<P2LOG>(stage, P.in, sp, (chunk + 1) * CK);
            }
            PHX_STAMP(3)
#pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) {
                const int tg = blk / NTW, t = blk % NTW;
                if constexpr (EARLY) {
                    constexpr int EPB = NBLK > 1 ? (NSL + NBLK - 2) / (NBLK - 1) : NSL;  // filter slices per later block
                    if (blk == 0 && more_chunks) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) stage_chunk_load(stagec, P.in, sc, (chunk + 1) * CK, i);
                    }
                    if (more_groups && (blk > 0 || NBLK == 1)) {
#pragma unroll
                        for (int s = 0; s < NSL; ++s) {
                            if (NBLK == 1 || s / EPB == blk - 1) copy_slice(wsrc_next, wdst_next, s);
                        }
                    }
                } else if (blk < DBLK) {
                    if (more_groups) {
                        // (loops with constant bounds: they must unroll, the staging registers are indexed by them)
#pragma unroll
                        for (int s = 0; s < NSL; ++s) {
                            if (s / DPB == blk) copy_slice(wsrc_next, wdst_next, s);
                        }
                    }
                } else if constexpr (CHUNKS) {
                    if (more_chunks) {
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            if (i / XPB == blk - DBLK) stage_chunk_load(stagec, P.in, sc, (chunk + 1) * CK, i);
                    }
                }
                const f16x8(&w)[NW] = wf[tg & 1];
                const f16x8(&x)[4] = xf[blk & 1];
                // the next block's operands are requested once this block is under way: everything
                // outstanding at the top of a block is then exactly what that block needs
                auto prefetch = [&]() {
                    __builtin_amdgcn_sched_barrier(0);
                    if (blk + 1 < NBLK) {
                        read_x(xf[(blk + 1) & 1], blk + 1);
                        if ((blk + 1) % NTW == 0) read_w(wf[(tg + 1) & 1], tg + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                };
                if constexpr (MODE == 16) {
                    // negative blocks of the Hamilton matrix only ever use -w1, -w2, -w3
                    f16x8 nw[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) nw[r] = neg8(w[r]);
#pragma unroll
                    for (int p = 0; p < NP; ++p) {
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            acc[t][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qneg(p, q) ? nw[p ^ q] : w[p ^ q], x[p],
                                                                               acc[t][q], 0, 0, 0);
                        if (p == 0) prefetch();
                    }
                } else {
                    // factorized form: eight independent products of a left lane with a right lane (packed).
                    // Each product is followed by the arithmetic for one lane of the next block; the
                    // components of the block after that are requested as soon as their registers are free.
                    __builtin_amdgcn_sched_barrier(0);
                    // (block numbers from NBLK on are the next group's, reached only with carry; the third
                    // block of the next group is requested at that group's start, once its first is consumed)
                    // The requests go out after the first product: whatever the wait in front of that
                    // product covers was requested a whole block ago.
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[i], Lf[blk & 1][i], acc[t][i], 0, 0, 0);
                        if (blk + 1 < NBLK || carry) lane_step(xf[(blk + 1) & 1], Lf[(blk + 1) & 1], i);
                        __builtin_amdgcn_sched_barrier(0);
                        // (last block: after the lane arithmetic, whose waits sit behind run-time branches there
                        // and are therefore complete ones)
                        if (i == (blk == NBLK - 1 ? 7 : 0)) {
                            if (blk > 0 && (blk + 2 < NBLK || carry)) read_x(xf[blk & 1], blk + 2);
                            if (t == NTW - 1 && tg + 1 < TG) read_w(wf[(tg + 1) & 1], tg + 1);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                // pin the accumulators to the AGPR file: left alone, the allocator parks one column tile in
                // VGPRs and copies 64 registers in and out around every block
                if constexpr (PIN) {
#pragma unroll
                    for (int q = 0; q < NW; ++q) asm volatile("" : "+a"(acc[t][q]));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            x_in_flight = CHUNKS && !EARLY && more_chunks;
            carried = carry;
            PHX_STAMP(4)
        }
        if (++g == ngroups) { g = 0; ++chunk; }
    }

    if (CHUNKS && P.nhwc) conv_epilogue_cl<MODE, NTW, NW>(P, acc, (ct * WCO + wco) * 32, oaddr, pvalid);
    else conv_epilogue<_Float16, MODE, NTW, NW>(P, acc, (ct * WCO + wco) * 32 + 4 * kk, oaddr, pvalid);
#ifdef PHX_PHASE_TIMING
    __builtin_amdgcn_s_waitcnt(0x0F70);  // (charge the stores to the epilogue; otherwise the wave ends with them in flight)
#endif
    PHX_STAMP(5)
    PHX_PHASES_REPORT("fwd_f16_lds: barrier / store / wait+barrier / prefetch / mfma / epilogue", 6)
}

// Filter packing for qconv_fwd_f16_lds_kernel (conjugated / mirrored / transposed for MAP_DGRAD) into the
// image described above; taps beyond the filter (last group of a chunk) and channels beyond the tensor are zero.
struct PackLdsArgs {
    PackArgs base;
    int WCO;       // filter sub-tiles per workgroup tile
    int ngroups;   // tap groups per chunk
    int pw;        // pointwise trick: the taps of a group are pw consecutive 16-channel sub-chunks (0 = off)
};

template <int MODE, int MAP>
__device__ __forceinline__ void pack_filters_f16_lds_body(const PackLdsArgs& A, long first, long stride) {
    const PackArgs& P = A.base;
    constexpr int TG = F16_TG;
    constexpr int NW = (MODE == 16) ? 4 : 8;
    // One thread per reduced channel (element i of a 16-byte vector).  16-product: of one vector (one component);
    // 8-product: of the eight lane vectors of a (tap, sub-tile, lane) slot, which all derive from the same four
    // filter values.  Neighbouring threads write neighbouring halves: every store instruction fills whole vectors.
    constexpr int PER = (MODE == 16) ? 1 : NW;
    const int taps = A.pw ? A.pw : P.Kh * P.Kw;
    // element index = (((((tile*nchunks + chunk)*ngroups + g)*TG + tg)*WCO + wco)*NW + r)*64 + lane)*8 + i
    const long total = (long)P.row_tiles * P.nchunks * A.ngroups * TG * A.WCO * (NW / PER) * 64 * 8;
    const _Float16* w = static_cast<const _Float16*>(P.w);
    _Float16* outh = static_cast<_Float16*>(P.out);
    for (long idx = first; idx < total; idx += stride) {
        const int i = idx & 7;
        const int lane = (idx >> 3) & 63;
        long s = idx >> 9;
        int r = 0;
        if constexpr (PER == 1) { r = s % NW; s /= NW; }
        const long slot = s;  // (tile, chunk, g, tg, wco)
        const int wco = s % A.WCO; s /= A.WCO;
        const int tg = s % TG; s /= TG;
        const int g = s % A.ngroups; s /= A.ngroups;
        const int chunk = s % P.nchunks;
        const int tile = s / P.nchunks;
        const int tap = g * TG + tg;
        const int row = (tile * A.WCO + wco) * 32 + (lane & 31);
        const int k16 = (lane >> 5) * 8 + i;
        const int red = A.pw ? (chunk * A.pw + tap) * 16 + k16 : chunk * F16_CK + k16;
        _Float16 val[PER];
#pragma unroll
        for (int q = 0; q < PER; ++q) val[q] = (_Float16)0;
        if (tap < taps && row < P.rows && red < P.red) {
            int kh = tap / P.Kw, kw = tap - kh * P.Kw;
            if (MAP == MAP_DGRAD) { kh = P.khm - kh * P.khs; kw = P.kwm - kw * P.kws; }
            if (A.pw) {  // the one real tap (of a strided convolution's phase: the filter tap that reaches it)
                kh = (MAP == MAP_DGRAD) ? P.khm : 0;
                kw = (MAP == MAP_DGRAD) ? P.kwm : 0;
            }
            const int o = (MAP == MAP_DGRAD) ? red : row;
            const int in = (MAP == MAP_DGRAD) ? row : red;
            const long off = o * P.so + in * P.si + kh * P.skh + kw * P.skw;
            if constexpr (MODE == 16) {
                const float sgn = (MAP == MAP_DGRAD && r > 0) ? -1.f : 1.f;  // conjugate
                val[0] = (_Float16)(sgn * (float)w[r * P.wcs + off]);
            } else {
                // input gradient: dx = g (x) conj(w) is the forward product of the gradient with the
                // conjugated filter, so the forward kernel serves it and only the packing differs
                float wv[4], R[8];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    wv[c] = ((MAP == MAP_DGRAD && c > 0) ? -1.f : 1.f) * (float)w[c * P.wcs + off];
                lanes_right(wv, R);  // formed in fp32, rounded once
#pragma unroll
                for (int q = 0; q < 8; ++q) val[q] = (_Float16)R[q];
            }
        }
        if constexpr (PER == 1) {
            outh[idx] = val[0];
        } else {
#pragma unroll
            for (int q = 0; q < PER; ++q) outh[(((slot * NW + q) * 64 + lane) << 3) + i] = val[q];
        }
    }
}

template <int MODE, int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_f16_lds_kernel(const PackLdsArgs A0) {
    PackLdsArgs A = A0;
    A.base = group_view(A0.base);
    pack_filters_f16_lds_body<MODE, MAP>(A, (long)blockIdx.x * blockDim.x + threadIdx.x, (long)gridDim.x * blockDim.x);
}

// ---------------------------------------------------------------------------------------------
// Filter gradient on fp16 MFMA (v_mfma_f32_16x16x32_f16).  GEMM view per tap: rows = output
// channels (A operand = output gradient), columns = input channels (B operand = input shifted by
// the tap), reduction over batch x output pixels -- the contiguous index of NCHW, so both operands
// are staged as they lie: 16-byte chunks of 8 consecutive pixels of one row.
//   Reduction space: every output row (n, ho) is cut into ceil(Wo/8) chunks of 8 pixels; a pixel
//   tile is any 8 consecutive chunks of that list (64 reduction indices, two K steps of 32).
//   Elements past the row end, padding columns and padding rows are cleared with a per-chunk bit
//   mask after the (unconditional) load, so the loads themselves are plain 16-byte global loads
//   at 2-byte alignment.  The few chunks whose load would reach outside the tensor allocation
//   (first / last rows of the first / last plane) are filled element by element instead.
//   One workgroup = (CoT x CiT channel tile) x (one filter row kh, TPW adjacent kw) x (slice of
//   the reduction); CoT = 32*MT, CiT = 32*NT, the 4 waves form a 2x2 grid, each owning MT x NT
//   MFMA tiles of 16x16 channels for every tap of the group and all four components (16-product:
//   signs folded into a negated copy of the gradient operand) or all eight lanes (8-product).
//   TPW == 3 or 4 (unit stride and dilation along W): one 10- or 12-pixel load per input chunk yields the
//   three copies shifted by 0/1/2 pixels with byte-align operations; each copy is written to its
//   own LDS plane so every MFMA operand is one aligned 16-byte LDS read.
//   SW == 2: the input chunk is 16 consecutive pixels of which the even ones are kept.
//   Flat chunk list (P.flat; unit strides, output and input rows of the same length >= 7): a row of 28 or 14
//   pixels fills its last chunk half, an eighth of all chunks' work multiplies zeros.  Here the whole image plane
//   is cut into chunks of 8 consecutive pixels instead (row-major, so a chunk may run over a row end): the input
//   pixel of output pixel q under tap (kh, kw) is the plane's pixel q + (kh*dh - pt)*W + (kw*dw - pl), again 8 (or
//   10, 12) consecutive pixels of memory; which of them are padding depends on the pixel's own row and column,
//   so the masks are per tap and pixel, built from the at most two row segments of a chunk.
//   Partial sums go to workspace[z]; reduce_wgrad_kernel adds them in a fixed order.
//   Channels-last tensors (CL; 64x64 channel tiles, unit stride, one or three taps): the reduction index is no
//   longer the contiguous one, 8 consecutive CHANNELS of a pixel are.  A thread then stages (chunk of 8 pixels) x
//   (component, 8 channels): one 16-byte load per pixel -- 8 for the gradient, 8 + TPW - 1 for the input, whose taps
//   are shifts by whole pixels -- and an 8x8 transposition in registers (byte permutes) on the way to the same LDS
//   rows of 8 pixels per channel, under the same pixel masks.  Load and store counts per thread are those of the
//   channels-first form; the multiplications and the epilogue do not know the difference.
// ---------------------------------------------------------------------------------------------
constexpr int WG16_KP = 64;         // reduction indices per pixel tile
constexpr int WG16_PITCH = 64 + 8;  // LDS halves per staged channel row (16-byte skew against bank conflicts)

struct WgChunk {  // where one 8-pixel chunk of the reduction space lies (flat list: ho = 0, wo0 = pixel of the plane)
    bool live;    // inside the reduction space
    int n, ho, wo0;
    int gi;       // index in the chunk list
};

struct WgStep {   // advance of a thread's chunk from one of its tiles to the next (uniform)
    int dgi, dwo, dho, dn;
};

__device__ __forceinline__ WgStep wg_step(const WgradArgs& P) {
    WgStep s;
    s.dgi = 8 * P.zsplit;
    const int drow = s.dgi / P.cpr;
    s.dwo = (s.dgi - drow * P.cpr) * 8;
    s.dn = drow / P.rows;
    s.dho = drow - s.dn * P.rows;
    return s;
}

// the same chunk position one tile step later, without divisions
__device__ __forceinline__ void wg_advance(WgChunk& c, const WgStep& s, const WgradArgs& P) {
    c.gi += s.dgi;
    c.live = c.gi < P.nchunks;
    c.wo0 += s.dwo;
    const bool c1 = c.wo0 >= P.cpr * 8;
    c.wo0 -= c1 ? P.cpr * 8 : 0;
    c.ho += s.dho + (c1 ? 1 : 0);
    const bool c2 = c.ho >= P.rows;
    c.ho -= c2 ? P.rows : 0;
    c.n += s.dn + (c2 ? 1 : 0);
}

__device__ __forceinline__ WgChunk wg_chunk(const WgradArgs& P, int tile, int j) {
    WgChunk c;
    const int gi = tile * 8 + j;
    c.live = gi < P.nchunks;
    const int row = gi / P.cpr;
    c.wo0 = (gi - row * P.cpr) * 8;
    c.n = row / P.rows;
    c.ho = row - c.n * P.rows;
    c.gi = gi;
    return c;
}

template <int MODE, int MT, int NT, int TPW, int SW, bool CL = false>
__global__ void __launch_bounds__(WG_THREADS) qconv_wgrad_f16_kernel(const WgradArgs P0) {
    const WgradArgs P = group_view(P0);
    static_assert(TPW == 1 || ((TPW == 3 || TPW == 4) && SW == 1), "shifted copies need unit stride");
    static_assert(!CL || (MT == 2 && NT == 2 && SW == 1 && (TPW == 1 || TPW == 3)), "channels-last staging: 64x64 tiles, unit stride");
    constexpr int CoT = 32 * MT, CiT = 32 * NT;
    constexpr int NL = (MODE == 16) ? 4 : 8;  // accumulators per (tap, tile): components or lanes
    constexpr int KPp = WG16_PITCH;
    constexpr int GE = 4 * MT, XE = 4 * NT;                  // chunks per thread and tile: gradient / input planes
    constexpr int XR = (TPW == 3) ? 5 : (TPW == 4) ? 6 : (SW == 2 ? 8 : 4);   // dwords loaded per input chunk
    extern __shared__ f16x8 lds16[];
    _Float16* gl = reinterpret_cast<_Float16*>(lds16);  // [4][CoT][KPp]
    _Float16* xl = gl + 4 * CoT * KPp;                   // [TPW][4][CiT][KPp]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const int m = lane & 15, kb = lane >> 4;
    // workgroups that share a reduction slice read the same gradient / input rows: keep them on one XCD
    int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int cot = bid % P.co_tiles;  bid /= P.co_tiles;
    const int cit = bid % P.ci_tiles;  bid /= P.ci_tiles;
    const int ngroups = P.groups_per_row * P.Kh;
    const int grp = bid % ngroups;
    const int zi = bid / ngroups;
    const int kh = grp / P.groups_per_row;
    const int kw0 = (grp % P.groups_per_row) * TPW;

    // staging role: chunk j of the tile, planes pg + 32*i of every component
    const int j = tid & 7, pg = tid >> 3;
    const int Ho = P.g.Hd, Wo = P.g.Wd, H = P.x.Hd, W = P.x.Wd;
    const long gplane = (long)Ho * Wo, xplane = (long)H * W;
    const _Float16* gbase = static_cast<const _Float16*>(P.g.base);
    const _Float16* xbase = static_cast<const _Float16*>(P.x.base);
    const int co_first = cot * CoT + pg, ci_first = cit * CiT + pg;
    // channels-last staging role: chunk j, component clq, channels clo*8 .. clo*8 + 7 of both channel tiles
    const int clq = pg >> 3, clo = pg & 7;
    constexpr int NXP = 8 + TPW - 1;  // input pixels a chunk touches over the taps of the group (unit stride)

    // 64x64 channel tiles: one 32x32 MFMA tile per wave (v_mfma_f32_32x32x16_f16 sustains its full rate from a
    // single wave per SIMD, the 16x16 shape does not); smaller tiles: MT x NT tiles of 16x16 per wave
    constexpr bool BIG = (MT == 2 && NT == 2);
    f32x4 acc[BIG ? 1 : TPW][MT][NT][NL];
    f32x16 accb[BIG ? TPW : 1][NL];
#pragma unroll
    for (int t = 0; t < (BIG ? 1 : TPW); ++t)
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int jn = 0; jn < NT; ++jn)
#pragma unroll
                for (int a = 0; a < NL; ++a) acc[t][i][jn][a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < (BIG ? TPW : 1); ++t)
#pragma unroll
        for (int a = 0; a < NL; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) accb[t][a][r] = 0.f;

    u32x4 sg[GE];
    unsigned int sx[CL ? 1 : XE][XR];
    u32x4 cx[CL ? NXP : 1];  // channels-last: the 8 channels of input pixel k of the chunk
    // Flat chunk list: the masks of every chunk of a plane under this workgroup's taps, as the 16-byte AND masks the
    // staging stores use ([chunk][gradient, tap 0, tap 1, ...]; entry P.cpr is all zeros, for chunks that are not
    // staged by vector loads) and as bits ([chunk][taps packed 8 bits each, gradient]).  Pixels q0 .. q0+7 of the
    // plane form a first segment in row r0 from column c0 on and a second one in row r0 + 1 (rows are at least 7
    // pixels long).
    u32x4* fmask = reinterpret_cast<u32x4*>(xl + TPW * 4 * CiT * KPp);
    unsigned int* fbits = reinterpret_cast<unsigned int*>(fmask + (P.cpr + 1) * (TPW + 1));
    if (P.flat) {
        for (int ch = tid; ch <= P.cpr; ch += WG_THREADS) {
            const int q0 = ch * 8, r0 = q0 / Wo, c0 = q0 - r0 * Wo, iw = Wo - c0;
            const int ra = r0 + kh * P.dh - P.pt;
            const bool rowa = ra >= 0 && ra < H, rowb = ra + 1 >= 0 && ra + 1 < H;
            const unsigned int inplane = ch < P.cpr ? interval_bits(0, Ho * Wo - q0) : 0u;
            unsigned int packed = 0u;
            fmask[ch * (TPW + 1)] = expand_half_mask(inplane);
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
                const int dc = (kw0 + t) * P.dw - P.pl;          // input column = output column + dc
                const int lo = dc < 0 ? -dc : 0, hi = W - dc < Wo ? W - dc : Wo;  // valid output columns [lo, hi)
                const unsigned int a = rowa ? interval_bits(lo - c0, hi - c0 < iw ? hi - c0 : iw) : 0u;
                const unsigned int b = rowb ? interval_bits(lo + iw, hi + iw) : 0u;
                const unsigned int bits = (a | b) & inplane;
                fmask[ch * (TPW + 1) + 1 + t] = expand_half_mask(bits);
                packed |= bits << (8 * t);
            }
            if (ch < P.cpr) {
                fbits[2 * ch] = packed;
                fbits[2 * ch + 1] = inplane;
            }
        }
        __syncthreads();
    }

    u32x4 mg;                // keeps the gradient pixels that lie inside their row (flat list: inside the plane)
    u32x4 mx[TPW];           // per tap: keeps the pixels whose input pixel lies inside the image
    unsigned int gbits = 0, xbits[TPW];  // the same as bit masks, whether or not the chunk is filled element by element
    bool careful = false;    // this thread's chunk of the tile in flight is filled element by element

    auto xcol0 = [&](const WgChunk& c) { return c.wo0 * SW + kw0 * P.dw - P.pl; };
    auto xrow = [&](const WgChunk& c) { return c.ho * P.sh + kh * P.dh - P.pt; };
    // element offset of the chunk's first loaded input pixel from its plane's first pixel
    auto xlin = [&](const WgChunk& c) {
        return P.flat ? c.wo0 + (kh * P.dh - P.pt) * W + (kw0 * P.dw - P.pl) : xrow(c) * W + xcol0(c);
    };

    // Loads of one tile: every address is (uniform component/plane-group base) + (one 32-bit element
    // offset per thread), so a tile costs a handful of address instructions.  Chunks outside the
    // reduction space or on padding rows load from offset 0 and are masked to zero; channels beyond
    // the tensor re-read its last channel (their rows of the partial result are never reduced).
    // 32-bit element offsets inside one component: the host guarantees they fit
    const int gimg = P.g.Cs * (int)gplane, ximg = P.x.Cs * (int)xplane;
    // elements from the base to the end of the last image's channels, per component
    const int gcomp = (P.g.N - 1) * gimg + P.g.C * (int)gplane, xcomp = (P.x.N - 1) * ximg + P.x.C * (int)xplane;
    const int xnc = P.x.ncomp;                              // 1 for a real-valued input: components 1..3 are zero
    int gch[MT], xch[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i) gch[i] = (co_first + 32 * i < P.g.C ? co_first + 32 * i : P.g.C - 1) * (int)gplane;
#pragma unroll
    for (int i = 0; i < NT; ++i) xch[i] = (ci_first + 32 * i < P.x.C ? ci_first + 32 * i : P.x.C - 1) * (int)xplane;

    unsigned int lgoff[MT], lxoff[NT];  // load offsets of the tile being fetched
    // channels-last: first channel of this thread's octets (octets beyond the tensor re-read its last one), elements
    // per component, and the distance between two pixels of the tile being fetched (0 where everything is masked:
    // such loads all read the tensor's first bytes)
    const int gch0 = cot * CoT + clo * 8 < P.g.C ? cot * CoT + clo * 8 : P.g.C - 8;
    const int xch0 = cit * CiT + clo * 8 < P.x.C ? cit * CiT + clo * 8 : P.x.C - 8;
    const int gcomp_cl = P.g.N * (int)gplane * P.g.Cs, xcomp_cl = P.x.N * (int)xplane * P.x.Cs;
    int lgstep = 0, lxstep = 0;
    auto prep = [&](const WgChunk& c) {
        bool any_x = c.live;
        if (!P.flat) {
            const int hi = xrow(c), wi0 = xcol0(c);
            const bool rowok = c.live && hi >= 0 && hi < H;
            gbits = c.live ? interval_bits(0, Wo - c.wo0) : 0u;
            const unsigned int window = rowok ? interval_bits<2 * XR>(-wi0, W - wi0) : 0u;  // loaded columns inside the image
            any_x = rowok;
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
                if constexpr (SW == 1) {
                    xbits[t] = (window >> t) & 0xFFu;
                } else {
                    unsigned int b = 0u;
#pragma unroll
                    for (int i = 0; i < 8; ++i) b |= ((window >> (i * SW + t)) & 1u) << i;
                    xbits[t] = b;
                }
            }
        }
        int goff[MT], xoff[NT];
        if constexpr (CL) {
            // element offsets of the chunk's first pixel (gradient) / first loaded pixel (input) at the thread's octet
            goff[0] = (c.n * (int)gplane + (P.flat ? c.wo0 : c.ho * Wo + c.wo0)) * P.g.Cs + gch0;
            xoff[0] = (c.n * (int)xplane + xlin(c)) * P.x.Cs + xch0;
            careful = (c.live && goff[0] + 7 * P.g.Cs + 8 > gcomp_cl) ||
                      (any_x && (xoff[0] < 0 || xoff[0] + (NXP - 1) * P.x.Cs + 8 > xcomp_cl));
        } else {
            const int grow = c.n * gimg + (P.flat ? c.wo0 : c.ho * Wo + c.wo0);
            const int xrow_off = c.n * ximg + xlin(c);
#pragma unroll
            for (int i = 0; i < MT; ++i) goff[i] = grow + gch[i];
#pragma unroll
            for (int i = 0; i < NT; ++i) xoff[i] = xrow_off + xch[i];
            // would any of this thread's vector loads leave the tensors?
            careful = (c.live && goff[MT - 1] + 8 > gcomp) || (any_x && (xoff[0] < 0 || xoff[NT - 1] + 2 * XR > xcomp));
        }
        const bool gok = c.live && !careful, xok = any_x && !careful;
        if constexpr (CL) {
            lgstep = gok ? P.g.Cs : 0;
            lxstep = xok ? P.x.Cs : 0;
        }
        if (P.flat) {  // the masks of a chunk depend on its place in the plane only: looked up
            const u32x4* entry = fmask + (gok ? (c.wo0 >> 3) : P.cpr) * (TPW + 1);
            mg = entry[0];
#pragma unroll
            for (int t = 0; t < TPW; ++t) mx[t] = entry[1 + t];
        } else {
            mg = expand_half_mask(gok ? gbits : 0u);
#pragma unroll
            for (int t = 0; t < TPW; ++t) mx[t] = expand_half_mask(xok ? xbits[t] : 0u);
        }
#pragma unroll
        for (int i = 0; i < (CL ? 1 : MT); ++i) lgoff[i] = (unsigned int)(gok ? goff[i] : 0);
#pragma unroll
        for (int i = 0; i < (CL ? 1 : NT); ++i) lxoff[i] = (unsigned int)(xok ? xoff[i] : 0);
    };
    // the load instructions of a tile, one "slot" each, so that they can be spread over the MFMA blocks:
    // a wave that issues them back to back stalls until the memory pipeline has taken them all
    constexpr int XL = (XR == 4) ? 1 : 2;          // load instructions per input chunk
    constexpr int NLOADS = CL ? 8 + NXP : GE + XE * XL;
    const _Float16* gbase_cl = gbase + clq * P.g.comp_stride;
    const _Float16* xbase_cl = xbase + clq * P.x.comp_stride;
    auto load_slot = [&](int sl) {
        if constexpr (CL) {  // one pixel per slot: the gradient's 8, then the input's
            if (sl < 8) sg[sl] = load16_a2(gbase_cl + lgoff[0] + sl * lgstep);
            else if (sl < NLOADS) cx[sl - 8] = load16_a2(xbase_cl + lxoff[0] + (sl - 8) * lxstep);
        } else if (sl < GE) {
            sg[sl] = load16_a2(gbase + (sl / MT) * P.g.comp_stride + lgoff[sl % MT]);
        } else if (sl < NLOADS) {
            const int e = (sl - GE) / XL, part = (sl - GE) % XL;
            const _Float16* ptr = xbase + ((e / NT) < xnc ? (e / NT) * P.x.comp_stride + lxoff[e % NT] : 0);
            if (part == 0) {
                const u32x4 a = load16_a2(ptr);
                sx[e][0] = a[0]; sx[e][1] = a[1]; sx[e][2] = a[2]; sx[e][3] = a[3];
            } else if constexpr (XR == 5) {
                sx[e][4] = load4_a2(ptr + 8);
            } else if constexpr (XR == 6) {
                const u32x2 b = load8_a2(ptr + 8);
                sx[e][4] = b[0]; sx[e][5] = b[1];
            } else if constexpr (XR == 8) {
                const u32x4 b = load16_a2(ptr + 8);
                sx[e][4] = b[0]; sx[e][5] = b[1]; sx[e][6] = b[2]; sx[e][7] = b[3];
            }
        }
    };

    // element-wise fill of this thread's chunk (only next to the ends of the tensors).  The loads of
    // one plane are independent of each other, so their latencies overlap.
    auto fill_careful = [&](int tile) {
        constexpr int NEL = 7 * SW + TPW;  // input pixels one chunk touches over all taps of the group
        const WgChunk c = wg_chunk(P, tile, j);
        const int glin = P.flat ? c.wo0 : c.ho * Wo + c.wo0, lin = xlin(c);
        if (P.flat) {
            const u32x2 entry = *reinterpret_cast<const u32x2*>(fbits + 2 * (c.wo0 >> 3));
            gbits = c.live ? entry[1] : 0u;
#pragma unroll
            for (int t = 0; t < TPW; ++t) xbits[t] = c.live ? (entry[0] >> (8 * t)) & 0xFFu : 0u;
        }
        if constexpr (CL) {
            const _Float16* gsrc = gbase_cl + ((long)c.n * gplane + glin) * P.g.Cs + gch0;
            const _Float16* xsrc = xbase_cl + ((long)c.n * xplane + lin) * P.x.Cs + xch0;  // (before the tensor where lin < 0: read under its bits only)
#pragma unroll 2
            for (int i = 0; i < 8; ++i) {
#pragma unroll
                for (int c8 = 0; c8 < 8; ++c8)
                    gl[(clq * CoT + clo * 8 + c8) * KPp + j * 8 + i] = ((gbits >> i) & 1u) ? gsrc[(long)i * P.g.Cs + c8] : (_Float16)0;
            }
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
#pragma unroll 2
                for (int i = 0; i < 8; ++i) {
#pragma unroll
                    for (int c8 = 0; c8 < 8; ++c8)
                        xl[((t * 4 + clq) * CiT + clo * 8 + c8) * KPp + j * 8 + i] =
                            ((xbits[t] >> i) & 1u) ? xsrc[(long)(i + t) * P.x.Cs + c8] : (_Float16)0;
                }
            }
            return;
        }
#pragma unroll 2
        for (int e = 0; e < GE; ++e) {
            const int q = e / MT, cc = (e % MT) * 32;
            const int ch = co_first + cc < P.g.C ? co_first + cc : P.g.C - 1;
            const _Float16* src = gbase + q * P.g.comp_stride + ((long)c.n * P.g.Cs + ch) * gplane + glin;
            _Float16 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = ((gbits >> i) & 1u) ? src[i] : (_Float16)0;
#pragma unroll
            for (int i = 0; i < 8; ++i) gl[(q * CoT + cc + pg) * KPp + j * 8 + i] = v[i];
        }
#pragma unroll 2
        for (int e = 0; e < XE; ++e) {
            const int q = e / NT, cc = (e % NT) * 32;
            const int ch = ci_first + cc < P.x.C ? ci_first + cc : P.x.C - 1;
            const _Float16* src = xbase + q * P.x.comp_stride + ((long)c.n * P.x.Cs + ch) * xplane + lin;
            // a pixel that some tap keeps is a pixel of the image; the others are not read
            unsigned int used = 0u;
#pragma unroll
            for (int t = 0; t < TPW; ++t)
#pragma unroll
                for (int i = 0; i < 8; ++i) used |= ((xbits[t] >> i) & 1u) << (i * SW + t);
            _Float16 w[NEL];
#pragma unroll
            for (int k = 0; k < NEL; ++k) w[k] = (q < xnc && ((used >> k) & 1u)) ? src[k] : (_Float16)0;
#pragma unroll
            for (int t = 0; t < TPW; ++t)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    xl[((t * 4 + q) * CiT + cc + pg) * KPp + j * 8 + i] = ((xbits[t] >> i) & 1u) ? w[i * SW + t] : (_Float16)0;
        }
    };

    const int ntiles = P.ntiles;
    const WgStep step = wg_step(P);
    WgChunk nextc = wg_chunk(P, zi, j);
    prep(nextc);
#pragma unroll
    for (int sl = 0; sl < NLOADS; ++sl) load_slot(sl);
    PHX_PHASES_BEGIN(5)
    for (int tile = zi; tile < ntiles; tile += P.zsplit) {
        __syncthreads();
        PHX_STAMP(0)
        if constexpr (CL) {
            // 8 pixels x 8 channels -> 8 channel rows of 8 pixels: dword m of a row pairs pixels 2m and 2m + 1
#pragma unroll
            for (int c8 = 0; c8 < 8; ++c8) {
                u32x4 v;
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    v[d] = __builtin_amdgcn_perm(sg[2 * d + 1][c8 >> 1], sg[2 * d][c8 >> 1], (c8 & 1) ? 0x07060302u : 0x05040100u);
                *reinterpret_cast<u32x4*>(gl + (clq * CoT + clo * 8 + c8) * KPp + j * 8) = v & mg;
            }
#pragma unroll
            for (int t = 0; t < TPW; ++t) {
#pragma unroll
                for (int c8 = 0; c8 < 8; ++c8) {
                    u32x4 v;
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        v[d] = __builtin_amdgcn_perm(cx[t + 2 * d + 1][c8 >> 1], cx[t + 2 * d][c8 >> 1],
                                                     (c8 & 1) ? 0x07060302u : 0x05040100u);
                    *reinterpret_cast<u32x4*>(xl + ((t * 4 + clq) * CiT + clo * 8 + c8) * KPp + j * 8) = v & mx[t];
                }
            }
            if (careful) fill_careful(tile);
        } else {
#pragma unroll
            for (int e = 0; e < GE; ++e) {
                const int q = e / MT, cc = (e % MT) * 32;
                *reinterpret_cast<u32x4*>(gl + (q * CoT + cc + pg) * KPp + j * 8) = sg[e] & mg;
            }
#pragma unroll
            for (int e = 0; e < XE; ++e) {
                const int q = e / NT, cc = (e % NT) * 32;
                unsigned int w[XR];
#pragma unroll
                for (int d = 0; d < XR; ++d) w[d] = q < xnc ? sx[e][d] : 0u;
#pragma unroll
                for (int t = 0; t < TPW; ++t) {
                    u32x4 v;
                    if constexpr (XR == 8) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) v[d] = __builtin_amdgcn_perm(w[2 * d + 1], w[2 * d], 0x05040100u);
                    } else if (t & 1) {  // shifted by an odd number of pixels: halves of two neighbouring dwords
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            v[d] = __builtin_amdgcn_alignbyte(w[(d + (t >> 1) + 1) % XR], w[(d + (t >> 1)) % XR], 2);
                    } else {
#pragma unroll
                        for (int d = 0; d < 4; ++d) v[d] = w[(d + (t >> 1)) % XR];
                    }
                    *reinterpret_cast<u32x4*>(xl + ((t * 4 + q) * CiT + cc + pg) * KPp + j * 8) = v & mx[t];
                }
            }
            if (careful) fill_careful(tile);
        }
        PHX_STAMP(1)
        __syncthreads();
        PHX_STAMP(2)
        // the next tile's loads and masks are issued without a branch (past the end they turn into
        // masked loads of offset 0), so that they interleave with the multiplications below
        wg_advance(nextc, step, P);
        prep(nextc);  // free to mix with the first MFMA block
        PHX_STAMP(3)

        if constexpr (BIG) {
            // blocks b = (K step of 16, tap); lane = (channel row/column lane % 32, K half lane / 32)
            constexpr int NBLK = (WG16_KP / 16) * TPW;
            const int m32 = lane & 31, kb2 = lane >> 5;
            f16x8 gf[2][4], xf[2][4];
            auto read_g = [&](f16x8 (&g)[4], int ks) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    g[q] = *reinterpret_cast<const f16x8*>(gl + (q * CoT + wm * 32 + m32) * KPp + ks * 16 + kb2 * 8);
            };
            auto read_x = [&](f16x8 (&x)[4], int blk) {
                const int ks = blk / TPW, t = blk % TPW;
#pragma unroll
                for (int p = 0; p < 4; ++p)
                    x[p] = *reinterpret_cast<const f16x8*>(xl + ((t * 4 + p) * CiT + wn * 32 + m32) * KPp + ks * 16 + kb2 * 8);
            };
            read_g(gf[0], 0);
            read_x(xf[0], 0);
            constexpr int LPB = (NLOADS + NBLK - 1) / NBLK;  // global loads issued per block
#pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) {
                const int ks = blk / TPW, t = blk % TPW;
#pragma unroll
                for (int sl = blk * LPB; sl < (blk + 1) * LPB; ++sl) load_slot(sl);
                if (blk + 1 < NBLK) {
                    read_x(xf[(blk + 1) & 1], blk + 1);
                    if ((blk + 1) % TPW == 0) read_g(gf[(ks + 1) & 1], ks + 1);
                }
                __builtin_amdgcn_sched_barrier(0);  // the reads of the next block stay ahead of this block's MFMAs
                const f16x8(&x)[4] = xf[blk & 1];
                const f16x8(&g)[4] = gf[ks & 1];
                if constexpr (MODE == 16) {
                    f16x8 nx[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) nx[p] = neg8(x[p]);
#pragma unroll
                    for (int p = 0; p < 4; ++p)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            accb[t][p ^ q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(g[q], qneg(p, q) ? nx[p] : x[p],
                                                                                   accb[t][p ^ q], 0, 0, 0);
                } else {
                    f16x8 L[8], Gl[8];
                    lanes_left(x, L);
                    lanes_grad(g, Gl, (_Float16)0.5f);
#pragma unroll
                    for (int l = 0; l < 8; ++l)
                        accb[t][l] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Gl[l], L[l], accb[t][l], 0, 0, 0);
                }
            }
        } else {
        // MFMA blocks b = (K step, tap, column tile); the operands of block b+1 are read from LDS while
        // block b multiplies.  TPW is exact here (the host picks TPW == 3 only for Kw % 3 == 0).
        constexpr int BPK = TPW * NT;               // blocks per K step
        constexpr int NBLK = (WG16_KP / 32) * BPK;
        f16x8 gf[2][MT][4], xf[2][4];
        auto read_g = [&](f16x8 (&g)[MT][4], int ks) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    g[i][q] = *reinterpret_cast<const f16x8*>(gl + (q * CoT + (wm * MT + i) * 16 + m) * KPp + ks * 32 + kb * 8);
        };
        auto read_x = [&](f16x8 (&x)[4], int blk) {
            const int ks = blk / BPK, t = (blk % BPK) / NT, jn = blk % NT;
#pragma unroll
            for (int p = 0; p < 4; ++p)
                x[p] = *reinterpret_cast<const f16x8*>(xl + ((t * 4 + p) * CiT + (wn * NT + jn) * 16 + m) * KPp + ks * 32 + kb * 8);
        };
        read_g(gf[0], 0);
        read_x(xf[0], 0);
        constexpr int LPB = (NLOADS + NBLK - 1) / NBLK;  // global loads issued per block
#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk) {
            const int ks = blk / BPK, t = (blk % BPK) / NT, jn = blk % NT;
#pragma unroll
            for (int sl = blk * LPB; sl < (blk + 1) * LPB; ++sl) load_slot(sl);
            if (blk + 1 < NBLK) {
                read_x(xf[(blk + 1) & 1], blk + 1);
                if ((blk + 1) % BPK == 0) read_g(gf[(ks + 1) & 1], ks + 1);
            }
            const f16x8(&x)[4] = xf[blk & 1];
            const f16x8(&g)[MT][4] = gf[ks & 1];
            if constexpr (MODE == 16) {
                f16x8 nx[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) nx[p] = neg8(x[p]);
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        if (p >= xnc) continue;  // real-valued input: components 1..3 are zero, their products too
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            acc[t][i][jn][p ^ q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                g[i][q], qneg(p, q) ? nx[p] : x[p], acc[t][i][jn][p ^ q], 0, 0, 0);
                    }
            } else {
                f16x8 L[8];
                lanes_left(x, L);
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    f16x8 Gl[8];
                    lanes_grad(g[i], Gl, (_Float16)0.5f);
#pragma unroll
                    for (int l = 0; l < 8; ++l)
                        acc[t][i][jn][l] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Gl[l], L[l], acc[t][i][jn][l], 0, 0, 0);
                }
            }
        }
            }
        PHX_STAMP(4)
    }

    PHX_PHASES_REPORT("wgrad_f16: barrier / store / barrier / prepare / mfma", 5)
    // partial[z][tap][r][co][ci]
    const int taps = P.Kh * P.Kw;
    const long tap_stride = 4L * P.CoP * P.CiP;
    float* dst = P.partial + (long)zi * taps * tap_stride;
    auto merged = [&](const float (&l)[NL], float (&y)[4]) {
        if constexpr (MODE == 16) {
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = l[r];
        } else {
            merge_right_grad(l, y);
        }
    };
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        float* d = dst + (long)(kh * P.Kw + kw0 + t) * tap_stride;
        if constexpr (BIG) {
            // 32x32 D tile: lane holds column ci = lane % 32, register e holds row 8*(e/4) + 4*(lane/32) + e%4
            const int ci = cit * CiT + wn * 32 + (lane & 31);
            const int co_base = cot * CoT + wm * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float l[NL], y[4];
#pragma unroll
                for (int a = 0; a < NL; ++a) l[a] = accb[t][a][e];
                merged(l, y);
                const int co = co_base + 8 * (e >> 2) + (e & 3);
#pragma unroll
                for (int r = 0; r < 4; ++r) d[((long)r * P.CoP + co) * P.CiP + ci] = y[r];
            }
        } else {
            // 16x16 D tiles: lane holds column ci = lane % 16, rows co = 4*(lane/16) + 0..3
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int jn = 0; jn < NT; ++jn) {
                    const int ci = cit * CiT + (wn * NT + jn) * 16 + m;
                    const int co_base = cot * CoT + (wm * MT + i) * 16 + 4 * kb;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float l[NL], y[4];
#pragma unroll
                        for (int a = 0; a < NL; ++a) l[a] = acc[t][i][jn][a][e];
                        merged(l, y);
#pragma unroll
                        for (int r = 0; r < 4; ++r) d[((long)r * P.CoP + co_base + e) * P.CiP + ci] = y[r];
                    }
                }
        }
    }
}

}  // namespace phx
