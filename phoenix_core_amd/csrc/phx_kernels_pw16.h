// Pointwise (1x1, unit stride, unpadded) quaternion convolution on fp16 matrix cores, forward and input gradient,
// 16-product form: out[q][n][co][px] = sum_p sum_ci s(p,q) * w_{p^q}[co][ci] * in[p][n][ci][px].
//
// A pointwise convolution streams: per output pixel it reads Cin and writes Cout values and multiplies them by a
// filter that is the same everywhere, so the kernel is built around the data path, not around a halo window:
//   * both operands reach LDS by the register-less copy path (global_load_lds, 16 bytes per lane), activations
//     exactly as they lie in NCHW memory -- rows of (component, channel) x consecutive pixels, no transposition,
//     no masks, no staging registers; a ring of stages (one 16-channel K step each) keeps the copies ahead of the
//     matrix instructions (one step here, two in the channels-last kernel), one barrier per step;
//   * the MFMA B operand wants 8 consecutive channels of one pixel per lane, NCHW has 8 consecutive pixels of one
//     channel: the transposition happens on the way from LDS to the registers.  A lane owns TWO neighbouring
//     pixels: it reads one dword (two pixels) per channel, and byte permutes split the eight dwords of a channel
//     pack into the two operands (one v_perm per matrix instruction);
//   * the activations are the A operand of the matrix instruction (rows = pixels) and the filters the B operand
//     (columns = output channels), so a lane receives, for ONE output channel, eight consecutive pixels per group
//     of four accumulator registers (the two pixels of its pair x four row registers interleave exactly so): one
//     16-byte store per group, no cross-lane shuffle;
//   * stored like that, the 64 lanes of a store instruction would write 32 channel rows x 32 bytes: four
//     instructions to complete a 128-byte line, and the address path handles a line at a time.  So a wave passes
//     each component's 4 KB through a small LDS buffer of its own ([channel][8-pixel piece], rows padded by one
//     piece against bank conflicts) and reads it back with the lanes along the pixels: a store instruction then
//     writes 8 channel rows x 128 bytes (WCO > 1; the 256-pixel tiles of WCO == 1 have no LDS to spare);
//   * a wave owns 32 output channels x 64 pixels x 4 output components = 8 accumulator tiles (128 registers),
//     so two workgroups fit a CU and one's stores and start-up run under the other's products;
//   * pixels are addressed in groups of 8 (one 16-byte copy lane); an image whose plane is not a multiple of 8
//     pixels has its last group moved back to end at the plane's end (a few pixels are computed twice, with the
//     same result), so no copy ever leaves its row and no lane needs a mask;
//   * workgroups are persistent: each walks over (pixel tile, output-channel tile) items, the copy ring running on
//     across item boundaries.
// Requirements (checked on the host): fp16 tensors, all four components present, plane size even and >= 8.
#pragma once

#include <type_traits>

#include "phx_kernels_f16.h"

namespace phx {

// eight fp16 sums (each rounded once, as an fp16 addition is) of two 16-byte vectors of halves
__device__ __forceinline__ u32x4 add_halves(const u32x4& a, const u32x4& b) {
    const f16x8 s = __builtin_bit_cast(f16x8, a) + __builtin_bit_cast(f16x8, b);
    return __builtin_bit_cast(u32x4, s);
}

struct PwxArgs {
    const _Float16* in;     // [4][N][CinS][HW]
    long in_cs;             // elements between input components
    const f16x8* wpk;       // packed filters, see pack_filters_pwx_kernel
    const _Float16* bias;   // [4][CoutS] or null
    _Float16* out;          // [4][N][CoutS][HW]
    long out_cs;
    const _Float16* addend; // NCHW kernel: a tensor laid out like out that is added to the result (fp16 add), or null
    int N, Cin, CinS, Cout, CoutS, HW;
    int GI;                 // 8-pixel groups per image plane: ceil(HW / 8)
    int TGp;                // groups in all: N * GI
    int co_tiles;           // ceil(Cout / (32 * WCO))
    int nsteps;             // ceil(Cin / 16)
    int items;              // pixel tiles * co_tiles
    int NP;                 // channels-last kernel: pixels in all, N * HW
};

template <int WCO>
struct PwxShape {
    static constexpr int WPX = 4 / WCO;          // waves along the pixels
    static constexpr int GPT = 8 * WPX;          // 8-pixel groups per workgroup tile (64 pixels per wave)
    static constexpr int ROWDW = 32 * WPX;       // dwords per staged activation row
    static constexpr int WV = WCO * 4 * 64;      // 16-byte vectors of one filter stage
    static constexpr int XV = 64 * GPT;          // 16-byte vectors of one activation stage: 64 rows (4 components x 16 channels)
    static constexpr int SV = WV + XV;
    static constexpr int R = (WCO == 1) ? 2 : 3; // ring stages of the channels-last kernel (two workgroups per CU: at most 80 KiB each)
    static constexpr int NWI = WCO;              // filter copy instructions per wave and stage
    static constexpr int NXI = 2 * WPX;          // activation copy instructions per wave and stage
    static constexpr int NPS = NWI + NXI;
    static constexpr size_t lds_bytes = (size_t)R * SV * 16;
    // NCHW kernel: a ring of two stages does as well as three (a K step is bound by the copy instructions' issue
    // and the barrier, not by the copies' latency), which leaves room for the store transposition below
    static constexpr bool TSTORE = WCO > 1;      // stores regrouped through LDS into whole channel rows
    static constexpr int RN = 2;
    static constexpr int SCRV = 32 * 9;          // 16-byte vectors of a wave's transposition buffer: 32 channels x (8 + 1) pieces
    static constexpr size_t lds_bytes_nchw = (size_t)RN * SV * 16 + (TSTORE ? 4 * SCRV * 16 : 0);
};

// ADD: the instance that adds P.addend to what it stores (the plain instance carries none of that code: the extra
// registers of the addend's prefetch cost the plain kernel 4 % where both were one)
template <int WCO, bool ADD = false>
__global__ void __launch_bounds__(WG_THREADS, 2) qconv_pwx_f16_kernel(const PwxArgs P) {
    using S = PwxShape<WCO>;
    constexpr int WPX = S::WPX, GPT = S::GPT, ROWDW = S::ROWDW, WV = S::WV, SV = S::SV, R = S::RN, D = R - 1;
    constexpr int RPI = 64 / GPT;  // activation rows one copy instruction covers
    constexpr bool TSTORE = S::TSTORE;
    extern __shared__ f16x8 lds16[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wco = wave % WCO, wpx = wave / WCO;
    const int j = lane & 31, kk = lane >> 5;
    const int HW = P.HW;
    // Workgroups that run at the same time on one XCD take neighbouring items: the 128-byte row pieces of
    // neighbouring pixel tiles share cache lines (rows start at 32-byte, not 128-byte, boundaries), and the channel
    // tiles of one pixel tile read the same activations -- both should meet in one L2.
    const int wg = xcd_remap(blockIdx.x, gridDim.x);

    // ---- copy side: a lane always copies the same pixel group of the tile (64 % GPT == 0)
    const int g_l = lane % GPT, rl = lane / GPT;
    long xoff = 0;       // element offset of this lane's group inside a component (channel 0)
    bool xok = false;
    int p_item = wg, p_k = 0, p_ct = 0;  // item / K step / channel tile the next copy belongs to
    auto locate_copy = [&](int item) {
        const int tile = item / P.co_tiles;
        p_ct = item - tile * P.co_tiles;
        const int gg = tile * GPT + g_l;
        xok = item < P.items && gg < P.TGp;
        const int n = gg / P.GI, gi = gg - n * P.GI;
        const int off = min(gi * 8, HW - 8);  // the last group of a plane ends at the plane's end
        xoff = xok ? ((long)n * P.CinS) * HW + off : 0;
    };
    // The copies of one stage, (p_item, p_k) -> ring buffer buf, as NPS separate "slots": a wave that issues its
    // copies back to back stalls until the memory pipeline has taken them all, so the product loop deals them out
    // between its matrix instructions.  The last slot moves on to the next K step / item.
    auto issue_slot = [&](int buf, int slot) {
        f16x8* sb = lds16 + buf * SV;
        if (slot < S::NWI) {
            const int t = wave + 4 * slot;
            const f16x8* wsrc = P.wpk + ((long)p_ct * P.nsteps + p_k) * WV;
            lds_dma_16(wsrc + t * 64 + lane, sb + t * 64);
        } else {
            const int t = wave + 4 * (slot - S::NWI);
            const int r = t * RPI + rl, p = r >> 4, ch = p_k * 16 + (r & 15);
            // channels past the tensor meet zero filters; they, and groups past the last image, copy zeros
            const _Float16* src = (xok && ch < P.Cin) ? P.in + p * P.in_cs + xoff + (long)ch * HW : zero_ptr<_Float16>();
            lds_dma_16(src, sb + WV + t * 64);
        }
        if (slot == S::NPS - 1 && ++p_k == P.nsteps) {
            p_k = 0;
            p_item += gridDim.x;
            locate_copy(p_item);
        }
    };
    auto issue = [&](int buf) {
#pragma unroll
        for (int slot = 0; slot < S::NPS; ++slot) issue_slot(buf, slot);
    };

    // ---- product side.  The activations are the MFMA A operand (rows = pixels), the filters the B operand (columns
    // = output channels): lane (j, kk) feeds pixels 2j + m (m = 0, 1: two matrix instructions) and channels kk*8.. of
    // the K step on the A side, filter row j on the B side, and receives D[pixel row][channel column]: column =
    // output channel j of the wave's 32, register e = pixel row 8*(e/4) + 4*kk + e%4, i.e. pixel 2*row + m.  The four
    // registers of a group e/4, for m = 0 and 1, are therefore EIGHT CONSECUTIVE pixels 16*(e/4) + 8*kk .. + 7 of one
    // output channel: one 16-byte store, no cross-lane traffic at all.
    // (TSTORE: after the transposition a lane stores piece lane % 8 of the wave's 8 pixel groups, for channel
    // 8*i + lane / 8 in its i-th store: one address)
    constexpr int NOA = TSTORE ? 1 : 4;
    long oaddr[NOA];    // per register group: element offset of its 8-pixel group in an output component
    bool ovalid[NOA];
#pragma unroll
    for (int a = 0; a < NOA; ++a) { oaddr[a] = 0; ovalid[a] = false; }
    int c_item = wg, c_k = 0, c_ct = 0;
    auto locate_out = [&](int item) {
        const int tile = item / P.co_tiles;
        c_ct = item - tile * P.co_tiles;
#pragma unroll
        for (int a = 0; a < NOA; ++a) {
            const int gg = tile * GPT + wpx * 8 + (TSTORE ? (lane & 7) : 2 * a + kk);
            ovalid[a] = gg < P.TGp;
            const int n = gg / P.GI, gi = gg - n * P.GI;
            oaddr[a] = ((long)n * P.CoutS) * HW + min(gi * 8, HW - 8);
        }
    };

    f32x16 acc[4][2];
    const int my_items = P.items > wg ? (P.items - wg + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int total_steps = my_items * P.nsteps;
    locate_copy(p_item);
    locate_out(c_item);
#pragma unroll
    for (int s = 0; s < D; ++s)
        if (s < total_steps) issue(s);

    // One K step: operands from ring buffer buf, the copies of stage gs + D dealt out between the matrix
    // instructions.  FIRST: the accumulators start from zero (first step of an item).
    auto products = [&](int buf, bool more, int nbuf, auto first_tag) {
        constexpr bool FIRST = decltype(first_tag)::value;
        const f16x8* wb = lds16 + buf * SV + (wco * 4) * 64 + lane;
        const unsigned int* xb = reinterpret_cast<const unsigned int*>(lds16 + buf * SV + WV) + (kk * 8) * ROWDW + wpx * 32 + j;
        f16x8 w[4], nw[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = wb[r * 64];
        unsigned int raw[4][8];
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int i = 0; i < 8; ++i) raw[p][i] = xb[(p * 16 + i) * ROWDW];
#pragma unroll
        for (int r = 1; r < 4; ++r) nw[r] = neg8(w[r]);  // the negative blocks of the Hamilton matrix use -w1, -w2, -w3 only
        nw[0] = w[0];
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            u32x4 lo, hi;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                lo[d] = __builtin_amdgcn_perm(raw[p][2 * d + 1], raw[p][2 * d], 0x05040100u);
                hi[d] = __builtin_amdgcn_perm(raw[p][2 * d + 1], raw[p][2 * d], 0x07060302u);
            }
            const f16x8 x0 = __builtin_bit_cast(f16x8, lo), x1 = __builtin_bit_cast(f16x8, hi);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f16x8 f = qneg(p, q) ? nw[p ^ q] : w[p ^ q];
                acc[q][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x0, f, (FIRST && p == 0) ? zero : acc[q][0], 0, 0, 0);
                acc[q][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x1, f, (FIRST && p == 0) ? zero : acc[q][1], 0, 0, 0);
                // one copy of the stage after next behind every few pairs of matrix instructions
                constexpr int PAIRS = 16;
                const int pair = p * 4 + q;
                if (more) {
#pragma unroll
                    for (int slot = 0; slot < S::NPS; ++slot)
                        if (pair == (slot * PAIRS) / S::NPS) {
                            __builtin_amdgcn_sched_barrier(0);
                            issue_slot(nbuf, slot);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                }
            }
        }
    };

    // Waiting for a stage's copies.  A wave's copies complete in order among themselves, so in steady state the
    // copies of (at most D - 1) younger stages may stay in flight.  Output stores share the counter and complete
    // in no fixed order relative to the copies: a wave therefore drains its copies BEFORE it issues an item's
    // stores -- cheap, they were requested one and two steps earlier -- and then needs no wait at all for the next
    // D steps, whose stages that drain has covered; by the time it counts again the stores are long gone.
    int covered = 0;  // steps ahead whose copies are known to have landed
#ifdef PHX_PHASE_TIMING
    const long long t_wall0 = wall_clock64(), t_clk0 = clock64();
#endif
    PHX_PHASES_BEGIN(5)
    for (int gs = 0; gs < total_steps; ++gs) {
        const int buf = gs % R;
        if (covered > 0) --covered;
        else if (D == 2 && gs + 1 < total_steps) __builtin_amdgcn_s_waitcnt(0x0F70 | S::NPS);
        else wait_vmem_all();
        PHX_STAMP(0)
        __syncthreads();  // ... for every wave; and every wave is done with the buffer the next copies overwrite
        PHX_STAMP(1)
        const bool more = gs + D < total_steps;
        const int nbuf = (gs + D) % R;
        if (c_k == 0) products(buf, more, nbuf, std::true_type());
        else products(buf, more, nbuf, std::false_type());
        PHX_STAMP(3)
        if (++c_k == P.nsteps) {
            // the item is complete (see above for who holds what)
            const int co0 = (c_ct * WCO + wco) * 32;
            // (TSTORE) the addend's vectors of a component are requested a component ahead -- the first here, in
            // front of the drain, which then covers their latency; the others in front of the stores of the component
            // before -- so that no store waits for a load of its own
            u32x4 ad[4];
            auto request_addend = [&](int q, u32x4 (&dst)[4]) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int c = 8 * i + (lane >> 3);
                    const bool ok = ovalid[0] && co0 + c < P.Cout;
                    dst[i] = ok ? load16_a2(P.addend + q * P.out_cs + (long)(co0 + c) * HW + oaddr[0]) : u32x4{0u, 0u, 0u, 0u};
                }
            };
            if constexpr (TSTORE && ADD) request_addend(0, ad);
            wait_vmem_all();  // this wave's copies of the next D stages: landed
            covered = D;
            PHX_STAMP(2)
            const int co = co0 + j;
            const bool co_ok = co < P.Cout;
            u32x4* scr = reinterpret_cast<u32x4*>(lds16 + R * SV) + wave * S::SCRV;  // (TSTORE) this wave's own
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float bv = (P.bias && co_ok) ? (float)P.bias[q * P.CoutS + co] : 0.f;
                _Float16* dst = P.out + q * P.out_cs + (long)co * HW;
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    u32x4 v;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        f16x2 h;
                        h[0] = (_Float16)(acc[q][0][g4 * 4 + k] + bv);
                        h[1] = (_Float16)(acc[q][1][g4 * 4 + k] + bv);
                        v[k] = __builtin_bit_cast(unsigned int, h);
                    }
                    if constexpr (TSTORE) scr[j * 9 + 2 * g4 + kk] = v;  // channel j, piece 2*g4 + kk
                    else if (ovalid[g4] && co_ok) {
                        if constexpr (ADD) v = add_halves(v, load16_a2(P.addend + q * P.out_cs + (long)co * HW + oaddr[g4]));
                        *reinterpret_cast<u32x4_a2*>(dst + oaddr[g4]) = v;
                    }
                }
                if constexpr (TSTORE) {
                    // (LDS serves a wave's accesses in order: the reads see the writes above, and the next
                    // component's writes come after these reads)
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    u32x4 t[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        t[i] = scr[(8 * i + (lane >> 3)) * 9 + (lane & 7)];
                        if constexpr (ADD) t[i] = add_halves(t[i], ad[i]);
                    }
                    if constexpr (ADD) {
                        if (q < 3) request_addend(q + 1, ad);  // (in front of this component's stores)
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int c = 8 * i + (lane >> 3);
                        if (ovalid[0] && co0 + c < P.Cout)
                            *reinterpret_cast<u32x4_a2*>(P.out + q * P.out_cs + (long)(co0 + c) * HW + oaddr[0]) = t[i];
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
            }
            c_k = 0;
            c_item += gridDim.x;
            locate_out(c_item);
            PHX_STAMP(4)
        }
    }
#ifdef PHX_PHASE_TIMING
    const long long t_clk1 = clock64(), t_wall1 = wall_clock64();
    if ((blockIdx.x % 61) == 0 && (threadIdx.x & 63) == 0)
        printf("pwx wg %d (%d items): %lld shader clocks, %lld ticks of 10 ns, started at tick %lld\n", (int)blockIdx.x, my_items,
               t_clk1 - t_clk0, t_wall1 - t_wall0, t_wall0 % 1000000);
#endif
    PHX_PHASES_REPORT("pwx: copy wait / barrier / drain before stores / reads+products / stores", 5)
}

// ---------------------------------------------------------------------------------------------
// The same pipeline for CHANNELS-LAST tensors, in[4][N][HW][CinS] -> out[4][N][HW][CoutS] (DataFormat::NHWC of the
// reference, src/backend/tensor.hpp:17-31).  There the 8 consecutive channels of a pixel that the MFMA operand
// wants ARE 16 contiguous bytes, so nothing is transposed anywhere: a copy lane moves (pixel, channel half) of
// the K step to LDS, the B operand is one 16-byte LDS read, and the images need no telling apart (all N * HW
// pixels form one uniformly strided array).  The filters are the A operand here (rows = output channels), so a
// lane receives 4 consecutive output channels per register group at its pixel; one v_permlane32_swap per dword
// between the two lane halves turns its four groups into 16 consecutive channels: two 16-byte stores per tile.
// LDS slot of (pixel p of a 32-pixel block, half h): 2p + (h ^ (p / 8) % 2) -- neighbouring lanes still copy the two
// halves of one pixel (32 contiguous bytes), and the 16 lanes the LDS serves together read 16 different bank groups.
// Requirements (host): channel counts and channel strides multiples of 8.
// ---------------------------------------------------------------------------------------------
template <int WCO>
__global__ void __launch_bounds__(WG_THREADS, 2) qconv_pwx_nhwc_f16_kernel(const PwxArgs P) {
    using S = PwxShape<WCO>;
    constexpr int WPX = S::WPX, WV = S::WV, SV = S::SV, R = S::R, D = R - 1;
    constexpr int PXT = 64 * WPX;     // pixels per workgroup tile
    constexpr int BLK = 2 * WPX;      // 32-pixel blocks per tile (one copy instruction per component each)
    extern __shared__ f16x8 lds16[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wco = wave % WCO, wpx = wave / WCO;
    const int j = lane & 31, kk = lane >> 5;
    const int wg = xcd_remap(blockIdx.x, gridDim.x);

    // ---- copy side
    const int c_pxl = lane >> 1, c_half = (lane & 1) ^ ((c_pxl >> 3) & 1);
    int p_item = wg, p_k = 0, p_ct = 0, p_px0 = 0;
    auto locate_copy = [&](int item) {
        const int tile = item / P.co_tiles;
        p_ct = item - tile * P.co_tiles;
        p_px0 = item < P.items ? tile * PXT : P.NP;  // (past the last item: every pixel out of range)
    };
    auto issue_slot = [&](int buf, int slot) {
        f16x8* sb = lds16 + buf * SV;
        if (slot < S::NWI) {
            const int t = wave + 4 * slot;
            const f16x8* wsrc = P.wpk + ((long)p_ct * P.nsteps + p_k) * WV;
            lds_dma_16(wsrc + t * 64 + lane, sb + t * 64);
        } else {
            const int t = wave + 4 * (slot - S::NWI);
            const int p = t / BLK, b = t % BLK;
            const int gp = p_px0 + b * 32 + c_pxl, ch = p_k * 16 + c_half * 8;
            // channels past the tensor meet zero filters; they, and pixels past the last image, copy zeros
            const _Float16* src = (gp < P.NP && ch < P.Cin) ? P.in + p * P.in_cs + (long)gp * P.CinS + ch : zero_ptr<_Float16>();
            lds_dma_16(src, sb + WV + t * 64);
        }
        if (slot == S::NPS - 1 && ++p_k == P.nsteps) {
            p_k = 0;
            p_item += gridDim.x;
            locate_copy(p_item);
        }
    };
    auto issue = [&](int buf) {
#pragma unroll
        for (int slot = 0; slot < S::NPS; ++slot) issue_slot(buf, slot);
    };

    // ---- product side: lane (j, kk) is pixel j of the wave's two 32-pixel blocks m = 0, 1 and channels kk*8.. of a K step
    int c_item = wg, c_k = 0, c_ct = 0, c_px0 = 0;
    auto locate_out = [&](int item) {
        const int tile = item / P.co_tiles;
        c_ct = item - tile * P.co_tiles;
        c_px0 = tile * PXT + wpx * 64 + j;
    };
    const int xslot = 2 * j + (kk ^ ((j >> 3) & 1));

    f32x16 acc[4][2];
    const int my_items = P.items > wg ? (P.items - wg + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int total_steps = my_items * P.nsteps;
    locate_copy(p_item);
    locate_out(c_item);
#pragma unroll
    for (int s = 0; s < D; ++s)
        if (s < total_steps) issue(s);

    auto products = [&](int buf, bool more, int nbuf, auto first_tag) {
        constexpr bool FIRST = decltype(first_tag)::value;
        const f16x8* wb = lds16 + buf * SV + (wco * 4) * 64 + lane;
        const f16x8* xb = lds16 + buf * SV + WV + (wpx * 2) * 64 + xslot;
        f16x8 w[4], nw[4], x[4][2];
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = wb[r * 64];
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int m = 0; m < 2; ++m) x[p][m] = xb[(p * BLK + m) * 64];
#pragma unroll
        for (int r = 1; r < 4; ++r) nw[r] = neg8(w[r]);
        nw[0] = w[0];
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f16x8 f = qneg(p, q) ? nw[p ^ q] : w[p ^ q];
                acc[q][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f, x[p][0], (FIRST && p == 0) ? zero : acc[q][0], 0, 0, 0);
                acc[q][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f, x[p][1], (FIRST && p == 0) ? zero : acc[q][1], 0, 0, 0);
                constexpr int PAIRS = 16;
                const int pair = p * 4 + q;
                if (more) {
#pragma unroll
                    for (int slot = 0; slot < S::NPS; ++slot)
                        if (pair == (slot * PAIRS) / S::NPS) {
                            __builtin_amdgcn_sched_barrier(0);
                            issue_slot(nbuf, slot);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                }
            }
        }
    };

    int covered = 0;  // (the waiting protocol of qconv_pwx_f16_kernel)
    for (int gs = 0; gs < total_steps; ++gs) {
        const int buf = gs % R;
        if (covered > 0) --covered;
        else if (D == 2 && gs + 1 < total_steps) __builtin_amdgcn_s_waitcnt(0x0F70 | S::NPS);
        else wait_vmem_all();
        __syncthreads();
        const bool more = gs + D < total_steps;
        const int nbuf = (gs + D) % R;
        if (c_k == 0) products(buf, more, nbuf, std::true_type());
        else products(buf, more, nbuf, std::false_type());
        if (++c_k == P.nsteps) {
            wait_vmem_all();
            covered = D;
            // register e of a tile: output channel 8*(e/4) + 4*kk + e%4 of the wave's 32, at this lane's pixel.  After
            // the swaps the lower lane half holds channels 0..15 and the upper half 16..31, in order.
            const int co = (c_ct * WCO + wco) * 32 + 16 * kk;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    unsigned int d[4][2];
#pragma unroll
                    for (int g = 0; g < 4; ++g)
#pragma unroll
                        for (int i = 0; i < 2; ++i) {
                            float a = acc[q][m][4 * g + 2 * i], b = acc[q][m][4 * g + 2 * i + 1];
                            if (P.bias) {
                                const int cb = (c_ct * WCO + wco) * 32 + 8 * g + 4 * kk + 2 * i;
                                a += cb < P.Cout ? (float)P.bias[q * P.CoutS + cb] : 0.f;
                                b += cb + 1 < P.Cout ? (float)P.bias[q * P.CoutS + cb + 1] : 0.f;
                            }
                            f16x2 h;
                            h[0] = (_Float16)a;
                            h[1] = (_Float16)b;
                            d[g][i] = __builtin_bit_cast(unsigned int, h);
                        }
                    u32x4 v0, v1;
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(d[0][i], d[2][i], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(d[1][i], d[3][i], false, false);
                        v0[i] = s02[0]; v0[2 + i] = s02[1];
                        v1[i] = s13[0]; v1[2 + i] = s13[1];
                    }
                    const int gp = c_px0 + 32 * m;
                    _Float16* dst = P.out + q * P.out_cs + (long)gp * P.CoutS + co;
                    if (gp < P.NP && co < P.Cout) *reinterpret_cast<u32x4_a2*>(dst) = v0;
                    if (gp < P.NP && co + 8 < P.Cout) *reinterpret_cast<u32x4_a2*>(dst + 8) = v1;
                }
            }
            c_k = 0;
            c_item += gridDim.x;
            locate_out(c_item);
        }
    }
}

// Filter packing for the kernel above: one 16-byte vector per (output-channel tile of 32*WCO, K step, sub-tile,
// component, lane); lane = (row = lane % 32, kk = lane / 32) holds w_r[row][k*16 + kk*8 + 0..7], zero past either
// channel count.  MAP_DGRAD: rows are the convolution's input channels, the reduction runs over its output
// channels, the filter is conjugated (dx = g (x) conj(w)); the single tap is (khm, kwm) (it differs from (0, 0) only
// for the one phase of a strided pointwise convolution).
struct PackPwxArgs {
    PackArgs base;
    int WCO, nsteps;
};

template <int MAP>
__device__ __forceinline__ void pack_filters_pwx_body(const PackPwxArgs& A, long first, long stride) {
    const PackArgs& P = A.base;
    const long total = (long)P.row_tiles * A.nsteps * A.WCO * 4 * 64;
    const _Float16* w = static_cast<const _Float16*>(P.w);
    f16x8* outv = reinterpret_cast<f16x8*>(P.out);
    for (long idx = first; idx < total; idx += stride) {
        const int lane = idx & 63;
        long s = idx >> 6;
        const int r = s & 3; s >>= 2;
        const int wco = s % A.WCO; s /= A.WCO;
        const int k = s % A.nsteps;
        const int tile = s / A.nsteps;
        const int row = (tile * A.WCO + wco) * 32 + (lane & 31);
        const int kh = (MAP == MAP_DGRAD) ? P.khm : 0, kw = (MAP == MAP_DGRAD) ? P.kwm : 0;
        const float sgn = (MAP == MAP_DGRAD && r > 0) ? -1.f : 1.f;
        f16x8 vec;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int red = k * 16 + (lane >> 5) * 8 + i;
            float v = 0.f;
            if (row < P.rows && red < P.red) {
                const int o = (MAP == MAP_DGRAD) ? red : row;
                const int in = (MAP == MAP_DGRAD) ? row : red;
                v = sgn * (float)w[r * P.wcs + o * P.so + in * P.si + kh * P.skh + kw * P.skw];
            }
            vec[i] = (_Float16)v;
        }
        outv[idx] = vec;
    }
}

template <int MAP>
__global__ void __launch_bounds__(WG_THREADS) pack_filters_pwx_kernel(const PackPwxArgs A) {
    pack_filters_pwx_body<MAP>(A, (long)blockIdx.x * blockDim.x + threadIdx.x, (long)gridDim.x * blockDim.x);
}

}  // namespace phx
