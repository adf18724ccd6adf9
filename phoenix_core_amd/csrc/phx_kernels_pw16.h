// Pointwise (1x1, unit stride, unpadded) quaternion convolution on fp16 matrix cores, forward and input gradient,
// 16-product form: out[q][n][co][px] = sum_p sum_ci s(p,q) * w_{p^q}[co][ci] * in[p][n][ci][px].
//
// A pointwise convolution streams: per output pixel it reads Cin and writes Cout values and multiplies them by a
// filter that is the same everywhere, so the kernel is built around the data path, not around a halo window:
//   * both operands reach LDS by the register-less copy path (global_load_lds, 16 bytes per lane), activations
//     exactly as they lie in NCHW memory -- rows of (component, channel) x consecutive pixels, no transposition,
//     no masks, no staging registers; a ring of stages (one 16-channel K step each) keeps the copies ahead of the
//     matrix instructions (one step here, two in the channels-last kernel), one barrier per step;
//   * the MFMA A operand wants 8 consecutive channels of one pixel per lane, NCHW has consecutive pixels of one
//     channel: the transposition happens on the way from LDS to the registers, by the transposing LDS read of
//     gfx950 (ds_read_b64_tr_b16): sixteen lanes hand in the addresses of sixteen 8-byte runs -- four pixel quads
//     of each of four channel rows -- and lane i receives pixel i of the sixteen with its four channels.  Two
//     such reads are one matrix operand: no vector arithmetic touches the data on its way in.  The 16-byte pieces
//     of a staged row are stored XOR-swizzled by the row number (the copy lanes choose which piece of global
//     memory they fetch), so that the four rows of a read fall into four different bank groups;
//   * the activations are the A operand of the matrix instruction (rows = pixels) and the filters the B operand
//     (columns = output channels), so a lane receives, for ONE output channel, four consecutive pixels per group
//     of four accumulator registers;
//   * stored like that, the 64 lanes of a store instruction would write 32 channel rows x 16 bytes.  So a wave
//     passes each component's 4 KB through a small LDS buffer of its own ([channel][8-pixel piece], rows padded by
//     one piece against bank conflicts) and reads it back with the lanes along the pixels: a store instruction then
//     writes 8 channel rows x 128 bytes (WCO > 1; the 256-pixel tiles of WCO == 1 have no LDS to spare and store
//     their quads directly);
//   * a wave owns 32 output channels x 64 pixels x 4 output components = 8 accumulator tiles (128 registers),
//     so two workgroups fit a CU and one's stores and start-up run under the other's products;
//   * pixels are addressed in groups of 8 (one 16-byte copy lane); an image whose plane is not a multiple of 8
//     pixels has its last group moved back to end at the plane's end (a few pixels are computed twice, with the
//     same result), so no copy ever leaves its row and no lane needs a mask;
//   * workgroups are persistent: each walks over (pixel tile, output-channel tile) items, the copy ring running on
//     across item boundaries.  Where the items do not divide among the workgroups and the last round would keep
//     at most half of them busy, the items of that round are cut in two along the pixels (half items: one of the
//     two 32-pixel column tiles of every wave), so that the round costs half an item instead of a whole one.
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
__device__ __forceinline__ u32x2 add_halves4(const u32x2& a, const u32x2& b) {
    const f16x4 s = __builtin_bit_cast(f16x4, a) + __builtin_bit_cast(f16x4, b);
    return __builtin_bit_cast(u32x2, s);
}

// The transposing LDS read (ds_read_b64_tr_b16).  Within each group of sixteen lanes, lane s hands in the address
// of four consecutive halves M[s][0..3]; lane i receives M[4r + i/4][i%4] for r = 0..3.
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f16x4 lds_read_tr16(const void* lds_base, unsigned int byte_offset) {
    const auto p = reinterpret_cast<__attribute__((address_space(3))) s16x4*>(
        (__attribute__((address_space(3))) char*)lds_base + byte_offset);
    return __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(p));
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
    int items;              // work items: whole items (pixel tiles * co_tiles), the last ones possibly as pairs of half items
    int items_whole;        // NCHW kernel: work items below this index are whole items, the others half items
    int NP;                 // channels-last kernel: pixels in all, N * HW
    int groups;             // grid rows: the groups of a grouped convolution run by this one launch (1 otherwise)
    long g_in, g_w, g_bias, g_out;  // bytes from one group's input / packed filters / bias / output (and addend) to the next group's
};

// the arguments as group blockIdx.y sees them
__device__ __forceinline__ PwxArgs group_view(const PwxArgs& P0) {
    PwxArgs P = P0;
    P.in = static_cast<const _Float16*>(group_shift(static_cast<const void*>(P0.in), P0.g_in));
    P.wpk = static_cast<const f16x8*>(group_shift(static_cast<const void*>(P0.wpk), P0.g_w));
    P.bias = static_cast<const _Float16*>(group_shift(static_cast<const void*>(P0.bias), P0.g_bias));
    P.out = static_cast<_Float16*>(group_shift(static_cast<void*>(P0.out), P0.g_out));
    P.addend = static_cast<const _Float16*>(group_shift(static_cast<const void*>(P0.addend), P0.g_out));
    return P;
}

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
    // NCHW kernel: the filters (from L2: short latency) go through a ring of two stages, one K step ahead of the
    // products; the activations (from HBM) through a ring of their own, two steps ahead where LDS has the room
    // (WCO == 4: 32 + 24 KiB of rings + 18 KiB of store transposition, two workgroups per CU)
    static constexpr bool TSTORE = WCO > 1;      // stores regrouped through LDS into whole channel rows
    static constexpr int RF = 2;                 // filter stages
    static constexpr int RA = (WCO == 4) ? 3 : 2;  // activation stages
    static constexpr int SCRV = 32 * 9;          // 16-byte vectors of a wave's transposition buffer: 32 channels x (8 + 1) pieces
    static constexpr size_t lds_bytes_nchw = ((size_t)RF * WV + (size_t)RA * XV + (TSTORE ? 4 * SCRV : 0)) * 16;
    // swizzle of the 16-byte pieces of staged activation row `row`: slot s of the row holds piece s ^ swz(row)
    // (four consecutive rows, read together by sixteen lanes, then lie in four different quarters of the 64 banks)
    __host__ __device__ static constexpr int swz(int row) { return WPX == 1 ? 4 * ((row >> 1) & 1) : 4 * (row & 3); }
};

// ADD: the instance that adds P.addend to what it stores (the plain instance carries none of that code: the extra
// registers of the addend's prefetch cost the plain kernel 4 % where both were one)
template <int WCO, bool ADD = false>
__global__ void __launch_bounds__(WG_THREADS, 2) qconv_pwx_f16_kernel(const PwxArgs P0) {
    const PwxArgs P = group_view(P0);
    using S = PwxShape<WCO>;
    constexpr int GPT = S::GPT, ROWDW = S::ROWDW, WV = S::WV, XV = S::XV, RF = S::RF, RA = S::RA;
    constexpr int DF = RF - 1, DA = RA - 1;  // steps the filter / activation copies run ahead of the products
    constexpr int RPI = 64 / GPT;      // activation rows one copy instruction covers
    constexpr int PITCH = ROWDW * 4;   // bytes of a staged activation row
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

    // work item i -> (whole item index, half): half < 0 for a whole item, else the column tile (0 / 1) it is cut down to
    auto decode = [&](int i, int& item, int& half) {
        if (i < P.items_whole) { item = i; half = -1; }
        else { item = P.items_whole + ((i - P.items_whole) >> 1); half = (i - P.items_whole) & 1; }
    };

    // ---- copy side: a lane always fills the same slot (row rl of its instruction's rows, slot s_l of that row), i.e.
    // copies the same pixel group of the tile: piece s_l ^ swz(row), and row % 4 does not depend on the instruction.
    // Two cursors run ahead of the products: the filters' (DF steps ahead) and the activations' (DA steps).
    f16x8* const fring = lds16;
    f16x8* const aring = lds16 + RF * WV;
    const int rl = lane / GPT;
    const int g_l = (lane % GPT) ^ S::swz(wave * RPI + rl);
    long xoff = 0;       // element offset of this lane's group inside a component (channel 0)
    bool xok = false;
    int pa_item = wg, pa_k = 0;            // work item / K step of the next activation copies
    int pf_item = wg, pf_k = 0, pf_ct = 0; // ... of the next filter copies, and their channel tile
    auto locate_act = [&](int i) {
        int item, half;
        decode(i, item, half);
        const int tile = item / P.co_tiles;
        const int gg = tile * GPT + g_l;
        xok = i < P.items && gg < P.TGp;
        const int n = gg / P.GI, gi = gg - n * P.GI;
        const int off = min(gi * 8, HW - 8);  // the last group of a plane ends at the plane's end
        xoff = xok ? ((long)n * P.CinS) * HW + off : 0;
    };
    auto locate_filter = [&](int i) {
        int item, half;
        decode(i, item, half);
        pf_ct = item % P.co_tiles;
    };
    // The copies of one step as NPS separate "slots" -- filters of the step DF ahead into filter stage fbuf, then
    // activations of the step DA ahead into activation stage abuf: a wave that issues its copies back to back stalls
    // until the memory pipeline has taken them all, so the product loop deals them out between its matrix
    // instructions.  The last slot of each kind moves its cursor on.  (A half item copies the whole tile: its twin
    // reads the other half of the same stage in another workgroup.)  The cursors run on past the last item -- filters
    // of some valid tile, zeros for activations, into stages nobody reads again -- so that every step issues the same
    // copies, without branches between the matrix instructions, and the waits can count them.
    auto issue_slot = [&](int fbuf, int abuf, int slot) {
        if (slot < S::NWI) {
            const int t = wave + 4 * slot;
            const f16x8* wsrc = P.wpk + ((long)pf_ct * P.nsteps + pf_k) * WV;
            lds_dma_16_untracked(wsrc + t * 64 + lane, fring + fbuf * WV + t * 64);
            if (slot == S::NWI - 1 && ++pf_k == P.nsteps) {
                pf_k = 0;
                pf_item += gridDim.x;
                locate_filter(pf_item);
            }
        } else {
            const int t = wave + 4 * (slot - S::NWI);
            const int r = t * RPI + rl, p = r >> 4, ch = pa_k * 16 + (r & 15);
            // channels past the tensor meet zero filters; they, and groups past the last image, copy zeros
            const _Float16* src = (xok && ch < P.Cin) ? P.in + p * P.in_cs + xoff + (long)ch * HW : zero_ptr<_Float16>();
            lds_dma_16_untracked(src, aring + abuf * XV + t * 64);
            if (slot == S::NPS - 1 && ++pa_k == P.nsteps) {
                pa_k = 0;
                pa_item += gridDim.x;
                locate_act(pa_item);
            }
        }
    };

    // ---- product side.  The activations are the MFMA A operand (rows = pixels), the filters the B operand (columns
    // = output channels).  Lane l of a transposing read: sixteen-lane group G = l / 16 reads channels kk*8 + 4h .. + 3
    // (kk = G / 2; h = first / second read of an operand) for pixels 32m + 16 (G % 2) .. + 15 of the wave's 64;
    // as a source lane it points at channel row (l % 16) / 4 of those four and pixel quad l % 4.  The lane receives
    // D[pixel row][channel column]: column = output channel j of the wave's 32, register e = pixel
    // 32m + 8 (e / 4) + 4 kk + e % 4: four consecutive pixels per register group.
    const int rr = (lane >> 2) & 3, qd = lane & 3;
    const int piece0 = wpx * 8 + 2 * ((lane >> 4) & 1) + (qd >> 1);
    unsigned int xrd[2];  // byte offsets of this lane's source run in a stage's activations, per column tile m
#pragma unroll
    for (int m = 0; m < 2; ++m)
        xrd[m] = (unsigned int)((kk * 8 + rr) * PITCH + (((piece0 + 4 * m) ^ S::swz(rr)) * 16) + (qd & 1) * 8);

    // (TSTORE: after the transposition a lane stores piece lane % 8 of the wave's 8 pixel groups, for channel
    // 8*i + lane / 8 in its i-th store: one address; else a lane stores the quads of all eight groups itself)
    constexpr int NOA = TSTORE ? 1 : 8;
    long oaddr[NOA];    // element offset of an 8-pixel group in an output component
    bool ovalid[NOA];
#pragma unroll
    for (int a = 0; a < NOA; ++a) { oaddr[a] = 0; ovalid[a] = false; }
    int c_item = wg, c_k = 0, c_ct = 0, c_half = -1;
    auto locate_out = [&](int i) {
        int item;
        decode(i, item, c_half);
        const int tile = item / P.co_tiles;
        c_ct = item - tile * P.co_tiles;
#pragma unroll
        for (int a = 0; a < NOA; ++a) {
            const int piece = TSTORE ? (lane & 7) : a;
            const int gg = tile * GPT + wpx * 8 + piece;
            ovalid[a] = gg < P.TGp && (c_half < 0 || (piece >> 2) == c_half);
            const int n = gg / P.GI, gi = gg - n * P.GI;
            oaddr[a] = ((long)n * P.CoutS) * HW + min(gi * 8, HW - 8);
        }
    };

    f32x16 acc[4][2];
    PHX_PHASES_BEGIN(5)
    const int my_items = P.items > wg ? (P.items - wg + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int total_steps = my_items * P.nsteps;
    // this workgroup's whole items come first, its half item (at most one: half items are the last round) last
    const int my_whole = P.items_whole > wg ? (P.items_whole - wg + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int whole_steps = my_whole * P.nsteps;
    locate_act(pa_item);
    locate_filter(pf_item);
    locate_out(c_item);
    // start-up, in the order the waits below count on: filters of the first DF steps, activations of the first DA
#pragma unroll
    for (int st = 0; st < DF; ++st)
#pragma unroll
        for (int slot = 0; slot < S::NWI; ++slot) issue_slot(st, 0, slot);
#pragma unroll
    for (int st = 0; st < DA; ++st)
#pragma unroll
        for (int slot = S::NWI; slot < S::NPS; ++slot) issue_slot(0, st, slot);
    int fcur = 0, acur = 0;  // filter / activation stage of the current step

    // One K step: operands from filter stage fcur and activation stage acur, the copies of the steps ahead dealt out
    // between the matrix instructions.  FIRST: the accumulators start from zero (first step of an item).  HALF: a
    // half item -- only column tile mh is multiplied, into acc[.][0].
    auto products = [&](int mh, auto first_tag, auto half_tag) {
        constexpr bool FIRST = decltype(first_tag)::value, HALF = decltype(half_tag)::value;
        constexpr int NM = HALF ? 1 : 2;
        const int fnext = fcur ^ 1, anext = acur == 0 ? RA - 1 : acur - 1;  // (DF = 1, DA = RA - 1 stages ahead)
        const f16x8* wb = fring + fcur * WV + (wco * 4) * 64 + lane;
        const f16x8* xs = aring + acur * XV;
        f16x8 w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = wb[r * 64];
        f16x8 x[4][NM];
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const unsigned int at = (HALF ? (mh ? xrd[1] : xrd[0]) : xrd[m]) + (unsigned int)(p * 16 * PITCH);
                const f16x4 lo = lds_read_tr16(xs, at), hi = lds_read_tr16(xs, at + 4 * PITCH);
                x[p][m] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            // (the negative blocks of the Hamilton matrix negate the ACTIVATION operand: a value that lives for one
            // component's products, where negated filters would be twelve registers held across the whole step)
            f16x8 nx[NM];
#pragma unroll
            for (int m = 0; m < NM; ++m) nx[m] = neg8(x[p][m]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    acc[q][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qneg(p, q) ? nx[m] : x[p][m], w[p ^ q],
                                                                       (FIRST && p == 0) ? zero : acc[q][m], 0, 0, 0);
                }
                // one copy of the steps ahead behind every few (pairs of) matrix instructions
                constexpr int PAIRS = 16;
                const int pair = p * 4 + q;
#pragma unroll
                for (int slot = 0; slot < S::NPS; ++slot)
                    if (pair == (slot * PAIRS) / S::NPS) {
                        __builtin_amdgcn_sched_barrier(0);
                        issue_slot(fnext, anext, slot);
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
        }
        fcur ^= 1;
        acur = acur == RA - 1 ? 0 : acur + 1;
    };

    // An item is complete: convert, add the bias (BIAS), regroup and store.  HALF: the results of column tile
    // c_half sit in acc[.][0].
    auto store_item = [&](auto bias_tag, auto half_tag) {
        constexpr bool BIAS = decltype(bias_tag)::value, HALF = decltype(half_tag)::value;
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
        wait_vmem_all();  // this wave's copies of the steps ahead: landed
        PHX_STAMP(2)
        const int co = co0 + j;
        const bool co_ok = co < P.Cout;
        char* scr = reinterpret_cast<char*>(lds16 + RF * WV + RA * XV) + wave * (S::SCRV * 16);  // (TSTORE) this wave's own
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float bv = 0.f;
            if constexpr (BIAS) bv = co_ok ? (float)P.bias[q * P.CoutS + co] : 0.f;
            _Float16* dst = P.out + q * P.out_cs + (long)co * HW;
#pragma unroll
            for (int m = 0; m < (HALF ? 1 : 2); ++m) {
                const int mt = HALF ? c_half : m;  // the column tile these registers belong to
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    u32x2 v;
#pragma unroll
                    for (int k2 = 0; k2 < 2; ++k2) {
                        f16x2 h;
                        if constexpr (BIAS) {
                            h[0] = (_Float16)(acc[q][m][g4 * 4 + 2 * k2] + bv);
                            h[1] = (_Float16)(acc[q][m][g4 * 4 + 2 * k2 + 1] + bv);
                        } else {
                            h[0] = (_Float16)acc[q][m][g4 * 4 + 2 * k2];
                            h[1] = (_Float16)acc[q][m][g4 * 4 + 2 * k2 + 1];
                        }
                        v[k2] = __builtin_bit_cast(unsigned int, h);
                    }
                    // pixels 32 mt + 8 g4 + 4 kk .. + 3 of channel j: half kk of piece 4 mt + g4
                    if constexpr (TSTORE) {
                        *reinterpret_cast<u32x2*>(scr + (j * 9 + 4 * mt + g4) * 16 + kk * 8) = v;
                    } else {
                        // (HALF: mt is not a compile-time index; the eight addresses are, so pick among them)
                        long oa = 0;
                        bool ov = false;
#pragma unroll
                        for (int a = 0; a < NOA; ++a)
                            if (a == 4 * mt + g4) { oa = oaddr[a]; ov = ovalid[a]; }
                        if (ov && co_ok) {
                            if constexpr (ADD) v = add_halves4(v, load8_a2(P.addend + q * P.out_cs + (long)co * HW + oa + 4 * kk));
                            *reinterpret_cast<u32x2_a2*>(dst + oa + 4 * kk) = v;
                        }
                    }
                }
            }
            if constexpr (TSTORE) {
                // (LDS serves a wave's accesses in order: the reads see the writes above, and the next
                // component's writes come after these reads)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                u32x4 t[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    t[i] = *reinterpret_cast<const u32x4*>(scr + ((8 * i + (lane >> 3)) * 9 + (lane & 7)) * 16);
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
    };

    // Waiting for a step's copies.  A wave's copies complete in the order of their issue, which is, step by step,
    // filters (of the step DF ahead) then activations (DA ahead): at the top of a step everything but the activation
    // copies issued during the step before has to have landed.  Output stores share the counter and complete in no
    // fixed order relative to the copies: a wave therefore drains its copies BEFORE it issues an item's stores --
    // cheap, they were requested one and two steps earlier -- and then needs no wait for the next step, whose
    // stages that drain has covered; a store still in flight a step later only makes that step's wait longer.
    int covered = 0;  // steps ahead whose copies are known to have landed
#ifdef PHX_PHASE_TIMING
    const long long t_wall0 = wall_clock64(), t_clk0 = clock64();
#endif
    auto step_loop = [&](int gs0, int gs1, auto half_tag) {
        for (int gs = gs0; gs < gs1; ++gs) {
            if (covered > 0) --covered;
            else if (DA >= 2 && gs + 1 < total_steps) __builtin_amdgcn_s_waitcnt(0x0F70 | S::NXI);  // (all but the youngest activation copies)
            else wait_vmem_all();
            PHX_STAMP(0)
            wg_barrier_no_vmem_wait();  // ... for every wave; and every wave is done with the stages the next copies overwrite
            PHX_STAMP(1)
            if (c_k == 0) products(c_half, std::true_type(), half_tag);
            else products(c_half, std::false_type(), half_tag);
            PHX_STAMP(3)
            if (++c_k == P.nsteps) {
                // the item is complete (see above for who holds what)
                if (P.bias) store_item(std::true_type(), half_tag);
                else store_item(std::false_type(), half_tag);
                covered = 1;
                c_k = 0;
                c_item += gridDim.x;
                locate_out(c_item);
                PHX_STAMP(4)
            }
        }
    };
    step_loop(0, whole_steps, std::false_type());
    step_loop(whole_steps, total_steps, std::true_type());
    wait_vmem_all();  // (the copies issued past the last item)
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
__global__ void __launch_bounds__(WG_THREADS, 2) qconv_pwx_nhwc_f16_kernel(const PwxArgs P0) {
    const PwxArgs P = group_view(P0);  // (grid rows: the reduction slices of a sliced pass)
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
            lds_dma_16_untracked(wsrc + t * 64 + lane, sb + t * 64);
        } else {
            const int t = wave + 4 * (slot - S::NWI);
            const int p = t / BLK, b = t % BLK;
            const int gp = p_px0 + b * 32 + c_pxl, ch = p_k * 16 + c_half * 8;
            // channels past the tensor meet zero filters; they, and pixels past the last image, copy zeros
            const _Float16* src = (gp < P.NP && ch < P.Cin) ? P.in + p * P.in_cs + (long)gp * P.CinS + ch : zero_ptr<_Float16>();
            lds_dma_16_untracked(src, sb + WV + t * 64);
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
        wg_barrier_no_vmem_wait();
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
__global__ void __launch_bounds__(WG_THREADS) pack_filters_pwx_kernel(const PackPwxArgs A0) {
    PackPwxArgs A = A0;
    A.base = group_view(A0.base);
    pack_filters_pwx_body<MAP>(A, (long)blockIdx.x * blockDim.x + threadIdx.x, (long)gridDim.x * blockDim.x);
}

}  // namespace phx
