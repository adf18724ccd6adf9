// Pointwise quaternion convolution on fp16 matrix cores with the WHOLE packed filter resident in LDS (forward and
// input gradient, 16-product form, channels-first tensors).  For layers whose packed filter fits -- input channels x
// output channels <= 128 x 128 with at most 128 output channels -- this replaces the streaming kernel of
// phx_kernels_pw16.h, whose workgroups meet at a barrier every 16 input channels:
//   * the filter image (K steps x sub-tiles of 32 output channels x 4 components, the layout the streaming kernel
//     consumes stage by stage) is copied to LDS once per workgroup; after that the four waves never synchronise;
//   * a wave owns 32 pixels x ALL output channels x 4 components (up to 16 accumulator tiles, 256 registers: one
//     wave per SIMD), so every activation is read from memory exactly once, by exactly one wave;
//   * the activations of a K step (64 rows of (component, channel) x 32 pixels, 4 KiB) reach a ring of stages that
//     belongs to the wave alone by four register-less copies (global_load_lds, 16 bytes per lane: a lane moves one
//     8-pixel group of one row), one step ahead of the products; the wave waits for its own copies (s_waitcnt) and
//     for nobody else.  The MFMA A operand (8 consecutive channels of one pixel per lane) comes out of the stage by
//     the transposing LDS read (ds_read_b64_tr_b16, see phx_kernels_pw16.h), two reads per operand;
//   * the B operand (filters) is one 16-byte LDS read per (sub-tile, component), read a sub-tile ahead;
//   * results: a lane holds four consecutive pixels per register quad for ONE output channel; one
//     v_permlane32_swap per packed dword between the two lane halves makes that 8 consecutive pixels, stored as
//     16-byte words;
//   * waves are persistent and walk over 32-pixel tiles; where the tiles do not divide among the waves the tiles of
//     the last round are cut along the output channels (one sub-tile of 32 per work item) and spread over all CUs.
// What it buys, measured: the products alone (copies and stores compiled out) take 40 us at 128 -> 128 channels,
// N = 128, 28x28 -- the matrix pipe accepts one v_mfma_f32_32x32x16_f16 per 47 shader clocks on random data, not per
// 32 -- the copies add 6 us, the stores 8, both together 24: reads and writes of 64- and 32-byte runs share a memory
// system that delivers 3.4 TB/s for this mix.  That is where the streaming kernel ends up as well, so by default
// only the problems of at most 32 output channels come here (1.15 - 1.5x faster than the streaming kernel, whose
// workgroup tile is then 256 pixels wide; several workgroups per CU fit).
// Requirements (host): fp16, all four components, unit stride, no padding, Cin a multiple of 16, plane size a multiple
// of 8 (a copy lane's 8 pixels lie in one image), one output-channel tile (Cout <= 32 * WCO), the filter image and
// the rings within 160 KiB of LDS.
#pragma once

#include <type_traits>

#include "phx_kernels_pw16.h"

namespace phx {

constexpr int PWR_STAGE_VEC = 256;  // 16-byte vectors of one activation stage: 64 rows x 32 pixels
constexpr int PWR_STAGES = 2;       // stages per wave

// one accumulator value out of the AGPR file, at the place of its use (left to the register allocator, the sixteen
// tiles of an item are all copied to vector registers where the epilogue begins, which spills)
__device__ __forceinline__ float agpr_value(float a) {
    float r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(a));
    return r;
}

// ADD: the instance that adds P.addend (a tensor laid out like the output; an fp16 addition to the rounded result)
// to what it stores.
template <int WCO, bool ADD = false>
__global__ void __launch_bounds__(WG_THREADS, 1) qconv_pwr_f16_kernel(const PwxArgs P0) {
    const PwxArgs P = group_view(P0);
    extern __shared__ f16x8 lds16[];  // filters [K step][sub-tile][component][lane], then the waves' rings
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, kk = lane >> 5;
    const int HW = P.HW;
    const int nvec = P.nsteps * WCO * 4 * 64;
    f16x8* const ring = lds16 + nvec + wave * (PWR_STAGES * PWR_STAGE_VEC);

    // the filter image, once (waited for below, together with the first activations)
    for (int v = wave * 64; v < nvec; v += WG_THREADS) lds_dma_16(P.wpk + v + lane, lds16 + v);

    const int gw = blockIdx.x * 4 + wave, GW = gridDim.x * 4;  // this wave among all
    // This wave's work list: whole items gw, gw + GW, ... below P.items_whole (neighbouring waves of a workgroup take
    // neighbouring tiles: their rows share cache lines), then sub-tile items.  Sub-tile item s = 0, 1, ... goes to
    // wave (s / workgroups) % 4 of workgroup s % workgroups: a last round of few items spreads over all CUs instead
    // of filling the first ones.  Position m in the list -> (pixel tile, sub-tile, valid); sub < 0 for a whole item.
    const int my_whole = P.items_whole > gw ? (P.items_whole - gw + GW - 1) / GW : 0;
    const int nsub = P.items - P.items_whole, first_sub = (int)blockIdx.x + (int)gridDim.x * wave;
    const int my_sub = nsub > first_sub ? (nsub - first_sub + GW - 1) / GW : 0;
    auto decode = [&](int m, int& tile, int& sub) {
        if (m < my_whole) { tile = gw + m * GW; sub = -1; return true; }
        const int s = first_sub + (m - my_whole) * GW;
        tile = P.items_whole + s / WCO;
        sub = s % WCO;
        return m < my_whole + my_sub;
    };

    // ---- copy side, one K step ahead of the products.  Copy instruction t of a step moves component t: lane l
    // the 8-pixel group l % 4 of channel row l / 4.
    int l_item = 0, l_k = 0;  // (position in the work list)
    long l_off = 0;      // element offset of (this lane's 8-pixel group, its channel row of K step 0) inside a component
    bool l_ok = false;
    auto locate_in = [&](int i) {
        int tile, sub;
        const bool valid = decode(i, tile, sub);
        const int gg = tile * 4 + (lane & 3);
        l_ok = valid && gg < P.TGp;
        const int n = l_ok ? gg / P.GI : 0, gi = gg - n * P.GI;
        l_off = ((long)n * P.CinS + (lane >> 2)) * HW + gi * 8;
    };
    auto issue_stage = [&](int stage) {  // the load cursor's step into `stage`; the cursor moves on
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            // (groups past the last image copy zeros, which nobody multiplies into anything that is stored)
            const _Float16* src = l_ok ? P.in + t * P.in_cs + l_off + (long)(l_k * 16) * HW : zero_ptr<_Float16>();
            lds_dma_16_untracked(src, ring + stage * PWR_STAGE_VEC + t * 64);
        }
        if (++l_k == P.nsteps) {
            l_k = 0;
            locate_in(++l_item);
        }
    };

    // ---- product side.  Transposing reads as in the streaming kernel: sixteen-lane group G = lane / 16 reads
    // channels 8 kk + 4 h .. + 3 (kk = G / 2; h = first / second read of an operand) for pixels 16 (G % 2) .. + 15; as a
    // source lane it points at channel row (lane % 16) / 4 of those four and pixel quad lane % 4.  Rows are 64 bytes.
    const unsigned int xrd = (unsigned int)((kk * 8 + ((lane >> 2) & 3)) * 64 + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2);

    // ---- store side: 8-pixel pieces kk and kk + 2 of the tile's four
    int c_item = 0, c_k = 0, c_sub = -1;
    long oaddr[2];
    bool ovalid[2];
    auto locate_out = [&](int i) {
        int tile;
        const bool valid = decode(i, tile, c_sub);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int gg = tile * 4 + kk + 2 * a;
            ovalid[a] = valid && gg < P.TGp;
            const int n = ovalid[a] ? gg / P.GI : 0;
            oaddr[a] = ((long)n * P.CoutS) * HW + (gg - n * P.GI) * 8;
        }
    };

    f32x16 acc[WCO][4];
    locate_in(l_item);
    locate_out(c_item);
    issue_stage(0);
    wait_vmem_all();
    __syncthreads();  // every wave's share of the filter image is in place
    int cur = 0;            // stage of the current step
    bool landed = true;     // the current step's copies are known to have landed

    // One K step: wait for this wave's copies of the step, request the next step's into the other stage (read a
    // step ago: those reads were consumed by that step's products), read the operands, multiply.  NCO sub-tiles from
    // sub-tile w0 on (whole items: all WCO from 0).
    auto step = [&](int w0, auto nco_tag, auto first_tag) {
        constexpr int NCO = decltype(nco_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;
        if (!landed) wait_vmem_all();
        landed = false;
        __builtin_amdgcn_sched_barrier(0);
        issue_stage(cur ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        const f16x8* wl = lds16 + ((c_k * WCO + w0) * 4) * 64 + lane;
        const f16x8* xs = ring + cur * PWR_STAGE_VEC;
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        f16x8 x[4], w[2][4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const f16x4 lo = lds_read_tr16(xs, xrd + p * 1024), hi = lds_read_tr16(xs, xrd + p * 1024 + 256);
            x[p] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) w[0][r] = wl[r * 64];
#pragma unroll
        for (int wc = 0; wc < NCO; ++wc) {
            if (wc + 1 < NCO) {
#pragma unroll
                for (int r = 0; r < 4; ++r) w[(wc + 1) & 1][r] = wl[((wc + 1) * 4 + r) * 64];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // (the negative blocks of the Hamilton matrix negate the activation operand)
                const f16x8 nx = neg8(x[p]);
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[wc][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qneg(p, q) ? nx : x[p], w[wc & 1][p ^ q],
                                                                       (FIRST && p == 0) ? zero : acc[wc][q], 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) asm volatile("" : "+a"(acc[wc][q]));  // (the accumulators stay in the AGPR file)
        }
        cur ^= 1;
        ++c_k;
    };

    auto store_item = [&](int w0, auto nco_tag) {
        constexpr int NCO = decltype(nco_tag)::value;
        // Stores share the counter of the copies and complete in no fixed order relative to them: the copies of the
        // next step (requested a step ago) are drained first, and the next step then needs no wait of its own.
        wait_vmem_all();
        landed = true;
#pragma unroll
        for (int wc = 0; wc < NCO; ++wc) {
            const int co = (w0 + wc) * 32 + j;
            const bool co_ok = co < P.Cout;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                __builtin_amdgcn_sched_barrier(0);  // (one tile at a time leaves the accumulator file)
                // (an unconditional load -- zeros where there is no bias -- keeps branches out of the epilogue)
                const float bv = (float)*(P.bias ? P.bias + q * P.CoutS + (co_ok ? co : 0) : zero_ptr<_Float16>());
                _Float16* dst = P.out + q * P.out_cs + (long)co * HW;
                u32x4 ad[2];  // (the addend's words are requested before the conversions, which then cover their latency)
                if constexpr (ADD) {
                    const _Float16* asrc = P.addend + q * P.out_cs + (long)co * HW;
#pragma unroll
                    for (int a = 0; a < 2; ++a) ad[a] = (ovalid[a] && co_ok) ? load16_a2(asrc + oaddr[a]) : u32x4{0u, 0u, 0u, 0u};
                }
                unsigned int d[4][2];  // [quad][pair]: pixels 8 g + 4 kk + 2 i, + 1
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        f16x2 h;
                        h[0] = (_Float16)(agpr_value(acc[wc][q][4 * g + 2 * i]) + bv);
                        h[1] = (_Float16)(agpr_value(acc[wc][q][4 * g + 2 * i + 1]) + bv);
                        d[g][i] = __builtin_bit_cast(unsigned int, h);
                    }
#pragma unroll
                for (int a = 0; a < 2; ++a) {  // quads 2a, 2a + 1 -> pixels 16 a + 8 kk .. + 7
                    u32x4 v;
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const auto s = __builtin_amdgcn_permlane32_swap(d[2 * a][i], d[2 * a + 1][i], false, false);
                        v[i] = s[0];
                        v[2 + i] = s[1];
                    }
                    if constexpr (ADD) v = add_halves(v, ad[a]);
                    if (ovalid[a] && co_ok) *reinterpret_cast<u32x4_a2*>(dst + oaddr[a]) = v;
                }
            }
        }
        c_k = 0;
        locate_out(++c_item);
    };

    // whole items, then this wave's sub-tile items (the last round).  An item is a straight sequence -- first step
    // (accumulators start from zero), the other steps, stores -- so that the accumulators never meet at a join of two
    // paths (the whole accumulator file is in use: a join would cost copies through memory).
    auto run_items = [&](int count, auto nco_tag) {
        constexpr int NCO = decltype(nco_tag)::value;
        for (int it = 0; it < count; ++it) {
            const int w0 = NCO == WCO ? 0 : c_sub;
            step(w0, nco_tag, std::true_type());
            int k = 1;
            do {  // (at least once: the host sends no problem with fewer than two K steps here)
                step(w0, nco_tag, std::false_type());
            } while (++k < P.nsteps);
            store_item(w0, nco_tag);
        }
    };
    run_items(my_whole, std::integral_constant<int, WCO>());
    run_items(my_sub, std::integral_constant<int, 1>());
    wait_vmem_all();  // (the copies requested past the last item)
}

}  // namespace phx
