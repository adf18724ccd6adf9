// Filter gradient for a real-valued input with few channels: the kernel described in phx_kernels_realx.h and its launch.
#include "phx_launch.h"

namespace phx {

// A 16-byte chunk of eight halves moved by s halves, zeros moving in: s > 0 drops the first s halves (the chunk
// wanted starts s halves to the right of the one loaded), s < 0 the last -s.  Chunks that stick out of their row are
// loaded from the nearest position inside it and put right with this when they are stored: no second memory access,
// and nothing between a load and its use that would make the compiler wait for loads meant to stay in flight.
__device__ __forceinline__ u32x4 realx_shift_halves(const u32x4 v, int s) {
    if (s == 0) return v;
    unsigned long long lo = v[0] | ((unsigned long long)v[1] << 32), hi = v[2] | ((unsigned long long)v[3] << 32);
    if (s > 0) {
        const int bits = 16 * s;
        if (bits >= 64) { lo = hi >> (bits - 64); hi = 0; }
        else { lo = (lo >> bits) | (hi << (64 - bits)); hi >>= bits; }
    } else {
        const int bits = -16 * s;
        if (bits >= 64) { hi = lo << (bits - 64); lo = 0; }
        else { hi = (hi << bits) | (lo >> (64 - bits)); lo <<= bits; }
    }
    return u32x4{(unsigned int)lo, (unsigned int)(lo >> 32), (unsigned int)hi, (unsigned int)(hi >> 32)};
}

__global__ void __launch_bounds__(WG_THREADS, 2) qconv_wgrad_f16_realx_kernel(const RealWgArgs P) {
    extern __shared__ f16x8 lds16[];
    _Float16* gl = reinterpret_cast<_Float16*>(lds16);   // [64][pitch]: row r * 16 + co
    _Float16* xl = gl + 64 * P.pitch;                     // [ntiles * 32][pitch]: row (ci * Kh + slot) * 4 + kw
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int mt = wave & 1, jt0 = (wave >> 1) * 3;       // a wave: one 32-row tile x three 32-column tiles
    const int m32 = lane & 31, kg = lane >> 5;
    const int cpr = P.Wo >> 3;                            // 16-byte chunks per output row
    const int ksteps = (P.Wo + 15) >> 4;
    const int total_rows = P.N * P.Ho;
    const int row0 = blockIdx.x * P.rows_per_wg;
    const int row1 = (row0 + P.rows_per_wg < total_rows) ? row0 + P.rows_per_wg : total_rows;

    // rows and row tails that no copy ever writes (channels past Co, columns past ncol, taps past Kw, the odd last
    // half of a K step) must read as zeros
    {
        const int nvec = (64 + P.ntiles * 32) * P.pitch / 8;
        const f16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int i = tid; i < nvec; i += WG_THREADS) lds16[i] = zero;
    }

    // what a thread copies per output row does not depend on the row: gradient chunks (r, co, c) ...
    int g_dst[REALX_GI];
    long g_off[REALX_GI];
#pragma unroll
    for (int i = 0; i < REALX_GI; ++i) {
        const int id = tid + i * WG_THREADS;
        const int rc = id / cpr, c = id - rc * cpr;
        const int r = rc / P.Co, co = rc - r * P.Co;
        g_dst[i] = (r < 4) ? (r * 16 + co) * P.pitch + c * 8 : -1;
        g_off[i] = r * P.g_cs + (long)co * P.Ho * P.Wo + c * 8;
    }
    // ... and input chunks (ci, c, kw) of one input row
    int x_dst[REALX_XI], x_shift[REALX_XI];
    long x_off[REALX_XI];
#pragma unroll
    for (int i = 0; i < REALX_XI; ++i) {
        const int id = tid + i * WG_THREADS;
        const int kw = id % P.Kw, t = id / P.Kw;
        const int c = t % cpr, ci = t / cpr;
        x_dst[i] = (ci < P.Ci) ? (ci * P.Kh * 4 + kw) * P.pitch + c * 8 : -1;
        // the chunk wanted starts at column col0; it is loaded from the nearest start inside the row (W >= 8)
        const int col0 = c * 8 + kw - P.pl;
        const int c0 = col0 < 0 ? 0 : (col0 + 8 > P.W ? P.W - 8 : col0);
        x_shift[i] = col0 - c0;
        x_off[i] = (long)ci * P.H * P.W + c0;
    }
    // the B rows a lane reads: column (ci, kh, kw) -> LDS row (ci * Kh + (oh + kh) % Kh) * 4 + kw
    int b_fix[3], b_kh[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int col = (jt0 + j) * 32 + m32;
        const int kw = col & 3, t = col >> 2;
        const int kh = t % P.Kh, ci = t / P.Kh;
        b_kh[j] = (col < P.ncol) ? kh : -1;
        // (columns past ncol: rows that stay zero; column tiles past the last one: any row, their products are dropped)
        b_fix[j] = (col < P.ncol) ? (ci * P.Kh * 4 + kw) : (col < P.ntiles * 32 ? col : 0);
    }

    f32x16 acc[3];
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;

    auto load_g = [&](u32x4 (&r)[REALX_GI], int n, int oh) {
        const _Float16* base = P.g + ((long)n * P.Co * P.Ho + oh) * P.Wo;
        // (every load is issued whatever the item: the number of loads in flight is then a constant, and the wait in
        // front of a row's stores can leave the loads of the row after it in flight)
#pragma unroll
        for (int i = 0; i < REALX_GI; ++i) r[i] = load16_a2(g_dst[i] >= 0 ? base + g_off[i] : P.g);
    };
    auto store_g = [&](const u32x4 (&r)[REALX_GI]) {
#pragma unroll
        for (int i = 0; i < REALX_GI; ++i)
            if (g_dst[i] >= 0) *reinterpret_cast<u32x4*>(gl + g_dst[i]) = r[i];
    };
    // input row ih of image n (zeros where it lies outside the image)
    // input row ih of image n; a row outside the image is stored as zeros (`inside` goes with the registers)
    auto load_x = [&](u32x4 (&r)[REALX_XI], bool& inside, int n, int ih, bool wanted) {
        inside = wanted && ih >= 0 && ih < P.H;
        const _Float16* base = P.x + ((long)n * P.Ci * P.H + (inside ? ih : 0)) * P.W;
#pragma unroll
        for (int i = 0; i < REALX_XI; ++i) r[i] = load16_a2((x_dst[i] >= 0 && inside) ? base + x_off[i] : P.x);
    };
    auto store_x = [&](const u32x4 (&r)[REALX_XI], bool inside, int slot) {
#pragma unroll
        for (int i = 0; i < REALX_XI; ++i) {
            if (x_dst[i] < 0) continue;
            const u32x4 v = inside ? realx_shift_halves(r[i], x_shift[i]) : u32x4{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(xl + x_dst[i] + slot * 4 * P.pitch) = v;
        }
    };

    // Operands of an output row on their way to LDS: loads issued two rows ahead (the products of one row are too
    // short to cover a global load), stored one row ahead.
    struct Pending {
        u32x4 g[REALX_GI], x[REALX_XI];
        int n, oh;
        bool valid, single, inside;  // single: the row continues its image, one new input row completes the ring
    };
    auto issue = [&](Pending& q, int row, bool first) {
        q.valid = row < row1;
        const int rr = q.valid ? row : row0;  // (past the end: the same loads from a row that exists, never stored)
        q.n = rr / P.Ho;
        q.oh = rr - q.n * P.Ho;
        q.single = q.oh > 0 && !first;
        load_g(q.g, q.n, q.oh);
        load_x(q.x, q.inside, q.n, q.oh + P.Kh - 1 - P.pt, q.single);
    };
    auto commit = [&](Pending& q) {
        if (!q.valid) return;
        store_g(q.g);
        if (q.single) {
            store_x(q.x, q.inside, (q.oh + P.Kh - 1) % P.Kh);
        } else {
            for (int kh = 0; kh < P.Kh; ++kh) {  // first row of a workgroup or of an image: the whole ring
                load_x(q.x, q.inside, q.n, q.oh + kh - P.pt, true);
                store_x(q.x, q.inside, (q.oh + kh) % P.Kh);
            }
        }
    };
    // The operands of K step ks + 1 are read while step ks multiplies.  Column tiles past the last one read row 0 and
    // multiply like the others (their accumulators are never written out): no branch anywhere in the loop.
    auto products = [&](int oh) {
        const _Float16* bp[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int brow = b_kh[j] >= 0 ? b_fix[j] + ((oh + b_kh[j]) % P.Kh) * 4 : b_fix[j];
            bp[j] = xl + brow * P.pitch + kg * 8;
        }
        const _Float16* ap = gl + (mt * 32 + m32) * P.pitch + kg * 8;
        f16x8 a = *reinterpret_cast<const f16x8*>(ap), b[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) b[j] = *reinterpret_cast<const f16x8*>(bp[j]);
        for (int ks = 0; ks < ksteps; ++ks) {
            const int kn = (ks + 1 < ksteps) ? ks + 1 : ks;  // (the last step reads its own operands again)
            const f16x8 a2 = *reinterpret_cast<const f16x8*>(ap + kn * 16);
            f16x8 b2[3];
#pragma unroll
            for (int j = 0; j < 3; ++j) b2[j] = *reinterpret_cast<const f16x8*>(bp[j] + kn * 16);
#pragma unroll
            for (int j = 0; j < 3; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[j], acc[j], 0, 0, 0);
            a = a2;
#pragma unroll
            for (int j = 0; j < 3; ++j) b[j] = b2[j];
        }
    };

    Pending pa, pb;
    __syncthreads();  // the zeros are in place
    issue(pa, row0, true);
    commit(pa);
    int oh_lds = pa.valid ? pa.oh : 0;  // the output row (within its image) whose operands are in LDS
    issue(pa, row0 + 1, false);
    for (int row = row0; row < row1; row += 2) {
        __syncthreads();  // row's operands are in LDS
        issue(pb, row + 2, false);
        products(oh_lds);
        __syncthreads();  // every wave is done with them
        commit(pa);
        if (row + 1 >= row1) break;
        oh_lds = pa.oh;
        __syncthreads();
        issue(pa, row + 3, false);
        products(oh_lds);
        __syncthreads();
        commit(pb);
        if (pb.valid) oh_lds = pb.oh;
    }

    // partial[z][tap][r][co][ci]; register e of a tile: row 8 * (e / 4) + 4 * (lane / 32) + e % 4, column lane % 32
    float* out = P.partial + (long)blockIdx.x * P.Kh * P.Kw * 4 * P.CoP * P.CiP;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int col = (jt0 + j) * 32 + m32;
        const int kw = col & 3, t = col >> 2;
        const int kh = t % P.Kh, ci = t / P.Kh;
        if (col >= P.ncol || kw >= P.Kw) continue;
        const int tap = kh * P.Kw + kw;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int m = mt * 32 + 8 * (e >> 2) + 4 * kg + (e & 3);
            const int r = m >> 4, co = m & 15;
            if (co < P.Co) out[(((long)tap * 4 + r) * P.CoP + co) * P.CiP + ci] = acc[j][e];
        }
    }
}

int launch_wgrad_f16_realx(const RealWgArgs& a, int nblocks, size_t lds_bytes, hipStream_t st) {
    constexpr auto kernel = qconv_wgrad_f16_realx_kernel;
    if (!BigLds<kernel>::registered) return -1;  // (more than 64 KiB of dynamic LDS: opted in per device at set-up)
    hipLaunchKernelGGL(kernel, dim3(nblocks), dim3(WG_THREADS), lds_bytes, st, a);
    return 0;
}

}  // namespace phx
