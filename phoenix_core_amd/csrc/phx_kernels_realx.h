// Filter gradient of a convolution whose input is real-valued (one stored component) and whose channel counts are
// small -- the first layer of a network on images (src/conv2d.hpp:384-430 is the reference's branch for it).
//
// With a real x, dw = conj(x) (x) g is four plain correlations dw_r = corr(x, g_r), and with at most 16 output and a
// dozen input channels the channel tiles of the general kernel (32 x 32 per component pair, one filter row per
// workgroup) are mostly padding.  Here ONE matrix product holds the whole filter gradient:
//   rows    M = (component r, output channel co)      -> 4 x 16 = 64 rows     (A operand: the gradient)
//   columns N = (input channel ci, tap row kh, tap kw) -> up to 192 columns   (B operand: shifted input rows)
//   reduction K = output pixels, one output row (n, oh) per step of the workgroup's loop
// so the gradient is read once (the general kernel reads it once per filter row) and every MFMA row is a real
// output.  Both operands are K-contiguous as they lie in NCHW memory (pixels along a row):
//   * the gradient rows of (n, oh) are copied to LDS as they are;
//   * an input row is copied Kw times, shifted by kw - pl pixels (global loads need only 2-byte alignment), so
//     that column (ci, kh, kw) reads its operand at the same offset as every other column; the Kh input rows that
//     an output row needs stay in a ring of LDS rows (slot = (oh + kh) % Kh), one new row per output row;
//   * the loads of the next output row are issued before the products of the current one.
// A workgroup owns a run of consecutive output rows and writes its partial sums where the split-K reduction of
// the general kernels (reduce_wgrad_kernel) expects them: partial[z][tap][r][co][ci].
// Requirements (host): fp16, unit stride and dilation, Kw <= 4, Co <= 16, Ci * Kh * 4 <= 192, Wo a multiple of 8.
#pragma once

#include "phx_device.h"  // (the kernel itself: phx_launch_wgrad_realx.hip)

namespace phx {

struct RealWgArgs {
    const _Float16* x;   // [N][Ci][H][W]
    const _Float16* g;   // [4][N][Co][Ho][Wo]
    long g_cs;           // elements between gradient components
    float* partial;      // [Z][Kh*Kw][4][CoP][CiP]
    int N, Ci, Co, H, W, Ho, Wo, Kh, Kw, pt, pl;
    int CoP, CiP;
    int rows_per_wg;     // output rows (n, oh) per workgroup
    int ncol;            // B columns in use: Ci * Kh * 4
    int ntiles;          // 32-column tiles: ceil(ncol / 32)
    int pitch;           // LDS row pitch in halves: >= Wo rounded up to 16, = 8 mod 64 (16-byte reads of 16 rows spread over the banks)
};

constexpr int REALX_GI = 4;  // gradient chunks a thread may own per output row (4 * Co * Wo / 8 <= 1024)
constexpr int REALX_XI = 3;  // input chunks a thread may own per new input row (Ci * Kw * Wo / 8 <= 768)

}  // namespace phx
