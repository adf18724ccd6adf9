/* 3x3 max pooling with stride 2 and padding 1 (the pooling layer behind a ResNet stem), forward and backward.
 *
 * No counterpart in the reference engine, which holds no model code: like include/phx_bn.h these entry points serve
 * the quaternion ResNet-50 harness that the images/s figure is quoted on (phoenix_core_amd/nn.py,
 * bench.py --workload c5_qresnet50).  A tensor is `planes` images of H x W (planes = rows x channels of an NCHW
 * tensor); the output is planes x Ho x Wo with Ho = (H - 1) / 2 + 1, Wo = (W - 1) / 2 + 1.  The forward pass also
 * writes, per output element, which of the window's nine positions held the maximum (0..8, row-major, the first one
 * on ties -- the choice torch.nn.functional.max_pool2d makes); the backward pass gathers: every input element sums
 * (in fp32) the output gradients of the at most four windows that selected it, in row-major window order.  HBM-bound.
 * Conventions as in phx_qconv.h. */
#ifndef PHX_POOL_H
#define PHX_POOL_H

#include "phx_qconv.h"

#ifdef __cplusplus
extern "C" {
#endif

int phx_maxpool3x3s2_fwd(int32_t dtype, int64_t planes, int32_t h, int32_t w, phx_stream_t stream, const void* x, void* y,
                         uint8_t* index);
int phx_maxpool3x3s2_bwd(int32_t dtype, int64_t planes, int32_t h, int32_t w, phx_stream_t stream, const void* dy,
                         const uint8_t* index, void* dx);

#ifdef __cplusplus
}
#endif
#endif
