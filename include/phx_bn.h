/* Training-mode batch normalisation (+ optional ReLU) for activations in the engine's layout.
 *
 * No counterpart in the reference engine, which holds no model code: these entry points serve the
 * quaternion ResNet-50 harness that the images/s figure is quoted on (phoenix_core_amd/nn.py,
 * bench.py --workload c5_qresnet50).  A tensor is [rows, C, H, W] with rows = 4N (the four quaternion
 * components stacked on the batch axis, src/backend/tensor.hpp:489-581); every channel is normalised
 * over rows x H x W, i.e. the four components of a quaternion channel share one mean and variance,
 * exactly what torch.nn.BatchNorm2d computes on such a tensor.  HBM-bound: two reads and one write of
 * the activations forward, four reads and one write backward, spread over many workgroups per channel
 * (a library kernel with one workgroup per channel leaves a 16-channel layer on 16 of 256 CUs).
 *
 * Same conventions as phx_qconv.h: device pointers, work enqueued on the given stream, non-zero
 * return = error (phx_status_string), caller-owned workspace of phx_bn_workspace_bytes().
 * gamma, beta, the running statistics and the saved statistics are fp32 whatever the tensor type. */
#ifndef PHX_BN_H
#define PHX_BN_H

#include "phx_qconv.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct phx_bn_desc {
    int32_t dtype;   /* phx_dtype of x, y, dy, dx */
    int32_t rows;    /* batch rows (4N) */
    int32_t c;       /* channels */
    int32_t hw;      /* H * W */
    float eps;
    float momentum;  /* running = (1 - momentum) * running + momentum * batch (variance unbiased) */
    int32_t relu;    /* y = max(0, bn(x)); the backward pass masks dy where bn(x) <= 0 */
} phx_bn_desc;

size_t phx_bn_workspace_bytes(const phx_bn_desc* desc);

/* y = gamma * (x - mean) / sqrt(var + eps) + beta (+ residual) with the batch statistics of x, then the
 * optional ReLU; save_mean and save_invstd ([C] each) receive the statistics for the backward pass;
 * running_mean / running_var ([C]) are updated when non-null.  The residual (same shape as x, e.g. the
 * identity branch of a bottleneck block) is added in front of the ReLU. */
int phx_bn_fwd_train(const phx_bn_desc* desc, phx_stream_t stream, const void* x, const void* residual_or_null,
                     const float* gamma, const float* beta, void* y, float* save_mean, float* save_invstd,
                     float* running_mean_or_null, float* running_var_or_null, void* workspace, size_t workspace_bytes);

/* dx, dgamma, dbeta from x, dy and the saved statistics (beta and the residual are read for the ReLU mask
 * only); with a residual (relu must be set), dresidual receives its gradient, dy behind the ReLU. */
int phx_bn_bwd(const phx_bn_desc* desc, phx_stream_t stream, const void* x, const void* residual_or_null, const void* dy,
               const float* gamma, const float* beta, const float* save_mean, const float* save_invstd, void* dx,
               void* dresidual_or_null, float* dgamma, float* dbeta, void* workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif
