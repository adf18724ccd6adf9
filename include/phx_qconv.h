/*
 * phx_qconv.h -- C ABI of the MI355X (gfx950) quaternion Conv2D / Dense engine.
 *
 * Plain C: pointers, sizes and POD structs only.  Every entry point enqueues work on the given
 * HIP stream and returns without synchronising; tensors live in device memory owned by the caller.
 * A non-zero return value is an error (see phx_status_string); nothing has been enqueued then.
 *
 * Tensor layout (identical to the reference engine's, src/backend/tensor.hpp:527-535 and
 * src/conv2d.hpp:169): activations are NCHW with the four quaternion components stacked on the
 * batch axis, x[4*n, ci, h, w] with component p in rows [p*n, (p+1)*n); filters carry the
 * component outermost, w[4, co, ci, kh, kw] (OIHW) or w[4, co, kh, kw, ci] (OHWI); bias is
 * [4, co].  Dense: x[4*n, ni], w[4, ni, no] (layout IO), bias[4, no].
 *
 * Product convention: y = x (x) w, input on the left (src/algebras.cc:28-49).
 */
#ifndef PHX_QCONV_H
#define PHX_QCONV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* phx_stream_t; /* a hipStream_t; NULL is the default stream */

enum phx_status {
    PHX_OK = 0,
    PHX_ERR_INVALID_ARGUMENT = 1, /* malformed descriptor or null pointer */
    PHX_ERR_NOT_SUPPORTED = 2,    /* valid request outside what the kernels cover */
    PHX_ERR_WORKSPACE = 3,        /* workspace smaller than phx_*_workspace_bytes() */
    PHX_ERR_RUNTIME = 4,          /* HIP runtime reported an error */
    PHX_ERR_SCRATCH_LIMIT = 5     /* phx_qconv2d_fwd_noalloc: the call needs more than PHX_NOALLOC_SCRATCH_BYTES */
};

enum phx_dtype { PHX_F32 = 0, PHX_F16 = 1 };

/* Filter layouts (FilterLayout, src/backend/types.hpp:91-97; dimension order src/backend/conv2d_descriptor.hpp:14-37):
 * the component index is outermost in all of them, [4, O, I, H, W] / [4, O, H, W, I] / [4, H, W, I, O]. */
enum phx_filter_layout { PHX_OIHW = 0, PHX_OHWI = 1, PHX_HWIO = 2 };

/* Dense filter layouts (src/backend/dense_descriptor.hpp:30-37): [4, in, out] or [4, out, in]. */
enum phx_dense_layout { PHX_IO = 0, PHX_OI = 1 };

/* Layout of the activation tensors (DataFormat, src/backend/types.hpp:85; dimension numbers
 * src/backend/tensor.hpp:17-31).  The kernels compute on channels-first planes; a channels-last call
 * transposes its activations into the workspace on the way in and out (two extra passes over each tensor). */
enum phx_data_format { PHX_NCHW = 0, PHX_NHWC = 1 };

/* Algebra of the tensors (Algebra, src/algebras.hpp:17-22; zero is the quaternions here, so that a descriptor filled
 * without this field means what it always meant).  The quaternion algebra runs on the kernels directly.  REAL,
 * COMPLEX and GA_300 run as one quaternion call on rearranged tensors: a GA_300 multivector (blades 1, e1, e2, e3,
 * e12, e13, e23, e123; src/algebras.cc:58-131) is A + e123 B with quaternion-like A = (m0, m4, m5, -m6) and
 * B = (m7, -m3, m2, m1), and (A1 + I B1)(A2 + I B2) = (A1 A2 - B1 B2) + I (A1 B2 + B1 A2), i.e. one quaternion
 * convolution of twice the channel counts.  COMPLEX and REAL run in place on grouped images -- two (four) images
 * of the batch read as one quaternion image, q = z_A + conj(z_B) j, the filter relabelled to (u0, 0, u1, 0) /
 * (w, 0, 0, 0) -- and fall back to an embedding with zero components only for batches that cannot be grouped
 * (odd n; n not a multiple of 4 for REAL).  For these
 * algebras activations have dims * n batch rows (dims = 1, 2, 8), filters are [dims, co, ci, kh, kw] (Dense:
 * [dims, ni, no]), bias [dims, co]; every data format, filter layout and group count of the quaternion path (the
 * reference's generic path is algebra-agnostic in these, src/conv2d.hpp:237-275), no real-valued input. */
enum phx_algebra { PHX_QUATERNION = 0, PHX_REAL = 1, PHX_COMPLEX = 2, PHX_GA_300 = 3 };

/* Which Hamilton-product formulation runs.
 * Mirrors Context::preferSpeedToMemory() (src/backend/backend.hpp:58): the reference's default is
 * the factorized 8-product path (src/conv2d.hpp:167-234), UPSTRIDE_MEMORY_OPTIMIZED=1 selects the
 * 16-product path (src/conv2d.hpp:237-275).
 * PHX_PRODUCT_16 always runs the 16-product kernels.  PHX_PRODUCT_8 is the "prefer speed" setting: the
 * factorized 8-product kernels run wherever they are the faster ones (every fp32 pass; fp16 forward and
 * input gradient with more than one filter tap); the fp16-MFMA filter gradient and fp16-MFMA pointwise
 * passes are faster in 16-product form and run that way (phx_last_kernel_name() tells which ran). */
enum phx_product_mode { PHX_PRODUCT_16 = 16, PHX_PRODUCT_8 = 8 };

/* UPSTRIDE_CONV_FP16_POLICY (src/backend/backend.cc:35-42, src/backend/backend.hpp:60-66).
 * Applies to PHX_F16 tensors only; accumulation is fp32 under every policy.
 *   FULL32      fp32 MFMA in every pass (operands widened while staged)
 *   BACKWARD32  fp16 MFMA forward, fp32 MFMA backward
 *   FULL16      fp16 MFMA in every pass */
enum phx_fp16_policy { PHX_FP16_FULL32 = 0, PHX_FP16_BACKWARD32 = 1, PHX_FP16_FULL16 = 2 };

enum phx_pass { PHX_PASS_FWD = 0, PHX_PASS_BWD_DATA = 1, PHX_PASS_BWD_WEIGHTS = 2 };

/* Quaternion Conv2D geometry; replaces the per-call arguments the reference passes to
 * UpstrideConv2DFunctor / UpstrideConv2DGradFunctor (src/conv2d.hpp:40-58, 72-79, 297-316,
 * 331-339) after Conv2DDescriptor has resolved the padding (src/backend/conv2d_descriptor.hpp:132-174). */
typedef struct phx_qconv_desc {
    int32_t dtype;         /* phx_dtype of every tensor of the call */
    int32_t n;             /* images; activation tensors have 4*n batch rows */
    int32_t ci, co;        /* quaternion channels in / out */
    int32_t h, w;          /* input spatial size */
    int32_t kh, kw;        /* filter size */
    int32_t stride_h, stride_w;
    int32_t dilation_h, dilation_w;
    int32_t pad_top, pad_left, pad_bottom, pad_right;
    int32_t filter_layout; /* phx_filter_layout */
    int32_t product_mode;  /* phx_product_mode */
    int32_t fp16_policy;   /* phx_fp16_policy */
    int32_t has_bias;      /* forward only: bias pointer must be non-null when set */
    int32_t real_input;    /* real-valued input (realValuedInput, src/backend/conv2d_descriptor.hpp:262-278,
                              src/conv2d.hpp:122-164, 384-430): 0 or 1; when set x is [n, ci, h, w] with no
                              imaginary parts, filters, outputs and output gradients stay quaternion-valued, has_bias
                              must be 0 (src/conv2d.hpp:125-127) and
                              phx_qconv2d_bwd_data is refused as the reference refuses it (src/conv2d.hpp:394-398) */
    int32_t groups;        /* grouped convolution: ci and co are the totals, both multiples of groups; the filter is
                              [4, co, ci/groups, kh, kw] (OHWI: [4, co, kh, kw, ci/groups], HWIO: [4, kh, kw, ci/groups,
                              co]); 0 or 1 = ungrouped */
    int32_t data_format;   /* phx_data_format of x, y and their gradients: PHX_NCHW [4n, c, h, w] or PHX_NHWC
                              [4n, h, w, c]; filters and bias are unaffected (filter_layout is separate) */
    int32_t algebra;       /* phx_algebra */
} phx_qconv_desc;

/* Quaternion Dense geometry (src/backend/dense_descriptor.hpp:11-59). */
typedef struct phx_qdense_desc {
    int32_t dtype;
    int32_t n;             /* batch; activation tensors have 4*n rows */
    int32_t ni, no;        /* quaternion features in / out */
    int32_t product_mode;
    int32_t fp16_policy;
    int32_t has_bias;
    int32_t filter_layout; /* phx_dense_layout */
    int32_t algebra;       /* phx_algebra */
} phx_qdense_desc;

const char* phx_status_string(int status);

/* One-time set-up for the device that is current on the calling thread: opts every kernel variant that needs it
 * into more than 64 KiB of dynamic LDS and looks up the device address of the built-in scratch array.  Every
 * compute entry point does the same on its first call with a device current, so calling this is optional --
 * except in front of a stream capture (HIP graphs), where it keeps the set-up calls out of the captured region.
 * Plays the part of the reference's per-device context construction (src/backend/cudnn/context.hpp:57-66,
 * src/backend/cudnn/device.hpp:55-73). */
int phx_init(void);

/* Developer hook: reads the PHX_TUNE_* planner overrides and UPSTRIDE_VERBOSE again (they are otherwise read once,
 * on first use) and forgets the cached plans.  Not to be called while another thread is inside a compute entry
 * point.  No counterpart in the reference, whose Context reads its switches once (src/backend/backend.cc:45-48). */
int phx_tuning_reload(void);

/* The plans (tile choice, reduction slices, packed-image sizes) are kept per distinct problem in a bounded,
 * process-wide cache: a miss that finds more than 200 entries drops all but the 100 most recently used -- the
 * policy of the reference's per-device operation cache (KEEP_TOP_100, src/backend/op_collections.cc:21-59;
 * looked up per descriptor in src/backend/op_collections.hpp:121-144).  Reports the entries held now and the
 * entries dropped so far; either pointer may be null.  Host-only. */
int phx_plan_cache_stats(long* entries, long* evictions);

/* The rearrangement that carries an algebra onto the quaternion kernels: `dims` blades, `halves` quaternion-like
 * parts; quaternion component p of half h is sign[h * 4 + p] * blade[h * 4 + p] (blade -1: the component is zero).
 * Host-only (no GPU work): lets a caller, or a test, check the map against the algebra's sign table
 * (src/algebras.cc:5-145). */
int phx_algebra_map(int algebra, int32_t* dims, int32_t* halves, int32_t blade[8], int32_t sign[8]);

/* Output spatial size for the descriptor's explicit padding (src/utils.cc:42-51). */
int phx_qconv2d_output_hw(const phx_qconv_desc* desc, int32_t* ho, int32_t* wo);

/* Scratch bytes one call of the given pass needs (packed filters, split-K partial sums).  The workspace a caller
 * passes must be 16-byte aligned (any hipMalloc allocation is); a misaligned one is refused with
 * PHX_ERR_INVALID_ARGUMENT. */
size_t phx_qconv2d_workspace_bytes(const phx_qconv_desc* desc, int pass);
size_t phx_qdense_workspace_bytes(const phx_qdense_desc* desc, int pass);

/* y = x (x) w (+ bias).  Replaces UpstrideConv2DFunctor<Device,T>::operator() for the quaternion
 * algebra (src/conv2d.hpp:72-95, 167-275) and the forward custom-kernel hook
 * QuatKernelPointwiseConvForwardFunctor::operator() (src/backend/backend.hpp:163-185). */
int phx_qconv2d_fwd(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* w,
                    const void* bias_or_null, void* y, void* workspace, size_t workspace_bytes);

/* The forward pass for callers that cannot allocate device memory or provide a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * operations always draw their temporaries from the caller's allocator (src/backend/memory_request.hpp:73-114).
 * Same arithmetic and kernels as phx_qconv2d_fwd; what that entry point stages in the caller's workspace (the
 * packed filters; rearranged copies for channels-last, space-to-depth or non-quaternion calls) goes to an array of
 * PHX_NOALLOC_SCRATCH_BYTES that is part of the library's code object: each GPU the library runs on holds its own
 * copy until the process ends.  The call allocates nothing; a descriptor whose forward pass needs more than that
 * (phx_qconv2d_workspace_bytes(desc, PHX_PASS_FWD)) is refused with PHX_ERR_SCRATCH_LIMIT and nothing is
 * enqueued.  All calls on one GPU share that GPU's array, which keeps the previous call's contents (every byte a
 * call reads it has written first): calls that overlap in time on one GPU -- different streams, or different
 * threads -- race on it and must be serialized by the caller. */
#define PHX_NOALLOC_SCRATCH_BYTES (16u << 20)
int phx_qconv2d_fwd_noalloc(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* w,
                            const void* bias_or_null, void* y);

/* dx = g (x) conj(w), spatially transposed.  Replaces the input-gradient half of
 * UpstrideConv2DGradFunctor<Device,T>::operator() (src/conv2d.hpp:331-357, 433-562) and of
 * QuatKernelPointwiseConvBackwardFunctor::operator() (src/backend/backend.hpp:196-220). */
int phx_qconv2d_bwd_data(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad, const void* w,
                         void* dx, void* workspace, size_t workspace_bytes);

/* dw = conj(x) (x) g, reduced over batch and space.  Replaces the filter-gradient half of the
 * same two reference operators. */
int phx_qconv2d_bwd_weights(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* grad,
                            void* dw, void* workspace, size_t workspace_bytes);

/* Filters packed ahead of the passes that read them.  Every forward and input-gradient call above first rewrites
 * the filter into the operand order of the kernel it runs (for the factorized product: into the eight right-hand
 * lanes, the job of decomposeRightInput in the reference, src/backend/cudnn/kernels_quat.cu:34-49, which the
 * reference likewise repeats in every call, src/conv2d.hpp:176-207, 442-495).  A caller whose filter changes once
 * per training step, or never (inference), can do that once: phx_qconv2d_pack_filters writes the images of the
 * forward pass and of the input gradient with ONE kernel launch, and the *_prepacked entry points run the same
 * kernels on them without packing.  No counterpart in the reference's interface.
 *   phx_qconv2d_packed_filter_bytes(desc, pass): bytes of the image for pass PHX_PASS_FWD or PHX_PASS_BWD_DATA;
 *     0 = this descriptor has no prepacked form for that pass (non-quaternion algebra, empty input, the
 *     space-to-depth forward path of strided convolutions with at most 4 input channels, the input gradient of a
 *     real-valued input): use the plain entry point.
 *   phx_qconv2d_pack_filters: either image pointer may be NULL (that image is not made); buffers 16-byte aligned.
 *   An image is valid for the descriptor it was packed for (same sizes, dtype, policy and product mode; and the
 *   same PHX_TUNE_* developer overrides, which select kernels), on any stream ordered after the packing call, until
 *   the filter changes.  Results are bit-identical to the plain
 *   entry points'.  The workspace of a prepacked call is that of the plain call (phx_qconv2d_workspace_bytes). */
size_t phx_qconv2d_packed_filter_bytes(const phx_qconv_desc* desc, int pass);
int phx_qconv2d_pack_filters(const phx_qconv_desc* desc, phx_stream_t stream, const void* w, void* packed_fwd,
                             size_t packed_fwd_bytes, void* packed_bwd_data, size_t packed_bwd_data_bytes);
int phx_qconv2d_fwd_prepacked(const phx_qconv_desc* desc, phx_stream_t stream, const void* x, const void* packed_fwd,
                              size_t packed_fwd_bytes, const void* bias_or_null, void* y, void* workspace,
                              size_t workspace_bytes);
int phx_qconv2d_bwd_data_prepacked(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad,
                                   const void* packed_bwd_data, size_t packed_bwd_data_bytes, void* dx, void* workspace,
                                   size_t workspace_bytes);

/* Input gradient plus a tensor: dx = conv2DBwd's dx + addend, addend shaped and typed like dx and not dx itself.  No
 * counterpart in the reference's interface (src/upstride.hpp:35-51 returns the gradient alone); it is what a framework
 * does next when the convolution's input has a second consumer -- the identity branch of a residual block -- and it
 * saves that elementwise pass: the pointwise fp16 kernels add the tensor in their epilogue, every other path adds it
 * in a pass of its own behind the kernel.  The sum is the tensor type's own addition of the rounded gradient and the
 * addend (fp16: rounded once more), i.e. bit for bit what the separate addition gives.  packed_bwd_data_or_null: the
 * image of phx_qconv2d_pack_filters (then w is not read) or NULL (then w is).  Workspace as phx_qconv2d_bwd_data. */
int phx_qconv2d_bwd_data_add(const phx_qconv_desc* desc, phx_stream_t stream, const void* grad, const void* w,
                             const void* packed_bwd_data_or_null, size_t packed_bwd_data_bytes, const void* addend, void* dx,
                             void* workspace, size_t workspace_bytes);

/* Dense trio.  Replaces UpstrideDenseFunctor / UpstrideDenseGradFunctor for the quaternion
 * algebra (src/dense.hpp:52-62, 77-180, 223-237, 252-377). */
int phx_qdense_fwd(const phx_qdense_desc* desc, phx_stream_t stream, const void* x, const void* w,
                   const void* bias_or_null, void* y, void* workspace, size_t workspace_bytes);
int phx_qdense_bwd_data(const phx_qdense_desc* desc, phx_stream_t stream, const void* grad, const void* w,
                        void* dx, void* workspace, size_t workspace_bytes);
int phx_qdense_bwd_weights(const phx_qdense_desc* desc, phx_stream_t stream, const void* x, const void* grad,
                           void* dw, void* workspace, size_t workspace_bytes);

/* Device plumbing for hosts that do not link the HIP runtime themselves.  Replaces what
 * device::CUDA does for the reference (src/backend/cudnn/device.hpp:13-229: malloc/free on the
 * device, the stream the operations are enqueued on) and the host<->device copies of
 * TensorManipulations<device::CUDA> (src/backend/cudnn/tensor.hpp:19-111). */
int phx_device_count(int32_t* count);
int phx_device_malloc(void** ptr, size_t bytes);
int phx_device_free(void* ptr);
int phx_memcpy_h2d(void* dst, const void* src, size_t bytes, phx_stream_t stream);
int phx_memcpy_d2h(void* dst, const void* src, size_t bytes, phx_stream_t stream);
int phx_memset_zero(void* dst, size_t bytes, phx_stream_t stream);
int phx_stream_create(phx_stream_t* stream);
int phx_stream_destroy(phx_stream_t stream);
int phx_stream_synchronize(phx_stream_t stream);

/* Kernel timing for benchmarks.  phx_profile_enable(capacity > 0) allocates `capacity` HIP event
 * pairs for the process; from then on every compute entry point, from whatever thread, brackets its dominant kernel (the MFMA kernel, not the filter packing or the split-K reduction)
 * with the next pair, recorded on the call's stream, until the pairs run out.  Nothing
 * synchronises while recording.  phx_profile_collect() waits for the recorded pairs, writes their
 * elapsed times in call order, returns how many there were through `count` and rearms the pairs.
 * phx_profile_enable(0) stops recording.  No counterpart in the reference, whose profiler
 * (src/backend/cudnn/kernels.cc:54-85) times candidate launch configurations instead. */
int phx_profile_enable(int capacity);
int phx_profile_collect(float* milliseconds, int max_count, int* count);

/* Name of the kernel variant the last successful call on this thread dispatched to (for
 * profiling and tests); a static string. */
const char* phx_last_kernel_name(void);

#ifdef __cplusplus
}
#endif
#endif
