/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU oracle: a plain-C restatement of the reference engine's CPU path for Conv2D and Dense over
 * its algebras (real, complex, quaternion, GA(3,0,0)).  It exists to check the HIP kernels; it is
 * never linked into, imported by or shipped with the product library.
 *
 * The scalar convolution / matmul arithmetic of the reference lives in oneDNN (an un-vendored git
 * submodule, version unpinned, API usage bounds it to 1.2 <= v < 3.0); it is restated here from
 * its published semantics (cross-correlation with zero padding, plain matmul, alpha=1, beta=0).
 *
 * Pinning status of each group of functions (what independent evidence checks it):
 *   sign tables, product / backprop term order   reference build of src/algebras.cc (oracle/_ref),
 *                                                 known-answer vectors of tests/tests.cpp
 *   generic forward conv / dense                 known-answer vectors of tests/tests.cpp:224-423,
 *                                                 562-648; closed-form Hamilton product; torch CPU
 *   factorized forward                           known-answer vector tests/tests.cpp:292-315;
 *                                                 identity with the generic path
 *   scalar conv / matmul (oneDNN's part)         torch.nn.functional.conv2d / matmul on CPU
 *   backward (generic and factorized)            adjoint identities and finite differences in
 *                                                 fp64, closed forms g*conj(w), conj(x)*g; the
 *                                                 reference holds no backward test vector
 *   padding arithmetic                           tests/tests.cpp:694-727 and the TensorFlow rule
 *   env-switch parsing                           reference build of src/backend/backend.cc
 */
#ifndef QORACLE_H
#define QORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { QO_OK = 0, QO_ERR_ARG = -1, QO_ERR_MEM = -2, QO_ERR_UNSUPPORTED = -3 };

/* algebra numbering of src/algebras.hpp:17-22 */
enum { QO_REAL = 0, QO_COMPLEX = 1, QO_QUATERNION = 2, QO_GA_300 = 3 };

/* padding presets of src/backend/types.hpp:76-80 */
enum { QO_PAD_SAME = 0, QO_PAD_VALID = 1, QO_PAD_EXPLICIT = 2 };

/* per-blade convolution geometry (one scalar convolution) */
typedef struct {
    int n;          /* images per blade */
    int ci, co;     /* channels per blade */
    int h, w;       /* input spatial size */
    int kh, kw;     /* filter size */
    int sh, sw;     /* stride (height, width) */
    int dh, dw;     /* dilation (height, width), 1 = dense filter */
    int pt, pl;     /* zero padding before (top, left) */
    int pb, pr;     /* zero padding after (bottom, right) */
} qo_geom;

/* one entry of a Clifford product sign table (src/algebras.hpp:32-35) */
typedef struct {
    int left, right;
    int positive;
} qo_sign;

typedef struct {
    int dims;
    const qo_sign* table;
    const int* layout;          /* dims+1 row starts */
    const int* backprop_order;  /* dims*dims indices into table */
} qo_algebra_spec;

/* one scalar operation of the unrolled product, in execution order */
typedef struct {
    int left, right, dim;
    int positive;
    int fill; /* 1: result overwrites the destination blade, 0: accumulated with sign */
} qo_term;

const qo_algebra_spec* qo_get_algebra(int algebra);
int qo_multivector_dim(int algebra);
int qo_product_terms(int algebra, qo_term* out);
int qo_backprop_terms(int algebra, qo_term* out);

int qo_out_h(const qo_geom* g);
int qo_out_w(const qo_geom* g);
size_t qo_in_numel(const qo_geom* g);
size_t qo_w_numel(const qo_geom* g);
size_t qo_out_numel(const qo_geom* g);

int qo_padding_preset(int input, int filter, int dilation, int stride, int preset, int* before, int* after);
int qo_output_size(int input, int filter, int dilation, int stride, int before, int after);

/* env-switch semantics of src/backend/backend.cc:17-48; value strings may be NULL (unset) */
int qo_env_memory_optimized(const char* value);
int qo_env_fp16_policy(const char* value); /* 0 full16, 1 backward32, 2 fp32 */

/* closed-form fp64 quaternion convolution built on the textbook Hamilton product */
void qo_qconv2d_fwd_hamilton(const qo_geom* g, const double* x, const double* w, const double* bias, double* y);
void qo_qconv2d_bwd_data_hamilton(const qo_geom* g, const double* w, const double* grad, double* dx);
void qo_qconv2d_bwd_weights_hamilton(const qo_geom* g, const double* x, const double* grad, double* dw);

#define QO_DECLARE(T, S)                                                                                              \
    void qo_scalar_conv2d_fwd##S(const qo_geom*, const T* x, const T* w, const T* bias, T* y);                        \
    void qo_scalar_conv2d_bwd_weights##S(const qo_geom*, const T* x, const T* grad, T* dw);                           \
    void qo_scalar_conv2d_bwd_data##S(const qo_geom*, const T* w, const T* grad, T* dx);                              \
    void qo_scalar_dense_fwd##S(int n, int ni, int no, const T* x, const T* w, const T* bias, T* y);                  \
    void qo_scalar_dense_bwd##S(int n, int ni, int no, const T* x, const T* w, const T* grad, T* dw, T* dx, int);     \
    void qo_decompose_left##S(const T* const in[4], T* const out[8], size_t len);                                     \
    void qo_decompose_right##S(const T* const in[4], T* const out[8], size_t len);                                    \
    void qo_decompose_grad##S(const T* const in[4], T* const out[8], size_t len);                                     \
    void qo_recompose_output##S(const T* const in[8], T* const out[4], size_t len);                                   \
    void qo_recompose_left_grad##S(const T* const in[8], T* const out[4], size_t len);                                \
    void qo_recompose_right_grad##S(const T* const in[8], T* const out[4], size_t len);                               \
    int qo_conv2d_fwd_generic##S(int algebra, int real_in, const qo_geom*, const T* x, const T* w, const T* b, T* y); \
    int qo_conv2d_fwd_factorized##S(const qo_geom*, const T* x, const T* w, const T* b, T* y);                        \
    int qo_conv2d_bwd_generic##S(int algebra, const qo_geom*, const T* x, const T* w, const T* g, T* dw, T* dx, int); \
    int qo_conv2d_bwd_real_input##S(int algebra, const qo_geom*, const T* x, const T* w, const T* g, T* dw);          \
    int qo_conv2d_bwd_factorized##S(const qo_geom*, const T* x, const T* w, const T* g, T* dw, T* dx, int);           \
    int qo_dense_fwd_generic##S(int algebra, int n, int ni, int no, const T* x, const T* w, const T* b, T* y);        \
    int qo_dense_fwd_factorized##S(int n, int ni, int no, const T* x, const T* w, const T* b, T* y);                  \
    int qo_dense_bwd_generic##S(int algebra, int n, int ni, int no, const T* x, const T* w, const T* g, T* dw, T* dx, \
                                int);                                                                                 \
    int qo_dense_bwd_factorized##S(int n, int ni, int no, const T* x, const T* w, const T* g, T* dw, T* dx, int);

QO_DECLARE(float, _f32)
QO_DECLARE(double, _f64)

#ifdef __cplusplus
}
#endif
#endif
