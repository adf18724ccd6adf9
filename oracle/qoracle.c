/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the quaternion Conv2D / Dense path.
 * See qoracle.h for what this restates and how each part is pinned.
 * Build: gcc -O2 -fopenmp -shared -fPIC qoracle.c -o libqoracle.so   (oracle/build.py)
 */
#include "qoracle.h"

#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------
 * Sign tables.  The reference lists, for every output blade, one entry per left blade in
 * increasing order (src/algebras.cc:12-145); the entries are derived here from the defining
 * relations of each algebra instead of being carried as literals, and compared entry by entry
 * with the reference's tables by the tests when the reference build is available.
 * ---------------------------------------------------------------------------------------------- */

static qo_sign tab_real[1], tab_complex[4], tab_quat[16], tab_ga300[64];
static int lay_real[2], lay_complex[3], lay_quat[5], lay_ga300[9];

/* evaluation orders for the backward pass: the first `dims` entries are positive terms covering
 * every left and every right blade once (src/algebras.cc:10, 26, 53, 141-146) */
static const int bp_real[] = {0};
static const int bp_complex[] = {2, 3, 0, 1};
static const int bp_quat[] = {10, 11, 12, 13, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 14, 15};
static const int bp_ga300[] = {0,  1,  2,  21, 22, 23, 44, 59, 3,  4,  5,  6,  7,  8,  9,  10, 11, 12, 13, 14, 15, 16,
                               17, 18, 19, 20, 24, 25, 26, 27, 28, 29, 30, 31, 32, 33, 34, 35, 36, 37, 38, 39, 40, 41,
                               42, 43, 45, 46, 47, 48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 60, 61, 62, 63};

static qo_algebra_spec specs[4] = {
    {1, tab_real, lay_real, bp_real},
    {2, tab_complex, lay_complex, bp_complex},
    {4, tab_quat, lay_quat, bp_quat},
    {8, tab_ga300, lay_ga300, bp_ga300},
};
static int tables_ready = 0;

/* e_a * e_b = sign * e_result for the quaternion basis {1, i, j, k} with i*j = k */
static void quat_basis_mul(int a, int b, int* result, int* sign) {
    if (a == 0) { *result = b; *sign = 1; return; }
    if (b == 0) { *result = a; *sign = 1; return; }
    if (a == b) { *result = 0; *sign = -1; return; }
    *result = 6 - a - b;                     /* the remaining imaginary unit */
    *sign = ((b - a + 3) % 3 == 1) ? 1 : -1; /* cyclic order 1 -> 2 -> 3 -> 1 is positive */
}

/* Cl(3,0) blades as bit masks over {e1, e2, e3}; reference blade order 1, e1, e2, e3, e12, e13, e23, e123 */
static const int ga300_mask[8] = {0, 1, 2, 4, 3, 5, 6, 7};

static void ga300_basis_mul(int a, int b, int* result, int* sign) {
    const int ma = ga300_mask[a], mb = ga300_mask[b];
    int swaps = 0;
    for (int t = ma >> 1; t; t >>= 1) swaps += __builtin_popcount(t & mb);
    const int mr = ma ^ mb; /* all generators square to +1 */
    for (int i = 0; i < 8; ++i)
        if (ga300_mask[i] == mr) *result = i;
    *sign = (swaps & 1) ? -1 : 1;
}

typedef void (*basis_mul_fn)(int, int, int*, int*);

static void real_basis_mul(int a, int b, int* r, int* s) { (void)a; (void)b; *r = 0; *s = 1; }
static void complex_basis_mul(int a, int b, int* r, int* s) { *r = a ^ b; *s = (a && b) ? -1 : 1; }

static void build_table(int dims, basis_mul_fn mul, qo_sign* table, int* layout) {
    int k = 0;
    for (int dim = 0; dim < dims; ++dim) {
        layout[dim] = k;
        for (int left = 0; left < dims; ++left)
            for (int right = 0; right < dims; ++right) {
                int res = -1, sign = 0;
                mul(left, right, &res, &sign);
                if (res == dim) {
                    table[k].left = left;
                    table[k].right = right;
                    table[k].positive = sign > 0;
                    ++k;
                }
            }
    }
    layout[dims] = k;
}

static void ensure_tables(void) {
    if (tables_ready) return;
    build_table(1, real_basis_mul, tab_real, lay_real);
    build_table(2, complex_basis_mul, tab_complex, lay_complex);
    build_table(4, quat_basis_mul, tab_quat, lay_quat);
    build_table(8, ga300_basis_mul, tab_ga300, lay_ga300);
    tables_ready = 1;
}

const qo_algebra_spec* qo_get_algebra(int algebra) {
    if (algebra < 0 || algebra > 3) return NULL;
    ensure_tables();
    return &specs[algebra];
}

/* src/algebras.hpp:27 */
int qo_multivector_dim(int algebra) {
    const qo_algebra_spec* s = qo_get_algebra(algebra);
    return s ? s->dims : QO_ERR_ARG;
}

/* Unrolls BinaryOperation::product (src/algebras.hpp:114-132): per output blade, the first table
 * entry fills the blade, the others are accumulated with their sign. */
int qo_product_terms(int algebra, qo_term* out) {
    const qo_algebra_spec* s = qo_get_algebra(algebra);
    if (!s) return QO_ERR_ARG;
    int k = 0;
    for (int dim = 0; dim < s->dims; ++dim) {
        const qo_sign* row = s->table + s->layout[dim];
        if (!row[0].positive) return QO_ERR_UNSUPPORTED; /* "Not implemented" in the reference */
        for (int t = 0; t < s->dims; ++t) {
            out[k].left = row[t].left;
            out[k].right = row[t].right;
            out[k].dim = dim;
            out[k].positive = row[t].positive;
            out[k].fill = (t == 0);
            ++k;
        }
    }
    return k;
}

/* Unrolls BinaryOperation::productBackprop (src/algebras.hpp:140-167) */
int qo_backprop_terms(int algebra, qo_term* out) {
    const qo_algebra_spec* s = qo_get_algebra(algebra);
    if (!s) return QO_ERR_ARG;
    const int total = s->layout[s->dims];
    for (int i = 0; i < total; ++i) {
        const int j = s->backprop_order[i];
        int dim = 0;
        while (dim < s->dims && j >= s->layout[dim + 1]) ++dim;
        out[i].left = s->table[j].left;
        out[i].right = s->table[j].right;
        out[i].dim = dim;
        out[i].positive = s->table[j].positive;
        out[i].fill = (i < s->dims);
        if (out[i].fill && !out[i].positive) return QO_ERR_UNSUPPORTED;
    }
    return total;
}

/* ------------------------------------------------------------------------------------------------
 * Shape arithmetic
 * ---------------------------------------------------------------------------------------------- */

/* src/utils.cc:10-39 (TensorFlow's windowed-output rule) */
int qo_padding_preset(int input, int filter, int dilation, int stride, int preset, int* before, int* after) {
    const int effective = (filter - 1) * dilation + 1;
    if (preset == QO_PAD_VALID) {
        *before = *after = 0;
        return (input - effective + stride) / stride;
    }
    if (preset == QO_PAD_SAME) {
        const int out = (input + stride - 1) / stride;
        int needed = (out - 1) * stride + effective - input;
        if (needed < 0) needed = 0;
        *before = needed / 2; /* the odd sample goes after */
        *after = needed - *before;
        return out;
    }
    return QO_ERR_ARG; /* the reference throws "Invalid padding" for EXPLICIT here */
}

/* src/utils.cc:42-51 */
int qo_output_size(int input, int filter, int dilation, int stride, int before, int after) {
    const int effective = (filter - 1) * dilation + 1;
    return (input + before + after - effective + stride) / stride;
}

int qo_out_h(const qo_geom* g) { return qo_output_size(g->h, g->kh, g->dh, g->sh, g->pt, g->pb); }
int qo_out_w(const qo_geom* g) { return qo_output_size(g->w, g->kw, g->dw, g->sw, g->pl, g->pr); }
size_t qo_in_numel(const qo_geom* g) { return (size_t)g->n * g->ci * g->h * g->w; }
size_t qo_w_numel(const qo_geom* g) { return (size_t)g->co * g->ci * g->kh * g->kw; }
size_t qo_out_numel(const qo_geom* g) { return (size_t)g->n * g->co * qo_out_h(g) * qo_out_w(g); }

/* ------------------------------------------------------------------------------------------------
 * Environment switches: src/backend/backend.cc:17-48
 * ---------------------------------------------------------------------------------------------- */

int qo_env_memory_optimized(const char* value) { return value ? (strtol(value, NULL, 10) > 0) : 0; }

int qo_env_fp16_policy(const char* value) {
    if (value && strcmp(value, "full16") == 0) return 0;
    if (value && strcmp(value, "backward32") == 0) return 1;
    return 2;
}

/* ------------------------------------------------------------------------------------------------
 * Closed-form fp64 quaternion convolution: every multiply-accumulate is a textbook Hamilton
 * product (a1 + b1 i + c1 j + d1 k)(a2 + b2 i + c2 j + d2 k), input sample on the left, filter
 * sample on the right.  Independent in form from the sign-table unrolling above; the backward
 * passes use g * conj(w) and conj(x) * g, the formulas of the reference's pointwise kernels
 * (src/backend/cudnn/quat_pointwise_conv2d.cu:280-283, 403-406).
 * ---------------------------------------------------------------------------------------------- */

static inline void hamilton_acc(double* acc, const double* p, const double* q) {
    acc[0] += p[0] * q[0] - p[1] * q[1] - p[2] * q[2] - p[3] * q[3];
    acc[1] += p[0] * q[1] + p[1] * q[0] + p[2] * q[3] - p[3] * q[2];
    acc[2] += p[0] * q[2] - p[1] * q[3] + p[2] * q[0] + p[3] * q[1];
    acc[3] += p[0] * q[3] + p[1] * q[2] - p[2] * q[1] + p[3] * q[0];
}

void qo_qconv2d_fwd_hamilton(const qo_geom* g, const double* x, const double* w, const double* bias, double* y) {
    const int ho = qo_out_h(g), wo = qo_out_w(g);
    const size_t xs = qo_in_numel(g), ws = qo_w_numel(g), ys = qo_out_numel(g);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < g->n; ++n)
        for (int o = 0; o < g->co; ++o)
            for (int oy = 0; oy < ho; ++oy)
                for (int ox = 0; ox < wo; ++ox) {
                    double acc[4] = {0, 0, 0, 0};
                    if (bias)
                        for (int p = 0; p < 4; ++p) acc[p] = bias[p * g->co + o];
                    for (int c = 0; c < g->ci; ++c)
                        for (int ky = 0; ky < g->kh; ++ky) {
                            const int iy = oy * g->sh - g->pt + ky * g->dh;
                            if (iy < 0 || iy >= g->h) continue;
                            for (int kx = 0; kx < g->kw; ++kx) {
                                const int ix = ox * g->sw - g->pl + kx * g->dw;
                                if (ix < 0 || ix >= g->w) continue;
                                const size_t xi = (((size_t)n * g->ci + c) * g->h + iy) * g->w + ix;
                                const size_t wi = (((size_t)o * g->ci + c) * g->kh + ky) * g->kw + kx;
                                const double xq[4] = {x[xi], x[xs + xi], x[2 * xs + xi], x[3 * xs + xi]};
                                const double wq[4] = {w[wi], w[ws + wi], w[2 * ws + wi], w[3 * ws + wi]};
                                hamilton_acc(acc, xq, wq);
                            }
                        }
                    const size_t yi = (((size_t)n * g->co + o) * ho + oy) * wo + ox;
                    for (int p = 0; p < 4; ++p) y[p * ys + yi] = acc[p];
                }
}

void qo_qconv2d_bwd_data_hamilton(const qo_geom* g, const double* w, const double* grad, double* dx) {
    const int ho = qo_out_h(g), wo = qo_out_w(g);
    const size_t xs = qo_in_numel(g), ws = qo_w_numel(g), ys = qo_out_numel(g);
    memset(dx, 0, 4 * xs * sizeof(double));
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < g->n; ++n)
        for (int c = 0; c < g->ci; ++c)
            for (int o = 0; o < g->co; ++o)
                for (int oy = 0; oy < ho; ++oy)
                    for (int ox = 0; ox < wo; ++ox) {
                        const size_t yi = (((size_t)n * g->co + o) * ho + oy) * wo + ox;
                        const double gq[4] = {grad[yi], grad[ys + yi], grad[2 * ys + yi], grad[3 * ys + yi]};
                        for (int ky = 0; ky < g->kh; ++ky) {
                            const int iy = oy * g->sh - g->pt + ky * g->dh;
                            if (iy < 0 || iy >= g->h) continue;
                            for (int kx = 0; kx < g->kw; ++kx) {
                                const int ix = ox * g->sw - g->pl + kx * g->dw;
                                if (ix < 0 || ix >= g->w) continue;
                                const size_t xi = (((size_t)n * g->ci + c) * g->h + iy) * g->w + ix;
                                const size_t wi = (((size_t)o * g->ci + c) * g->kh + ky) * g->kw + kx;
                                const double wc[4] = {w[wi], -w[ws + wi], -w[2 * ws + wi], -w[3 * ws + wi]};
                                double acc[4] = {0, 0, 0, 0};
                                hamilton_acc(acc, gq, wc);
                                for (int p = 0; p < 4; ++p) dx[p * xs + xi] += acc[p];
                            }
                        }
                    }
}

void qo_qconv2d_bwd_weights_hamilton(const qo_geom* g, const double* x, const double* grad, double* dw) {
    const int ho = qo_out_h(g), wo = qo_out_w(g);
    const size_t xs = qo_in_numel(g), ws = qo_w_numel(g), ys = qo_out_numel(g);
#pragma omp parallel for collapse(2) schedule(static)
    for (int o = 0; o < g->co; ++o)
        for (int c = 0; c < g->ci; ++c)
            for (int ky = 0; ky < g->kh; ++ky)
                for (int kx = 0; kx < g->kw; ++kx) {
                    double acc[4] = {0, 0, 0, 0};
                    for (int n = 0; n < g->n; ++n)
                        for (int oy = 0; oy < ho; ++oy) {
                            const int iy = oy * g->sh - g->pt + ky * g->dh;
                            if (iy < 0 || iy >= g->h) continue;
                            for (int ox = 0; ox < wo; ++ox) {
                                const int ix = ox * g->sw - g->pl + kx * g->dw;
                                if (ix < 0 || ix >= g->w) continue;
                                const size_t xi = (((size_t)n * g->ci + c) * g->h + iy) * g->w + ix;
                                const size_t yi = (((size_t)n * g->co + o) * ho + oy) * wo + ox;
                                const double xc[4] = {x[xi], -x[xs + xi], -x[2 * xs + xi], -x[3 * xs + xi]};
                                const double gq[4] = {grad[yi], grad[ys + yi], grad[2 * ys + yi], grad[3 * ys + yi]};
                                hamilton_acc(acc, xc, gq);
                            }
                        }
                    const size_t wi = (((size_t)o * g->ci + c) * g->kh + ky) * g->kw + kx;
                    for (int p = 0; p < 4; ++p) dw[p * ws + wi] = acc[p];
                }
}

/* ------------------------------------------------------------------------------------------------
 * Type-generic part, once in float (what the reference CPU backend computes in,
 * src/backend/onednn/context.hpp:16-20) and once in double (the exact yardstick).
 * ---------------------------------------------------------------------------------------------- */

#define T float
#define FN(name) name##_f32
#include "qoracle_impl.inc"
#undef T
#undef FN

#define T double
#define FN(name) name##_f64
#include "qoracle_impl.inc"
#undef T
#undef FN
