/*
 * zg_oracle.c -- TEST INFRASTRUCTURE ONLY (see zg_oracle.h).
 *
 * CPU restatement of the reference's HostDevice ops.  Citations are to files
 * under the reference checkout (src/...).  Built with -ffp-contract=off so
 * that `a*b + c` rounds twice, as separate fp32 operations.
 */
#define _GNU_SOURCE
#include "zg_oracle.h"

#include <dlfcn.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------
 * BLAS: the reference links the system `blas` or `mkl_rt` (build.zig:45) and calls nine cblas
 * routines (src/device/host_device.zig:224-337,573-580).  No cblas.h ships here, so the prototypes
 * are declared by hand and resolved with dlopen at first use.  When no library is found, plain
 * loops with the textbook definitions are used.
 * ---------------------------------------------------------------------------------------------- */
enum { ZO_ROW_MAJOR = 101, ZO_NO_TRANS = 111, ZO_TRANS = 112 };

typedef void (*sgemm_fn)(int, int, int, int, int, int, float, const float *, int, const float *, int, float, float *,
                         int);
typedef void (*sgemv_fn)(int, int, int, int, float, const float *, int, const float *, int, float, float *, int);
typedef void (*sger_fn)(int, int, int, float, const float *, int, const float *, int, float *, int);
typedef float (*sdot_fn)(int, const float *, int, const float *, int);
typedef void (*saxpy_fn)(int, float, const float *, int, float *, int);
typedef float (*sasum_fn)(int, const float *, int);
typedef void (*sscal_fn)(int, float, float *, int);
typedef float (*snrm2_fn)(int, const float *, int);
typedef size_t (*isamax_fn)(int, const float *, int);
typedef void (*set_threads_fn)(int);

static struct {
    int probed;
    int force_builtin;
    const char *name;
    void *handle;
    sgemm_fn sgemm;
    sgemv_fn sgemv;
    sger_fn sger;
    sdot_fn sdot;
    saxpy_fn saxpy;
    sasum_fn sasum;
    sscal_fn sscal;
    snrm2_fn snrm2;
    isamax_fn isamax;
    set_threads_fn set_threads;
    int threads;
} g_blas = {0, 0, "builtin", 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1};

static void blas_probe(void) {
    if (g_blas.probed) return;
    g_blas.probed = 1;
    static const char *const cands[][2] = {
        {"libmkl_rt.so", "mkl_rt"},       {"/opt/conda/lib/libmkl_rt.so", "mkl_rt"}, {"libmkl_rt.so.2", "mkl_rt"},
        {"libmkl_rt.so.1", "mkl_rt"},     {"libopenblas.so", "openblas"},            {"libopenblas.so.0", "openblas"},
        {"libblas.so", "blas"},           {"libblas.so.3", "blas"},
    };
    for (size_t i = 0; i < sizeof(cands) / sizeof(cands[0]); i++) {
        void *h = dlopen(cands[i][0], RTLD_NOW | RTLD_LOCAL);
        if (!h) continue;
        sgemm_fn f = (sgemm_fn)dlsym(h, "cblas_sgemm");
        if (!f) {
            dlclose(h);
            continue;
        }
        g_blas.handle = h;
        g_blas.name = cands[i][1];
        g_blas.sgemm = f;
        g_blas.sgemv = (sgemv_fn)dlsym(h, "cblas_sgemv");
        g_blas.sger = (sger_fn)dlsym(h, "cblas_sger");
        g_blas.sdot = (sdot_fn)dlsym(h, "cblas_sdot");
        g_blas.saxpy = (saxpy_fn)dlsym(h, "cblas_saxpy");
        g_blas.sasum = (sasum_fn)dlsym(h, "cblas_sasum");
        g_blas.sscal = (sscal_fn)dlsym(h, "cblas_sscal");
        g_blas.snrm2 = (snrm2_fn)dlsym(h, "cblas_snrm2");
        g_blas.isamax = (isamax_fn)dlsym(h, "cblas_isamax");
        g_blas.set_threads = (set_threads_fn)dlsym(h, "MKL_Set_Num_Threads");
        if (!g_blas.set_threads) g_blas.set_threads = (set_threads_fn)dlsym(h, "openblas_set_num_threads");
        return;
    }
}

static int use_blas(void) {
    blas_probe();
    return g_blas.handle != 0 && !g_blas.force_builtin;
}

const char *zo_blas_name(void) {
    return use_blas() ? g_blas.name : "builtin";
}

int zo_blas_set_threads(int n) {
    blas_probe();
    if (n < 1) n = 1;
    if (g_blas.handle && g_blas.set_threads) {
        g_blas.set_threads(n);
        g_blas.threads = n;
    } else {
        g_blas.threads = 1;
    }
    return g_blas.threads;
}

void zo_blas_force_builtin(int on) {
    g_blas.force_builtin = on;
}

/* ------------------------------------------------------------------------------------------------
 * elementwise binary: src/device/host_device.zig:205-219 (entry points), :975-1019 (elwise_binop)
 * Three regimes: a length-1 operand, equal lengths, and the chunked walk in which z advances by
 * min(x.len, y.len) and an operand whose length differs from z.len restarts at every chunk.
 * ---------------------------------------------------------------------------------------------- */
#define ZO_BINOP(NAME, EXPR)                                                                                       \
    void NAME(const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl) {                         \
        if (xl == 1 || yl == 1) {                                                                                  \
            if (zl == 1) {                                                                                         \
                float a = x[0], b = y[0];                                                                          \
                z[0] = EXPR;                                                                                       \
            } else if (xl == 1) {                                                                                  \
                float a = x[0];                                                                                    \
                for (size_t j = 0; j < zl; j++) {                                                                  \
                    float b = y[j];                                                                                \
                    z[j] = EXPR;                                                                                   \
                }                                                                                                  \
            } else {                                                                                               \
                float b = y[0];                                                                                    \
                for (size_t j = 0; j < zl; j++) {                                                                  \
                    float a = x[j];                                                                                \
                    z[j] = EXPR;                                                                                   \
                }                                                                                                  \
            }                                                                                                      \
            return;                                                                                                \
        }                                                                                                          \
        if (xl == yl) {                                                                                            \
            for (size_t j = 0; j < zl; j++) {                                                                      \
                float a = x[j], b = y[j];                                                                          \
                z[j] = EXPR;                                                                                       \
            }                                                                                                      \
            return;                                                                                                \
        }                                                                                                          \
        size_t mn = xl < yl ? xl : yl;                                                                             \
        size_t xs = (xl == zl) ? mn : 0, ys = (yl == zl) ? mn : 0;                                                 \
        size_t xo = 0, yo = 0, zo = 0;                                                                             \
        while (zo < zl) {                                                                                          \
            for (size_t j = 0; j < mn; j++) {                                                                      \
                float a = x[xo + j], b = y[yo + j];                                                                \
                z[zo + j] = EXPR;                                                                                  \
            }                                                                                                      \
            xo += xs;                                                                                              \
            yo += ys;                                                                                              \
            zo += mn;                                                                                              \
        }                                                                                                          \
    }

ZO_BINOP(zo_add, a + b)
ZO_BINOP(zo_sub, a - b)
ZO_BINOP(zo_mul, a *b)
ZO_BINOP(zo_div, a / b)

/* ------------------------------------------------------------------------------------------------
 * linear algebra
 * ---------------------------------------------------------------------------------------------- */

/* src/device/host_device.zig:224-230 (cblas_sdot) */
void zo_dot(const float *x, const float *y, size_t n, float *z) {
    if (use_blas() && g_blas.sdot) {
        z[0] = g_blas.sdot((int)n, x, 1, y, 1);
        return;
    }
    float s = 0.f;
    for (size_t i = 0; i < n; i++) s += x[i] * y[i];
    z[0] = s;
}

/* src/device/host_device.zig:232-240 (cblas_sgemv, row-major, lda = n; m,n are the stored dims of A) */
void zo_matvec(const float *A, const float *x, float *y, size_t m, size_t n, int trans_a, float alpha, float beta) {
    if (use_blas() && g_blas.sgemv) {
        g_blas.sgemv(ZO_ROW_MAJOR, trans_a ? ZO_TRANS : ZO_NO_TRANS, (int)m, (int)n, alpha, A, (int)n, x, 1, beta, y,
                     1);
        return;
    }
    if (!trans_a) {
        for (size_t i = 0; i < m; i++) {
            float s = 0.f;
            for (size_t j = 0; j < n; j++) s += A[i * n + j] * x[j];
            y[i] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[i];
        }
    } else {
        for (size_t j = 0; j < n; j++) {
            float s = 0.f;
            for (size_t i = 0; i < m; i++) s += A[i * n + j] * x[i];
            y[j] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[j];
        }
    }
}

static void matmul_builtin(const float *A, const float *B, float *C, size_t m, size_t n, size_t k, int ta, int tb,
                           size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    for (size_t i = 0; i < m; i++) {
        for (size_t j = 0; j < n; j++) {
            float s = 0.f;
            for (size_t p = 0; p < k; p++) {
                float a = ta ? A[p * lda + i] : A[i * lda + p];
                float b = tb ? B[j * ldb + p] : B[p * ldb + j];
                s += a * b;
            }
            /* BLAS semantics: C is not read when beta == 0 */
            C[i * ldc + j] = (beta == 0.f) ? alpha * s : alpha * s + beta * C[i * ldc + j];
        }
    }
}

/* src/device/host_device.zig:242-250 (cblas_sgemm, CblasRowMajor, explicit lda/ldb/ldc) */
void zo_matmul(const float *A, const float *B, float *C, size_t m, size_t n, size_t k, int trans_a, int trans_b,
               size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    if (use_blas()) {
        g_blas.sgemm(ZO_ROW_MAJOR, trans_a ? ZO_TRANS : ZO_NO_TRANS, trans_b ? ZO_TRANS : ZO_NO_TRANS, (int)m, (int)n,
                     (int)k, alpha, A, (int)lda, B, (int)ldb, beta, C, (int)ldc);
        return;
    }
    matmul_builtin(A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta);
}

void zo_matmul_f64acc(const float *A, const float *B, float *C, size_t m, size_t n, size_t k, int ta, int tb,
                      size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    for (size_t i = 0; i < m; i++) {
        for (size_t j = 0; j < n; j++) {
            double s = 0.0;
            for (size_t p = 0; p < k; p++) {
                double a = ta ? A[p * lda + i] : A[i * lda + p];
                double b = tb ? B[j * ldb + p] : B[p * ldb + j];
                s += a * b;
            }
            double r = (double)alpha * s;
            if (beta != 0.f) r += (double)beta * (double)C[i * ldc + j];
            C[i * ldc + j] = (float)r;
        }
    }
}

/* src/device/host_device.zig:277-313: one matmul per C batch; operand batch index i % n_batches */
void zo_bmm_acc(const float *A, const uint64_t *A_shape, const float *B, const uint64_t *B_shape, float *C,
                const uint64_t *C_shape, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha,
                float beta) {
    size_t nba = A_shape[0], nbb = B_shape[0], nbc = C_shape[0];
    size_t a_chunk = A_shape[1] * A_shape[2], b_chunk = B_shape[1] * B_shape[2], c_chunk = C_shape[1] * C_shape[2];
    for (size_t i = 0; i < nbc; i++) {
        const float *a = A + (i % nba) * a_chunk;
        const float *b = B + (i % nbb) * b_chunk;
        float *c = C + i * c_chunk;
        zo_matmul(a, b, c, C_shape[1], C_shape[2], A_shape[2], trans_a, trans_b, lda, ldb, ldc, alpha, beta);
    }
}

/* src/device/host_device.zig:252-258 (cblas_sger: A += alpha * x * y^T, lda = y.len) */
void zo_outer(const float *x, size_t xl, const float *y, size_t yl, float *A, float alpha) {
    if (use_blas() && g_blas.sger) {
        g_blas.sger(ZO_ROW_MAJOR, (int)xl, (int)yl, alpha, x, 1, y, 1, A, (int)yl);
        return;
    }
    for (size_t i = 0; i < xl; i++) {
        float ax = alpha * x[i];
        for (size_t j = 0; j < yl; j++) A[i * yl + j] += ax * y[j];
    }
}

/* src/device/host_device.zig:261-267: B = A^T + alpha * B (B is read even when alpha == 0) */
void zo_transpose(const float *A, float *B, size_t m, size_t n, float alpha) {
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) B[j * m + i] = A[i * n + j] + alpha * B[j * m + i];
}

/* src/device/host_device.zig:269-275 (cblas_saxpy; alpha passed by pointer) */
void zo_axpy(const float *x, float *y, size_t n, const float *alpha) {
    if (use_blas() && g_blas.saxpy) {
        g_blas.saxpy((int)n, alpha[0], x, 1, y, 1);
        return;
    }
    float a = alpha[0];
    for (size_t i = 0; i < n; i++) y[i] += a * x[i];
}

/* src/device/host_device.zig:315-321: cblas_sasum, i.e. the sum of ABSOLUTE values */
void zo_sum(const float *x, size_t n, float *y) {
    if (use_blas() && g_blas.sasum) {
        y[0] = g_blas.sasum((int)n, x, 1);
        return;
    }
    float s = 0.f;
    for (size_t i = 0; i < n; i++) s += fabsf(x[i]);
    y[0] = s;
}

/* src/device/host_device.zig:323-329 (cblas_sscal) */
void zo_scale(float *x, size_t n, float alpha) {
    if (use_blas() && g_blas.sscal) {
        g_blas.sscal((int)n, alpha, x, 1);
        return;
    }
    for (size_t i = 0; i < n; i++) x[i] *= alpha;
}

/* src/device/host_device.zig:331-337 (cblas_snrm2) */
void zo_nrm2(const float *x, size_t n, float *y) {
    if (use_blas() && g_blas.snrm2) {
        y[0] = g_blas.snrm2((int)n, x, 1);
        return;
    }
    double s = 0.0;
    for (size_t i = 0; i < n; i++) s += (double)x[i] * (double)x[i];
    y[0] = (float)sqrt(s);
}

/* src/device/host_device.zig:339-346 */
void zo_clip_nrm2(float *x, size_t n, float max_norm, float delta) {
    float norm;
    zo_nrm2(x, n, &norm);
    if (norm > max_norm) zo_scale(x, n, max_norm / (norm + delta));
}

/* ------------------------------------------------------------------------------------------------
 * unary forward/backward
 * ---------------------------------------------------------------------------------------------- */

/* src/device/host_device.zig:353-358 */
void zo_pow_fwd(const float *x, float *y, size_t n, float e) {
    for (size_t i = 0; i < n; i++) y[i] = powf(x[i], e);
}

/* src/device/host_device.zig:367-379 */
void zo_pow_bwd(const float *x, float *x_g, const float *y_g, size_t n, float e, float eps) {
    float em1 = e - 1.f;
    for (size_t i = 0; i < n; i++) {
        if (x[i] < eps)
            x_g[i] += 0.0f;
        else
            x_g[i] += e * powf(x[i], em1) * y_g[i];
    }
}

/* src/device/host_device.zig:382-386 */
void zo_sqrt_fwd(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = sqrtf(x[i]);
}

/* src/device/host_device.zig:395-407 */
void zo_sqrt_bwd(const float *x, float *x_g, const float *y_g, size_t n, float eps) {
    for (size_t i = 0; i < n; i++) {
        if (x[i] < eps)
            x_g[i] += 0.0f;
        else
            x_g[i] += 0.5f / sqrtf(x[i]) * y_g[i];
    }
}

/* src/device/host_device.zig:475-482 (native path: 1/sqrt(max(x, eps))) */
void zo_rsqrt_fwd(const float *x, float *y, size_t n, float eps) {
    for (size_t i = 0; i < n; i++) y[i] = 1.f / sqrtf(fmaxf(x[i], eps));
}

/* src/device/host_device.zig:486-503 */
void zo_rsqrt_bwd(const float *x, float *x_g, const float *y_g, size_t n, float eps) {
    for (size_t i = 0; i < n; i++) {
        if (x[i] < eps) {
            x_g[i] += 0.0f;
        } else {
            float s = sqrtf(x[i]);
            float inv = 1.0f / (x[i] * s);
            x_g[i] += (-0.5f * inv) * y_g[i];
        }
    }
}

/* src/device/host_device.zig:505-517 */
void zo_exp_fwd(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = expf(x[i]);
}

/* src/device/host_device.zig:519-522 */
void zo_exp_bwd(float *x_g, const float *y, const float *y_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] += y[i] * y_g[i];
}

/* src/device/host_device.zig:524-537 */
void zo_relu_fwd(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = x[i] > 0.f ? x[i] : 0.f;
}

/* src/device/host_device.zig:539-541 */
void zo_relu_bwd(const float *x, float *x_g, const float *y_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] += (x[i] > 0.f) ? y_g[i] : 0.f;
}

/* src/device/host_device.zig:543-547 */
void zo_relu_inplace_bwd(const float *x, float *x_g, size_t n) {
    for (size_t i = 0; i < n; i++)
        if (x[i] <= 0.f) x_g[i] = 0.f;
}

/* src/device/host_device.zig:549-551 */
void zo_tanh_fwd(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = tanhf(x[i]);
}

/* src/device/host_device.zig:553-555 */
void zo_tanh_bwd(float *x_g, const float *y, const float *y_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] += (1.f - (y[i] * y[i])) * y_g[i];
}

/* src/device/host_device.zig:557-559 */
void zo_tanh_inplace_bwd(const float *x, float *x_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] *= (1.f - (x[i] * x[i]));
}

/* src/device/host_device.zig:561-563 */
void zo_sigm_fwd(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = 1.f / (1.f + expf(-x[i]));
}

/* src/device/host_device.zig:565-567 */
void zo_sigm_bwd(float *x_g, const float *y, const float *y_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] += y[i] * (1.f - y[i]) * y_g[i];
}

/* src/device/host_device.zig:569-571 */
void zo_sigm_inplace_bwd(const float *x, float *x_g, size_t n) {
    for (size_t i = 0; i < n; i++) x_g[i] *= (x[i] * (1.f - x[i]));
}

/* src/device/host_device.zig:590-592 */
void zo_clamp_fwd(const float *x, float *y, size_t n, float lo, float hi) {
    for (size_t i = 0; i < n; i++) y[i] = fminf(hi, fmaxf(lo, x[i]));
}

/* src/device/host_device.zig:594-598 */
void zo_clamp_bwd(const float *x, float *x_g, const float *y_g, size_t n, float lo, float hi) {
    for (size_t i = 0; i < n; i++)
        if (lo < x[i] && x[i] < hi) x_g[i] += y_g[i];
}

/* src/device/host_device.zig:573-580: x[cblas_isamax(x)], the element of largest ABSOLUTE value
 * (first such index on ties, the BLAS definition of i?amax). */
void zo_max_fwd(const float *x, size_t n, float *y) {
    size_t idx = 0;
    if (use_blas() && g_blas.isamax) {
        idx = g_blas.isamax((int)n, x, 1);
    } else {
        /* a NaN counts as larger than anything, the first one wins: what mkl_rt documents for i?amax (the plain
         * comparison loop of the Fortran routine would skip NaNs unless one comes first) */
        float best = -1.f;
        for (size_t i = 0; i < n; i++) {
            float a = fabsf(x[i]);
            if (a != a) {
                idx = i;
                break;
            }
            if (a > best) {
                best = a;
                idx = i;
            }
        }
    }
    y[0] = x[idx];
}

/* src/device/host_device.zig:582-588 */
void zo_max_bwd(const float *x, float *x_g, size_t n, const float *y, const float *y_g) {
    float val = y[0], grd = y_g[0];
    for (size_t i = 0; i < n; i++)
        if (val == x[i]) x_g[i] += grd;
}

/* ------------------------------------------------------------------------------------------------
 * reductions: src/device/reduce.zig.  The reference accumulates in SIMD lanes of
 * std.simd.suggestVectorLength(f32); eight lanes (AVX2) are restated here.  The lane count changes
 * only the fp32 summation order.
 * ---------------------------------------------------------------------------------------------- */
#define ZO_LANES 8

static float lanes_reduce(const float *u) {
    /* pairwise tree, the shape of a horizontal vector add */
    float t[ZO_LANES];
    memcpy(t, u, sizeof(t));
    for (int w = ZO_LANES / 2; w >= 1; w /= 2)
        for (int i = 0; i < w; i++) t[i] = t[i] + t[i + w];
    return t[0];
}

/* src/device/reduce.zig:3-11 */
static void scaled_copy(const float *x, float *y, size_t n, float alpha, float beta) {
    for (size_t i = 0; i < n; i++) y[i] = alpha * x[i] + beta * y[i];
}

/* src/device/reduce.zig:13-46 */
static void flat_reduce(const float *x, size_t n, float *y, float alpha, float beta) {
    float u[ZO_LANES] = {0};
    size_t i = 0;
    for (; i + ZO_LANES <= n; i += ZO_LANES)
        for (int l = 0; l < ZO_LANES; l++) u[l] += x[i + l];
    float s = lanes_reduce(u);
    for (; i < n; i++) s += x[i];
    y[0] = alpha * s + beta * y[0];
}

/* src/device/reduce.zig:49-128: (row, col) -> (col); every column is summed over rows in row order */
static void fold_rows(const float *x, float *y, size_t row, size_t col, float alpha, float beta) {
    for (size_t j = 0; j < col; j++) {
        float s = x[j];
        for (size_t i = 1; i < row; i++) s += x[i * col + j];
        y[j] = alpha * s + beta * y[j];
    }
}

/* src/device/reduce.zig:131-164: (row, col) -> (row) */
static void fold_cols(const float *x, float *y, size_t row, size_t col, float alpha, float beta) {
    for (size_t i = 0; i < row; i++) {
        const float *xr = x + i * col;
        float u[ZO_LANES] = {0};
        size_t j = 0;
        for (; j + ZO_LANES <= col; j += ZO_LANES)
            for (int l = 0; l < ZO_LANES; l++) u[l] += xr[j + l];
        float s = 0.f;
        s += lanes_reduce(u);
        for (; j < col; j++) s += xr[j];
        y[i] = alpha * s + beta * y[i];
    }
}

static size_t prod(const uint64_t *s, size_t from, size_t to) {
    size_t n = 1;
    for (size_t i = from; i < to; i++) n *= (size_t)s[i];
    return n;
}

/* src/device/host_device.zig:798-847 */
void zo_sum_along(const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len, size_t dim,
                  float alpha, float beta) {
    size_t x_len = prod(x_shape, 0, x_rank);
    if (y_len == 1) {
        flat_reduce(x, x_len, y, alpha, beta);
        return;
    } else if (dim == 0) {
        fold_rows(x, y, x_shape[0], prod(x_shape, 1, x_rank), alpha, beta);
        return;
    } else if (dim + 1 == x_rank) {
        fold_cols(x, y, prod(x_shape, 0, dim), x_shape[dim], alpha, beta);
        return;
    }
    size_t n_chunks = prod(x_shape, 0, dim);
    size_t y_chunk = prod(x_shape, dim + 1, x_rank);
    size_t x_chunk = x_shape[dim] * y_chunk;
    for (size_t n = 0; n < n_chunks; n++) fold_rows(x + x_chunk * n, y + y_chunk * n, x_shape[dim], y_chunk, alpha, beta);
}

/* src/device/host_device.zig:852-874: strict '>' running max from -inf; alpha/beta are ignored */
void zo_max_along(const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len, size_t dim) {
    size_t max_dim = x_shape[dim];
    size_t slice = prod(x_shape, dim + 1, x_rank);
    for (size_t i = 0; i < y_len; i++) {
        float mv = -INFINITY;
        size_t base = (i / slice) * (slice * max_dim) + (i % slice);
        for (size_t j = 0; j < max_dim; j++) {
            float c = x[base + j * slice];
            if (c > mv) mv = c;
        }
        y[i] = mv;
    }
}

/* No reference device op.  The examples call std.mem.indexOfMax on a host row
 * (examples/mnist/src/main-simple.zig:124-125): the FIRST index holding the maximum.
 * Here applied to every slice along `dim`, with the slice addressing of max_along. */
void zo_argmax_along(const float *x, const uint64_t *x_shape, size_t x_rank, uint64_t *y, size_t y_len, size_t dim) {
    size_t max_dim = x_shape[dim];
    size_t slice = prod(x_shape, dim + 1, x_rank);
    for (size_t i = 0; i < y_len; i++) {
        size_t base = (i / slice) * (slice * max_dim) + (i % slice);
        float mv = x[base];
        uint64_t mi = 0;
        for (size_t j = 1; j < max_dim; j++) {
            float c = x[base + j * slice];
            if (c > mv) {
                mv = c;
                mi = j;
            }
        }
        y[i] = mi;
    }
}

/* src/ndarray.zig:701-719: scratch length requested before dispatching unbroadcast */
size_t zo_unbroadcast_scratch_len(const uint64_t *x_shape, size_t x_rank, const uint64_t *y_shape, size_t y_rank) {
    size_t x_size = prod(x_shape, 0, x_rank), y_size = prod(y_shape, 0, y_rank);
    size_t delta = x_rank - y_rank;
    size_t coef;
    if (delta > 0) {
        /* as written in the reference: the product of the first `delta` dims of x */
        coef = prod(x_shape, 0, delta);
    } else {
        size_t mm = x_rank;
        for (size_t i = 0; i < x_rank; i++)
            if (x_shape[i] != y_shape[i]) {
                mm = i;
                break;
            }
        if (mm == x_rank) return 0;
        coef = x_shape[mm];
    }
    size_t n = y_size * coef;
    return n == x_size ? 0 : n;
}

/* src/device/host_device.zig:709-780 */
void zo_unbroadcast(const float *x, const uint64_t *x_shape_in, size_t x_rank_in, float *y,
                    const uint64_t *y_shape_in, size_t y_rank_in, float *scratch, size_t scratch_len, float alpha,
                    float beta) {
    size_t x_len = prod(x_shape_in, 0, x_rank_in), y_len = prod(y_shape_in, 0, y_rank_in);
    if (x_len == y_len) {
        scaled_copy(x, y, x_len, alpha, beta);
        return;
    }
    uint64_t xs[8], ys[8];
    size_t xr = 0, yr = 0;
    { /* trim leading ones of x; trim leading and trailing ones of y */
        size_t s = 0;
        while (s < x_rank_in && x_shape_in[s] == 1) s++;
        for (size_t i = s; i < x_rank_in; i++) xs[xr++] = x_shape_in[i];
        size_t b = 0, e = y_rank_in;
        while (b < e && y_shape_in[b] == 1) b++;
        while (e > b && y_shape_in[e - 1] == 1) e--;
        for (size_t i = b; i < e; i++) ys[yr++] = y_shape_in[i];
    }
    size_t ones = 0;
    for (size_t i = 0; i < yr; i++) ones += (ys[i] == 1);

    if (xr > yr) {
        size_t dif = xr - yr;
        fold_rows(x, ones == 0 ? y : scratch, prod(xs, 0, dif), prod(xs, dif, xr), alpha, beta);
        if (ones == 0) return;
        for (size_t i = dif; i < xr; i++) xs[i - dif] = xs[i];
        xr -= dif;
    }
    size_t i = 0;
    while (ones > 0 && i < xr) {
        if (ys[i] == 1 && xs[i] != 1) {
            /* the reference compares the working rank with the caller's rank to decide whether a
             * previous stage already moved the data into scratch */
            const float *xd = (xr == x_rank_in) ? x : scratch;
            float *yd = (ones == 1) ? y : scratch;
            /* sum_along's flat-reduce test looks at the length of the slice it was handed */
            size_t yl = (ones == 1) ? y_len : scratch_len;
            zo_sum_along(xd, xs, xr, yd, yl, i, alpha, beta);
            for (size_t j = i + 1; j < xr; j++) xs[j - 1] = xs[j];
            for (size_t j = i + 1; j < yr; j++) ys[j - 1] = ys[j];
            xr--;
            yr--;
            ones--;
            continue;
        }
        i++;
    }
}

/* src/device/host_device.zig:782-795.  The equal-length branch lacks a `return`, so alpha/beta are
 * applied by scaled_copy and then again by the modulo loop; restated as written. */
void zo_broadcast(const float *x, size_t xl, float *y, size_t yl, float alpha, float beta) {
    if (xl == yl) scaled_copy(x, y, xl, alpha, beta);
    for (size_t i = 0; i < yl; i++) y[i] = alpha * x[i % xl] + beta * y[i % yl];
}

/* ------------------------------------------------------------------------------------------------
 * memory-style ops
 * ---------------------------------------------------------------------------------------------- */

/* src/device/host_device.zig:927-929 */
void zo_mem_fill(float *x, size_t n, float v) {
    for (size_t i = 0; i < n; i++) x[i] = v;
}

/* src/device/host_device.zig:948-954: a running `current += step` */
void zo_mem_sequence(float *x, size_t n, float initial, float step) {
    float cur = initial;
    for (size_t i = 0; i < n; i++) {
        x[i] = cur;
        cur += step;
    }
}

/* src/device/host_device.zig:955-958 */
void zo_mem_take(const float *src, size_t src_len, const uint64_t *idxs, size_t n, float *dst) {
    (void)src_len;
    for (size_t j = 0; j < n; j++) dst[j] = src[idxs[j]];
}

/* src/device/host_device.zig:931-945 defines WHAT is drawn (U[0,1), N(0,1), N(0,1)*sqrt(2/fan));
 * the stream comes from a host std.Random the caller passes, whose Ziggurat normals are not
 * reproducible here, so the stream is this documented one: splitmix64-seeded xoshiro256++,
 * uniform = top 24 bits * 2^-24, normal = Box-Muller on two uniforms (cosine branch) in fp32.
 * Pinned by the generators' published known-answer vectors through an independent restatement. */
static uint64_t rotl64(uint64_t x, int k) {
    return (x << k) | (x >> (64 - k));
}
typedef struct {
    uint64_t s[4];
} zo_rng;
static void rng_seed(zo_rng *r, uint64_t seed) {
    uint64_t z = seed;
    for (int i = 0; i < 4; i++) {
        z += 0x9e3779b97f4a7c15ULL;
        uint64_t v = z;
        v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ULL;
        v = (v ^ (v >> 27)) * 0x94d049bb133111ebULL;
        r->s[i] = v ^ (v >> 31);
    }
}
static uint64_t rng_next(zo_rng *r) {
    uint64_t *s = r->s;
    uint64_t result = rotl64(s[0] + s[3], 23) + s[0];
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}
static float rng_uniform(zo_rng *r) {
    return (float)(rng_next(r) >> 40) * (1.0f / 16777216.0f);
}
static float rng_normal(zo_rng *r) {
    float u1 = 1.0f - rng_uniform(r); /* (0,1] */
    float u2 = rng_uniform(r);
    return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
}
void zo_mem_random(float *x, size_t n, int kind, uint64_t fan, uint64_t seed) {
    zo_rng r;
    rng_seed(&r, seed);
    if (kind == 0) {
        for (size_t i = 0; i < n; i++) x[i] = rng_uniform(&r);
    } else if (kind == 1) {
        for (size_t i = 0; i < n; i++) x[i] = rng_normal(&r);
    } else {
        float sd = sqrtf(2.0f / (float)fan);
        for (size_t i = 0; i < n; i++) x[i] = rng_normal(&r) * sd;
    }
}

/* ------------------------------------------------------------------------------------------------
 * indexing
 * ---------------------------------------------------------------------------------------------- */

/* src/ndarray.zig:593-633 with src/ndarray/shape.zig strides (row-major, last stride 1):
 * offsets[i] = offset of (coord(i) with coord[dim] := indices[i]) in the source. */
int zo_gather_offsets(const uint64_t *src_shape, const uint64_t *idx_shape, size_t rank, const uint64_t *indices,
                      size_t dim, uint64_t *offsets) {
    for (size_t i = 0; i < rank; i++)
        if (i != dim && idx_shape[i] > src_shape[i]) return 1;
    uint64_t istr[8], sstr[8];
    uint64_t a = 1, b = 1;
    for (size_t i = rank; i-- > 0;) {
        istr[i] = a;
        a *= idx_shape[i];
        sstr[i] = b;
        b *= src_shape[i];
    }
    size_t n = (size_t)a;
    for (size_t i = 0; i < n; i++) {
        uint64_t rem = i, off = 0;
        for (size_t d = 0; d < rank; d++) {
            uint64_t c = rem / istr[d];
            rem = rem % istr[d];
            if (d == dim) {
                c = indices[i];
                if (c >= src_shape[dim]) return 2;
            }
            off += c * sstr[d];
        }
        offsets[i] = off;
    }
    return 0;
}

/* src/device/host_device.zig:1039-1087: dst[offsets[i]] += src[i], in index order */
/* src/device/host_device.zig:1325-1335 */
void zo_scatter_add_csr(const float *src, const uint64_t *row_ptr, size_t n_segments, float *dst, size_t dst_len) {
    for (size_t i = 0; i < n_segments; i++) {
        const float value = src[i];
        for (uint64_t j = row_ptr[i]; j < row_ptr[i + 1] && j < dst_len; j++) dst[j] += value;
    }
}

/* src/device/host_device.zig:1337-1353; the host sums each segment in SIMD lanes (vsum_contig), here sequentially:
 * the order is not pinned by the reference */
void zo_segment_sum_csr(const float *src, size_t src_len, const uint64_t *row_offsets, size_t n_segments, float *dst) {
    for (size_t i = 0; i < n_segments; i++) {
        float s = 0.0f;
        for (uint64_t j = row_offsets[i]; j < row_offsets[i + 1] && j < src_len; j++) s += src[j];
        dst[i] = s;
    }
}

void zo_scatter_add(const float *src, const uint64_t *offsets, size_t n, float *dst, size_t dst_len) {
    (void)dst_len;
    for (size_t i = 0; i < n; i++) dst[offsets[i]] += src[i];
}

/* src/ndtensor.zig:1481-1496: one copy of `stride` contiguous elements per selected index */
void zo_index_select_fwd(const float *src, size_t src_len, const uint64_t *indices, size_t n_idx, size_t stride,
                         float *dst) {
    (void)src_len;
    for (size_t d = 0; d < n_idx; d++) memcpy(dst + d * stride, src + indices[d] * stride, stride * sizeof(float));
}

/* src/ndtensor.zig:1453-1466: one add per selected index, in index order */
void zo_index_select_bwd(const float *y_grad, const uint64_t *indices, size_t n_idx, size_t stride, float *x_grad,
                         size_t x_len) {
    (void)x_len;
    for (size_t d = 0; d < n_idx; d++) {
        float *xg = x_grad + indices[d] * stride;
        const float *yg = y_grad + d * stride;
        for (size_t j = 0; j < stride; j++) xg[j] = yg[j] + xg[j];
    }
}

/* src/device/host_device.zig:1356-1370 */
void zo_scatter_gcn_deg_scaled(float *dst, const float *h, const float *deg, const uint64_t *src_indices,
                               const uint64_t *tgt_indices, size_t stride, size_t n_edge) {
    for (size_t e = 0; e < n_edge; e++) {
        size_t s = src_indices[e], t = tgt_indices[e];
        float w = deg[s] * deg[t];
        for (size_t j = 0; j < stride; j++) dst[t * stride + j] += w * h[s * stride + j];
    }
}

/* src/device/host_device.zig:1372-1403 */
void zo_scatter_gcn_deg_scaled_bwd(const float *grad_output, const float *h, const float *deg,
                                   const uint64_t *src_indices, const uint64_t *tgt_indices, float *grad_h,
                                   float *grad_deg, size_t stride, size_t n_edge) {
    for (size_t e = 0; e < n_edge; e++) {
        size_t s = src_indices[e], t = tgt_indices[e];
        float ds = deg[s], dt = deg[t];
        float gs = 0.f, gt = 0.f;
        for (size_t j = 0; j < stride; j++) {
            float go = grad_output[t * stride + j];
            float hv = h[s * stride + j];
            grad_h[s * stride + j] += go * ds * dt;
            gs += go * dt * hv;
            gt += go * ds * hv;
        }
        grad_deg[s] += gs;
        grad_deg[t] += gt;
    }
}

/* ------------------------------------------------------------------------------------------------
 * losses: src/nn/loss.zig
 * ---------------------------------------------------------------------------------------------- */

/* src/nn/loss.zig:175-215 restricted to the last dim of a rank<=2 tensor (the only case :135 admits) */
void zo_softmax_fwd(const float *x, float *y, size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++) {
        const float *xr = x + r * cols;
        float *yr = y + r * cols;
        float mx = xr[0];
        for (size_t j = 1; j < cols; j++) mx = fmaxf(mx, xr[j]);
        float se = 0.f;
        for (size_t j = 0; j < cols; j++) se += expf(xr[j] - mx);
        float lse = mx + logf(se);
        for (size_t j = 0; j < cols; j++) yr[j] = expf(xr[j] - lse);
    }
}

/* src/nn/loss.zig:223-246 */
void zo_softmax_bwd(const float *y, const float *y_g, float *x_g, size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++) {
        size_t b = r * cols;
        float sg = 0.f;
        for (size_t j = 0; j < cols; j++) sg += y[b + j] * y_g[b + j];
        for (size_t j = 0; j < cols; j++) x_g[b + j] += y[b + j] * (y_g[b + j] - sg);
    }
}

/* src/nn/loss.zig:130-146 */
void zo_smce_fwd(const float *logits, const float *target, float *probs, float *loss, size_t rows, size_t cols) {
    const float eps = 1e-7f;
    zo_softmax_fwd(logits, probs, rows, cols);
    float sum_loss = 0.f;
    for (size_t i = 0; i < rows * cols; i++) {
        float safe = fminf(fmaxf(probs[i], eps), 1.0f - eps);
        sum_loss -= target[i] * logf(safe);
    }
    loss[0] = sum_loss / (float)rows;
}

/* src/nn/loss.zig:150-159 */
void zo_smce_bwd(const float *probs, const float *target, float *grad, size_t rows, size_t cols) {
    float b = (float)rows;
    for (size_t i = 0; i < rows * cols; i++) grad[i] += (probs[i] - target[i]) / b;
}

/* The same computation with the one-hot row given by its index.  With target = e_label every term
 * of the loss sum except j == label is -0 * log(p) = 0, so the loss equals
 * -(1/B) * sum_r log(clamp(p[r, label_r])); the per-row log-sum-exp is what backward needs to
 * rebuild p = exp(x - lse) (src/nn/loss.zig:206-211). */
void zo_smce_label_fwd(const float *logits, const uint64_t *labels, float *lse, float *loss, size_t rows,
                       size_t cols) {
    const float eps = 1e-7f;
    float sum_loss = 0.f;
    for (size_t r = 0; r < rows; r++) {
        const float *xr = logits + r * cols;
        float mx = xr[0];
        for (size_t j = 1; j < cols; j++) mx = fmaxf(mx, xr[j]);
        float se = 0.f;
        for (size_t j = 0; j < cols; j++) se += expf(xr[j] - mx);
        float l = mx + logf(se);
        lse[r] = l;
        float p = expf(xr[labels[r]] - l);
        float safe = fminf(fmaxf(p, eps), 1.0f - eps);
        sum_loss -= logf(safe);
    }
    loss[0] = sum_loss / (float)rows;
}

void zo_smce_label_bwd(const float *logits, const uint64_t *labels, const float *lse, float *grad, size_t rows,
                       size_t cols) {
    float b = (float)rows;
    for (size_t r = 0; r < rows; r++) {
        for (size_t j = 0; j < cols; j++) {
            float p = expf(logits[r * cols + j] - lse[r]);
            float t = (j == labels[r]) ? 1.0f : 0.0f;
            grad[r * cols + j] += (p - t) / b;
        }
    }
}

/* src/nn/loss.zig:259-275 */
void zo_smooth_l1_fwd(const float *pred, const float *target, size_t n, float beta, float *loss) {
    float s = 0.f;
    for (size_t i = 0; i < n; i++) {
        float d = pred[i] - target[i];
        float ad = fabsf(d);
        if (ad < beta)
            s += 0.5f * (d * d) / beta;
        else
            s += ad - (0.5f * beta);
    }
    loss[0] = s / (float)n;
}

/* src/nn/loss.zig:279-294 */
void zo_smooth_l1_bwd(const float *pred, const float *target, float *grad, size_t n, float beta) {
    float nf = (float)n;
    for (size_t i = 0; i < n; i++) {
        float d = pred[i] - target[i];
        if (fabsf(d) < beta) {
            grad[i] += d / (beta * nf);
        } else {
            float sg = (d > 0.f) ? 1.f : ((d < 0.f) ? -1.f : 0.f);
            grad[i] += sg / nf;
        }
    }
}

/* src/nn/loss.zig:94-103 */
void zo_mse_fwd(const float *pred, const float *target, size_t n, float *loss) {
    float s = 0.f;
    for (size_t i = 0; i < n; i++) {
        float d = pred[i] - target[i];
        s += d * d;
    }
    loss[0] = s / (float)n;
}

/* src/nn/loss.zig:106-116 */
void zo_mse_bwd(const float *pred, const float *target, float *grad, size_t n) {
    float sc = 2.0f / (float)n;
    for (size_t i = 0; i < n; i++) grad[i] += sc * (pred[i] - target[i]);
}

/* ------------------------------------------------------------------------------------------------
 * optimizers: src/nn/optim.zig
 * ---------------------------------------------------------------------------------------------- */

/* src/nn/optim.zig:100-122: optional per-tensor clip, then param += (-lr) * grad via axpy */
void zo_sgd_step(float *param, float *grad, size_t n, float lr, int clip, float max_norm, float delta) {
    if (clip) zo_clip_nrm2(grad, n, max_norm, delta);
    float nlr = -lr;
    zo_axpy(grad, param, n, &nlr);
}

/* src/nn/optim.zig:189-191, all in fp32 */
float zo_adam_lr_t(uint64_t t, float lr, float beta1, float beta2) {
    float tf = (float)t;
    return lr * sqrtf(1.0f - powf(beta2, tf)) / (1.0f - powf(beta1, tf));
}

/* src/nn/optim.zig:177-234 */
void zo_adam_step(float *param, float *grad, float *m, float *v, size_t n, uint64_t t, float lr, float beta1,
                  float beta2, float epsilon, int clip, float max_norm, float delta) {
    float lr_t = zo_adam_lr_t(t, lr, beta1, beta2);
    if (clip) zo_clip_nrm2(grad, n, max_norm, delta);
    for (size_t i = 0; i < n; i++) {
        float g = grad[i];
        m[i] = beta1 * m[i] + (1.0f - beta1) * g;
        v[i] = beta2 * v[i] + (1.0f - beta2) * g * g;
        param[i] -= lr_t * m[i] / (sqrtf(v[i]) + epsilon);
    }
}
