/*
 * zg_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU restatement of Zigrad's HostDevice for the device-op hot path.
 * It exists to check the HIP backend and to serve as the reported CPU baseline.
 * Nothing in the shipped library may include, link or call it.
 *
 * Every function follows one reference routine; the citation is on the
 * definition in zg_oracle.c.  Slices of the reference become (pointer, length)
 * pairs, `usize` becomes uint64_t, all arithmetic is fp32 as in the reference.
 *
 * Parity status (what pins each restated routine is listed in tests/):
 *   every routine below is pinned by the reference's own vectors and/or by
 *   closed forms, brute force and published known-answer vectors that share
 *   no code with it; no routine is "parity unpinned".
 *   Two things are outside what can be pinned and are documented instead:
 *   zo_mem_random draws what the reference's mem_random draws (U[0,1), N(0,1),
 *   N(0,1)*sqrt(2/fan)) but from its own documented stream (splitmix64 ->
 *   xoshiro256++ -> 24-bit uniforms -> Box-Muller), because Zig's Ziggurat
 *   normal sampler cannot be reproduced without a Zig toolchain; that stream
 *   is pinned by the generators' published vectors and an independent
 *   restatement.  The exact rounding/summation order of the external BLAS
 *   (sgemm/sasum/snrm2/sdot/sgemv) at large sizes is not pinned by the
 *   reference either; those are held to tolerance against an fp64-accumulated
 *   result.
 */
#ifndef ZG_ORACLE_H
#define ZG_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* BLAS backend discovery. Returns a static string: "mkl_rt", "openblas", "blas" or "builtin". */
const char *zo_blas_name(void);
/* Set the BLAS thread count when the backend supports it; returns the count in effect. */
int zo_blas_set_threads(int n);
/* Force the built-in loops even when a BLAS is present (1) or restore discovery (0). */
void zo_blas_force_builtin(int on);

/* ---- elementwise binary ---- */
void zo_add(const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
void zo_sub(const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
void zo_mul(const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
void zo_div(const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);

/* ---- linear algebra ---- */
void zo_dot(const float *x, const float *y, size_t n, float *z);
void zo_matvec(const float *A, const float *x, float *y, size_t m, size_t n, int trans_a, float alpha, float beta);
void zo_matmul(const float *A, const float *B, float *C, size_t m, size_t n, size_t k, int trans_a, int trans_b,
               size_t lda, size_t ldb, size_t ldc, float alpha, float beta);
/* fp64-accumulated triple loop with the same argument meaning; the tolerance anchor for large GEMMs */
void zo_matmul_f64acc(const float *A, const float *B, float *C, size_t m, size_t n, size_t k, int trans_a, int trans_b,
                      size_t lda, size_t ldb, size_t ldc, float alpha, float beta);
void zo_bmm_acc(const float *A, const uint64_t *A_shape, const float *B, const uint64_t *B_shape, float *C,
                const uint64_t *C_shape, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha,
                float beta);
void zo_outer(const float *x, size_t xl, const float *y, size_t yl, float *A, float alpha);
void zo_transpose(const float *A, float *B, size_t m, size_t n, float alpha);
void zo_axpy(const float *x, float *y, size_t n, const float *alpha);
void zo_sum(const float *x, size_t n, float *y);
void zo_scale(float *x, size_t n, float alpha);
void zo_nrm2(const float *x, size_t n, float *y);
void zo_clip_nrm2(float *x, size_t n, float max_norm, float delta);

/* ---- unary forward / backward ---- */
void zo_pow_fwd(const float *x, float *y, size_t n, float e);
void zo_pow_bwd(const float *x, float *x_g, const float *y_g, size_t n, float e, float eps);
void zo_sqrt_fwd(const float *x, float *y, size_t n);
void zo_sqrt_bwd(const float *x, float *x_g, const float *y_g, size_t n, float eps);
void zo_rsqrt_fwd(const float *x, float *y, size_t n, float eps);
void zo_rsqrt_bwd(const float *x, float *x_g, const float *y_g, size_t n, float eps);
void zo_exp_fwd(const float *x, float *y, size_t n);
void zo_exp_bwd(float *x_g, const float *y, const float *y_g, size_t n);
void zo_relu_fwd(const float *x, float *y, size_t n);
void zo_relu_bwd(const float *x, float *x_g, const float *y_g, size_t n);
void zo_relu_inplace_bwd(const float *x, float *x_g, size_t n);
void zo_tanh_fwd(const float *x, float *y, size_t n);
void zo_tanh_bwd(float *x_g, const float *y, const float *y_g, size_t n);
void zo_tanh_inplace_bwd(const float *x, float *x_g, size_t n);
void zo_sigm_fwd(const float *x, float *y, size_t n);
void zo_sigm_bwd(float *x_g, const float *y, const float *y_g, size_t n);
void zo_sigm_inplace_bwd(const float *x, float *x_g, size_t n);
void zo_clamp_fwd(const float *x, float *y, size_t n, float lo, float hi);
void zo_clamp_bwd(const float *x, float *x_g, const float *y_g, size_t n, float lo, float hi);
void zo_max_fwd(const float *x, size_t n, float *y);
void zo_max_bwd(const float *x, float *x_g, size_t n, const float *y, const float *y_g);

/* ---- reductions ---- */
void zo_sum_along(const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len, size_t dim,
                  float alpha, float beta);
void zo_max_along(const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len, size_t dim);
/* first index of the maximum along `dim` (std.mem.indexOfMax semantics applied per slice) */
void zo_argmax_along(const float *x, const uint64_t *x_shape, size_t x_rank, uint64_t *y, size_t y_len, size_t dim);
/* number of scratch floats NDArray.unbroadcast_ would request for these shapes */
size_t zo_unbroadcast_scratch_len(const uint64_t *x_shape, size_t x_rank, const uint64_t *y_shape, size_t y_rank);
void zo_unbroadcast(const float *x, const uint64_t *x_shape, size_t x_rank, float *y, const uint64_t *y_shape,
                    size_t y_rank, float *scratch, size_t scratch_len, float alpha, float beta);
void zo_broadcast(const float *x, size_t xl, float *y, size_t yl, float alpha, float beta);

/* ---- memory-style ops ---- */
void zo_mem_fill(float *x, size_t n, float v);
void zo_mem_sequence(float *x, size_t n, float initial, float step);
void zo_mem_take(const float *src, size_t src_len, const uint64_t *idxs, size_t n, float *dst);
/* kind: 0 uniform [0,1), 1 normal, 2 kaiming (normal * sqrt(2/fan)).  Own generator (see zg_oracle.c). */
void zo_mem_random(float *x, size_t n, int kind, uint64_t fan, uint64_t seed);

/* ---- indexing ---- */
/* NDArray.gather offset computation; returns 0 on success, 1 InvalidIndexShape, 2 IndexOutOfBounds */
int zo_gather_offsets(const uint64_t *src_shape, const uint64_t *idx_shape, size_t rank, const uint64_t *indices,
                      size_t dim, uint64_t *offsets);
void zo_scatter_add(const float *src, const uint64_t *offsets, size_t n, float *dst, size_t dst_len);
void zo_scatter_add_csr(const float *src, const uint64_t *row_ptr, size_t n_segments, float *dst, size_t dst_len);
void zo_segment_sum_csr(const float *src, size_t src_len, const uint64_t *row_offsets, size_t n_segments, float *dst);
void zo_index_select_fwd(const float *src, size_t src_len, const uint64_t *indices, size_t n_idx, size_t stride,
                         float *dst);
void zo_index_select_bwd(const float *y_grad, const uint64_t *indices, size_t n_idx, size_t stride, float *x_grad,
                         size_t x_len);
void zo_scatter_gcn_deg_scaled(float *dst, const float *h, const float *deg, const uint64_t *src_indices,
                               const uint64_t *tgt_indices, size_t stride, size_t n_edge);
void zo_scatter_gcn_deg_scaled_bwd(const float *grad_output, const float *h, const float *deg,
                                   const uint64_t *src_indices, const uint64_t *tgt_indices, float *grad_h,
                                   float *grad_deg, size_t stride, size_t n_edge);

/* ---- losses (host loops of src/nn/loss.zig lifted to ops) ---- */
/* one-hot float targets; writes softmax probabilities to `probs` and the mean loss to loss[0] */
void zo_smce_fwd(const float *logits, const float *target, float *probs, float *loss, size_t rows, size_t cols);
void zo_smce_bwd(const float *probs, const float *target, float *grad, size_t rows, size_t cols);
/* integer-label form of the same computation (label = index of the 1 in the one-hot row); lse[rows] saved */
void zo_smce_label_fwd(const float *logits, const uint64_t *labels, float *lse, float *loss, size_t rows, size_t cols);
void zo_smce_label_bwd(const float *logits, const uint64_t *labels, const float *lse, float *grad, size_t rows,
                       size_t cols);
void zo_softmax_fwd(const float *x, float *y, size_t rows, size_t cols);
void zo_softmax_bwd(const float *y, const float *y_g, float *x_g, size_t rows, size_t cols);
void zo_smooth_l1_fwd(const float *pred, const float *target, size_t n, float beta, float *loss);
void zo_smooth_l1_bwd(const float *pred, const float *target, float *grad, size_t n, float beta);
void zo_mse_fwd(const float *pred, const float *target, size_t n, float *loss);
void zo_mse_bwd(const float *pred, const float *target, float *grad, size_t n);

/* ---- optimizers ---- */
void zo_sgd_step(float *param, float *grad, size_t n, float lr, int clip, float max_norm, float delta);
/* t is the already-incremented per-tensor step counter of the reference */
void zo_adam_step(float *param, float *grad, float *m, float *v, size_t n, uint64_t t, float lr, float beta1,
                  float beta2, float epsilon, int clip, float max_norm, float delta);
float zo_adam_lr_t(uint64_t t, float lr, float beta1, float beta2);

#ifdef __cplusplus
}
#endif
#endif
