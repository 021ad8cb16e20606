/* The batch-64 MLP train step of examples/mnist (model.zig:34-110, main-simple.zig:55-86) issued op by op through the
 * C ABI from plain C: the same op sequence the Python trainer (zigrad_amd/trainers.py: MLPTrainer) issues, without an
 * interpreter between the calls.  Reads parameters and one batch from a file of raw float32
 * (W1 b1 W2 b2 W3 b3 x onehot), runs `steps` SGD steps (lr 0.01, per-tensor clip 10 / 1e-6), prints the loss of every
 * step and the time per step.
 *
 *   mlp_step <input.bin> <steps> <batch> <d0> <d1> <d2> <d3> [fused]
 *
 * With `fused` the step goes through the fused entry points instead (linear_fwd, smce_fwd_bwd, linear_bwd,
 * sgd_step_multi): the same values in 13 launches instead of 43.
 */
#include <stdio.h>
#include <stdlib.h>
#include <time.h>
#include "zg_hip.h"

#define CHECK(call)                                                                    \
    do {                                                                               \
        if ((call) != 0) {                                                             \
            fprintf(stderr, "%s failed: %s\n", #call, zg_hip_last_error());            \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

enum { LAYERS = 3 };
static zg_hip_ctx *ctx;

typedef struct {
    float *ptr;
    uint64_t block;
} cached;

static cached cache_alloc(size_t n) {
    cached c;
    void *p = NULL;
    CHECK(zg_hip_mem_cache_alloc(ctx, n * sizeof(float), &p, &c.block));
    c.ptr = (float *)p;
    return c;
}
static void cache_free(cached c) { CHECK(zg_hip_mem_cache_free(ctx, c.ptr, c.block)); }

static float *upload(FILE *f, size_t n) {
    float *host = (float *)malloc(n * sizeof(float));
    void *dev = NULL;
    if (fread(host, sizeof(float), n, f) != n) {
        fprintf(stderr, "input file too short\n");
        exit(1);
    }
    CHECK(zg_hip_alloc(ctx, n * sizeof(float), &dev));
    CHECK(zg_hip_memcpy_h2d(ctx, dev, host, n * sizeof(float)));
    free(host);
    return (float *)dev;
}

/* C[M,N] = alpha * op(A) op(B) + beta * C through bmm_acc with one batch, as NDArray.bmm_acc_ sets it up */
static void bmm(const float *A, const float *B, float *C, size_t M, size_t N, size_t K, int ta, int tb, size_t lda,
                size_t ldb, float beta) {
    const uint64_t a[3] = {1, M, K}, b[3] = {1, K, N}, c[3] = {1, M, N};
    CHECK(zg_hip_bmm_acc(ctx, A, a, B, b, C, c, ta, tb, lda, ldb, N, 1.0f, beta));
}

int main(int argc, char **argv) {
    if (argc != 8 && argc != 9) {
        fprintf(stderr, "usage: %s input.bin steps batch d0 d1 d2 d3 [fused]\n", argv[0]);
        return 2;
    }
    const int fused = argc == 9;
    const int steps = atoi(argv[2]);
    const size_t B = (size_t)atol(argv[3]);
    size_t d[LAYERS + 1];
    for (int i = 0; i <= LAYERS; i++) d[i] = (size_t)atol(argv[4 + i]);
    const size_t C = d[LAYERS];
    FILE *f = fopen(argv[1], "rb");
    if (!f) {
        perror(argv[1]);
        return 2;
    }
    CHECK(zg_hip_init(0, &ctx));
    float *W[LAYERS], *b[LAYERS], *Wg[LAYERS], *bg[LAYERS];
    for (int l = 0; l < LAYERS; l++) {
        W[l] = upload(f, d[l + 1] * d[l]);
        b[l] = upload(f, d[l + 1]);
    }
    float *x = upload(f, B * d[0]);
    float *onehot = upload(f, B * C);
    fclose(f);
    for (int l = 0; l < LAYERS; l++) {
        void *p = NULL;
        CHECK(zg_hip_alloc(ctx, d[l + 1] * d[l] * sizeof(float), &p));
        Wg[l] = (float *)p;
        CHECK(zg_hip_alloc(ctx, d[l + 1] * sizeof(float), &p));
        bg[l] = (float *)p;
        CHECK(zg_hip_mem_fill(ctx, Wg[l], d[l + 1] * d[l], 0.0f));
        CHECK(zg_hip_mem_fill(ctx, bg[l], d[l + 1], 0.0f));
    }

    struct timespec t0, t1;
    const int warm = steps > 20 ? 10 : 0;
    for (int s = 0; s < steps; s++) {
        if (s == warm) {
            CHECK(zg_hip_sync(ctx));
            clock_gettime(CLOCK_MONOTONIC, &t0);
        }
        cached act[LAYERS + 1];
        act[0].ptr = x;
        if (fused) {
            for (int l = 0; l < LAYERS; l++) {
                act[l + 1] = cache_alloc(B * d[l + 1]);
                CHECK(zg_hip_linear_fwd(ctx, act[l].ptr, W[l], b[l], act[l + 1].ptr, B, d[l], d[l + 1], l + 1 < LAYERS));
            }
            cached loss = cache_alloc(1), probs = cache_alloc(B * C), g = cache_alloc(B * C);
            CHECK(zg_hip_smce_fwd_bwd(ctx, act[LAYERS].ptr, onehot, probs.ptr, loss.ptr, g.ptr, B, C, 0));
            float loss_host = 0.0f;
            CHECK(zg_hip_memcpy_d2h(ctx, &loss_host, loss.ptr, sizeof(float)));
            printf("loss %.9g\n", loss_host);
            cache_free(probs);
            cache_free(loss);
            for (int l = LAYERS - 1; l >= 0; l--) {
                cached g_prev = {NULL, 0};
                if (l > 0) g_prev = cache_alloc(B * d[l]);
                CHECK(zg_hip_linear_bwd(ctx, g.ptr, act[l].ptr, W[l], l > 0 ? act[l].ptr : NULL, Wg[l], bg[l], g_prev.ptr, B,
                                        d[l], d[l + 1]));
                cache_free(act[l + 1]);
                cache_free(g);
                g = g_prev;
            }
            float *params[2 * LAYERS], *grads[2 * LAYERS];
            size_t lens[2 * LAYERS];
            for (int l = 0; l < LAYERS; l++) {
                params[2 * l] = W[l], grads[2 * l] = Wg[l], lens[2 * l] = d[l + 1] * d[l];
                params[2 * l + 1] = b[l], grads[2 * l + 1] = bg[l], lens[2 * l + 1] = d[l + 1];
            }
            CHECK(zg_hip_sgd_step_multi(ctx, 2 * LAYERS, params, grads, lens, 0.01f, 1, 10.0f, 1e-6f, 1));
            continue;
        }
        /* forward: y = x . W^T, y += bias, relu in place (not after the last layer) */
        for (int l = 0; l < LAYERS; l++) {
            act[l + 1] = cache_alloc(B * d[l + 1]);
            bmm(act[l].ptr, W[l], act[l + 1].ptr, B, d[l + 1], d[l], 0, 1, d[l], d[l], 0.0f);
            CHECK(zg_hip_add(ctx, b[l], d[l + 1], act[l + 1].ptr, B * d[l + 1], act[l + 1].ptr, B * d[l + 1]));
            if (l + 1 < LAYERS) CHECK(zg_hip_relu_fwd(ctx, act[l + 1].ptr, act[l + 1].ptr, B * d[l + 1]));
        }
        cached loss = cache_alloc(1), probs = cache_alloc(B * C);
        CHECK(zg_hip_smce_fwd(ctx, act[LAYERS].ptr, onehot, probs.ptr, loss.ptr, B, C));
        float loss_host = 0.0f; /* loss.get(0): a blocking read before backward, as the reference's loop does */
        CHECK(zg_hip_memcpy_d2h(ctx, &loss_host, loss.ptr, sizeof(float)));
        printf("loss %.9g\n", loss_host);

        /* backward */
        cached loss_grad = cache_alloc(1), g = cache_alloc(B * C);
        CHECK(zg_hip_mem_fill(ctx, loss_grad.ptr, 1, 1.0f));
        CHECK(zg_hip_mem_fill(ctx, g.ptr, B * C, 0.0f));
        CHECK(zg_hip_smce_bwd(ctx, probs.ptr, onehot, g.ptr, B, C));
        cache_free(probs);
        cache_free(loss_grad);
        cache_free(loss);
        for (int l = LAYERS - 1; l >= 0; l--) {
            const size_t in = d[l], out = d[l + 1];
            if (l + 1 < LAYERS) CHECK(zg_hip_relu_inplace_bwd(ctx, act[l + 1].ptr, g.ptr, B * out));
            const uint64_t xs[2] = {B, out}, ys[1] = {out};
            const size_t scratch_len = zg_hip_unbroadcast_scratch_len(xs, 2, ys, 1);
            void *scratch = NULL;
            if (scratch_len) CHECK(zg_hip_mem_scratch(ctx, scratch_len * sizeof(float), &scratch));
            CHECK(zg_hip_unbroadcast(ctx, g.ptr, xs, 2, bg[l], ys, 1, (float *)scratch, scratch_len, 1.0f, 1.0f));
            cached g_prev = {NULL, 0};
            if (l > 0) { /* the network input needs no gradient */
                g_prev = cache_alloc(B * in);
                CHECK(zg_hip_mem_fill(ctx, g_prev.ptr, B * in, 0.0f));
                bmm(g.ptr, W[l], g_prev.ptr, B, in, out, 0, 0, out, in, 1.0f); /* dA += dC . B */
            }
            bmm(g.ptr, act[l].ptr, Wg[l], out, in, B, 1, 0, out, in, 1.0f);    /* dB += dC^T . A */
            cache_free(act[l + 1]);
            cache_free(g);
            g = g_prev;
        }
        /* optim.step(), then model.zero_grad() */
        for (int l = 0; l < LAYERS; l++) {
            CHECK(zg_hip_sgd_step(ctx, W[l], Wg[l], d[l + 1] * d[l], 0.01f, 1, 10.0f, 1e-6f));
            CHECK(zg_hip_sgd_step(ctx, b[l], bg[l], d[l + 1], 0.01f, 1, 10.0f, 1e-6f));
        }
        for (int l = 0; l < LAYERS; l++) {
            CHECK(zg_hip_mem_fill(ctx, Wg[l], d[l + 1] * d[l], 0.0f));
            CHECK(zg_hip_mem_fill(ctx, bg[l], d[l + 1], 0.0f));
        }
    }
    CHECK(zg_hip_sync(ctx));
    clock_gettime(CLOCK_MONOTONIC, &t1);
    if (steps > warm)
        printf("us_per_step %.2f\n",
               ((double)(t1.tv_sec - t0.tv_sec) * 1e6 + (double)(t1.tv_nsec - t0.tv_nsec) * 1e-3) / (steps - warm));
    CHECK(zg_hip_deinit(ctx));
    return 0;
}
