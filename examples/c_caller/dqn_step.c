/* One DQN update of examples/dqn (dqn_agent.zig:125-228 without its host-side clamps; network 4 -> 128 -> 128 -> 2)
 * issued op by op through the C ABI from plain C: the same op sequence the Python trainer (zigrad_amd/trainers.py:
 * DQNTrainer) issues, without an interpreter between the calls.  Reads the policy network's parameters (the target
 * network starts as a copy) and one replay batch from a file of raw values
 * (float32: W1 b1 W2 b2 W3 b3 states next_states rewards dones; then uint64: actions), runs `steps` updates
 * (Adam lr 1e-3, per-tensor clip 10 / 1e-6, gamma 0.99), prints the loss of every update and the time per update.
 *
 *   dqn_step <input.bin> <steps> <batch> <d0> <d1> <d2> <d3>
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

static cached cache_alloc_bytes(size_t bytes) {
    cached c;
    void *p = NULL;
    CHECK(zg_hip_mem_cache_alloc(ctx, bytes, &p, &c.block));
    c.ptr = (float *)p;
    return c;
}
static cached cache_alloc(size_t n) { return cache_alloc_bytes(n * sizeof(float)); }
static void cache_free(cached c) { CHECK(zg_hip_mem_cache_free(ctx, c.ptr, c.block)); }

static void *device_alloc(size_t bytes) {
    void *dev = NULL;
    CHECK(zg_hip_alloc(ctx, bytes, &dev));
    return dev;
}
static void *upload(FILE *f, size_t n, size_t elem) {
    void *host = malloc(n * elem);
    if (fread(host, elem, n, f) != n) {
        fprintf(stderr, "input file too short\n");
        exit(1);
    }
    void *dev = device_alloc(n * elem);
    CHECK(zg_hip_memcpy_h2d(ctx, dev, host, n * elem));
    free(host);
    return dev;
}
static float *zeros(size_t n) {
    float *p = (float *)device_alloc(n * sizeof(float));
    CHECK(zg_hip_mem_fill(ctx, p, n, 0.0f));
    return p;
}

/* C[M,N] = op(A) op(B) + beta * C through bmm_acc with one batch, as NDArray.bmm_acc_ sets it up */
static void bmm(const float *A, const float *B, float *C, size_t M, size_t N, size_t K, int ta, int tb, size_t lda,
                size_t ldb, float beta) {
    const uint64_t a[3] = {1, M, K}, b[3] = {1, K, N}, c[3] = {1, M, N};
    CHECK(zg_hip_bmm_acc(ctx, A, a, B, b, C, c, ta, tb, lda, ldb, N, 1.0f, beta));
}

/* y = x . W^T, y += bias, relu in place (not after the last layer); act[0] = x, act[l + 1] are cache allocations */
static void forward(float *const *W, float *const *b, const size_t *d, size_t B, cached *act) {
    for (int l = 0; l < LAYERS; l++) {
        act[l + 1] = cache_alloc(B * d[l + 1]);
        bmm(act[l].ptr, W[l], act[l + 1].ptr, B, d[l + 1], d[l], 0, 1, d[l], d[l], 0.0f);
        CHECK(zg_hip_add(ctx, b[l], d[l + 1], act[l + 1].ptr, B * d[l + 1], act[l + 1].ptr, B * d[l + 1]));
        if (l + 1 < LAYERS) CHECK(zg_hip_relu_fwd(ctx, act[l + 1].ptr, act[l + 1].ptr, B * d[l + 1]));
    }
}

int main(int argc, char **argv) {
    if (argc != 8) {
        fprintf(stderr, "usage: %s input.bin steps batch d0 d1 d2 d3\n", argv[0]);
        return 2;
    }
    const int steps = atoi(argv[2]);
    const size_t B = (size_t)atol(argv[3]);
    size_t d[LAYERS + 1];
    for (int i = 0; i <= LAYERS; i++) d[i] = (size_t)atol(argv[4 + i]);
    const size_t S = d[0], A = d[LAYERS];
    const float lr = 1e-3f, beta1 = 0.9f, beta2 = 0.999f, epsilon = 1e-8f;
    FILE *f = fopen(argv[1], "rb");
    if (!f) {
        perror(argv[1]);
        return 2;
    }
    CHECK(zg_hip_init(0, &ctx));
    float *W[LAYERS], *b[LAYERS], *Wt[LAYERS], *bt[LAYERS], *Wg[LAYERS], *bg[LAYERS];
    float *m[2 * LAYERS], *v[2 * LAYERS];
    for (int l = 0; l < LAYERS; l++) {
        const size_t nw = d[l + 1] * d[l], nb = d[l + 1];
        W[l] = (float *)upload(f, nw, sizeof(float));
        b[l] = (float *)upload(f, nb, sizeof(float));
        Wt[l] = (float *)device_alloc(nw * sizeof(float));
        bt[l] = (float *)device_alloc(nb * sizeof(float));
        CHECK(zg_hip_memcpy_d2d(ctx, Wt[l], W[l], nw * sizeof(float)));
        CHECK(zg_hip_memcpy_d2d(ctx, bt[l], b[l], nb * sizeof(float)));
        Wg[l] = zeros(nw), bg[l] = zeros(nb);
        m[2 * l] = zeros(nw), v[2 * l] = zeros(nw);
        m[2 * l + 1] = zeros(nb), v[2 * l + 1] = zeros(nb);
    }
    float *states = (float *)upload(f, B * S, sizeof(float));
    float *next_states = (float *)upload(f, B * S, sizeof(float));
    float *rewards = (float *)upload(f, B, sizeof(float));
    float *dones = (float *)upload(f, B, sizeof(float));
    uint64_t *actions = (uint64_t *)upload(f, B, sizeof(uint64_t));
    fclose(f);
    /* gamma and 1 stay on the host: scalar operands go to the device by value, as a binding passes the one-element
     * host slice of NDArray's scalar ops (src/ndarray.zig:247-257) */
    const float gamma = 0.99f, one = 1.0f;

    uint64_t t = 0; /* Adam's counter: once per parameter tensor update (src/nn/optim.zig:189) */
    struct timespec t0, t1;
    const int warm = steps > 20 ? 10 : 0;
    for (int s = 0; s < steps; s++) {
        if (s == warm) {
            CHECK(zg_hip_sync(ctx));
            clock_gettime(CLOCK_MONOTONIC, &t0);
        }
        /* TD target, no gradient: r + gamma * max_a Q_target(s', a) * (1 - done) */
        cached act_t[LAYERS + 1];
        act_t[0].ptr = next_states;
        forward(Wt, bt, d, B, act_t);
        cached max_next = cache_alloc(B);
        CHECK(zg_hip_mem_fill(ctx, max_next.ptr, B, 0.0f)); /* NDArray.max_along writes into a zero-filled output */
        const uint64_t q_shape[2] = {B, A};
        CHECK(zg_hip_max_along(ctx, act_t[LAYERS].ptr, q_shape, 2, max_next.ptr, B, 1));
        for (int l = 1; l <= LAYERS; l++) cache_free(act_t[l]);
        cached disc = cache_alloc(B);
        CHECK(zg_hip_mul_scalar(ctx, max_next.ptr, B, gamma, 0, disc.ptr));
        cached not_done = cache_alloc(B);
        CHECK(zg_hip_sub_scalar(ctx, dones, B, one, 1, not_done.ptr)); /* 1 - done: the scalar is the left operand */
        cached masked = cache_alloc(B);
        CHECK(zg_hip_mul(ctx, disc.ptr, B, not_done.ptr, B, masked.ptr, B));
        cached targets = cache_alloc(B);
        CHECK(zg_hip_add(ctx, rewards, B, masked.ptr, B, targets.ptr, B));
        cache_free(max_next);
        cache_free(disc);
        cache_free(not_done);
        cache_free(masked);

        /* Q(s, a) */
        cached act[LAYERS + 1];
        act[0].ptr = states;
        forward(W, b, d, B, act);
        const uint64_t idx_shape[2] = {B, 1};
        cached offsets = cache_alloc_bytes(B * sizeof(uint64_t)), q = cache_alloc(B);
        CHECK(zg_hip_gather(ctx, act[LAYERS].ptr, q_shape, idx_shape, 2, actions, 1, (uint64_t *)offsets.ptr, q.ptr, NULL));
        cached loss = cache_alloc(1), loss_grad = cache_alloc(1), g_q = cache_alloc(B);
        CHECK(zg_hip_smooth_l1_fwd(ctx, q.ptr, targets.ptr, B, 1.0f, loss.ptr));
        for (int l = 0; l < LAYERS; l++) { /* zero_grad() */
            CHECK(zg_hip_mem_fill(ctx, Wg[l], d[l + 1] * d[l], 0.0f));
            CHECK(zg_hip_mem_fill(ctx, bg[l], d[l + 1], 0.0f));
        }
        /* backward */
        CHECK(zg_hip_mem_fill(ctx, loss_grad.ptr, 1, 1.0f));
        CHECK(zg_hip_mem_fill(ctx, g_q.ptr, B, 0.0f));
        CHECK(zg_hip_smooth_l1_bwd(ctx, q.ptr, targets.ptr, g_q.ptr, B, 1.0f));
        cached g = cache_alloc(B * A);
        CHECK(zg_hip_mem_fill(ctx, g.ptr, B * A, 0.0f));
        CHECK(zg_hip_scatter_add(ctx, g_q.ptr, (const uint64_t *)offsets.ptr, B, g.ptr, B * A)); /* GatherBwd */
        cache_free(offsets);
        cache_free(g_q);
        cache_free(loss_grad);
        cache_free(q);
        cache_free(targets);
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
        /* optim.step(): weights, then bias, layer by layer */
        for (int l = 0; l < LAYERS; l++) {
            CHECK(zg_hip_adam_step(ctx, W[l], Wg[l], m[2 * l], v[2 * l], d[l + 1] * d[l], ++t, lr, beta1, beta2, epsilon, 1,
                                   10.0f, 1e-6f));
            CHECK(zg_hip_adam_step(ctx, b[l], bg[l], m[2 * l + 1], v[2 * l + 1], d[l + 1], ++t, lr, beta1, beta2, epsilon, 1,
                                   10.0f, 1e-6f));
        }
        float loss_host = 0.0f;
        CHECK(zg_hip_memcpy_d2h(ctx, &loss_host, loss.ptr, sizeof(float)));
        printf("loss %.9g\n", loss_host);
        cache_free(loss);
    }
    CHECK(zg_hip_sync(ctx));
    clock_gettime(CLOCK_MONOTONIC, &t1);
    if (steps > warm)
        printf("us_per_step %.2f\n",
               ((double)(t1.tv_sec - t0.tv_sec) * 1e6 + (double)(t1.tv_nsec - t0.tv_nsec) * 1e-3) / (steps - warm));
    CHECK(zg_hip_deinit(ctx));
    return 0;
}
