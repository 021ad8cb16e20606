/* One train step of the two-layer GCN of examples/gcn (model.zig:27-36, 100-224, 343-348; main.zig:68-84) issued op by op
 * through the C ABI from plain C: the same op sequence the Python trainer (zigrad_amd/trainers.py: GCNTrainer) issues,
 * without an interpreter between the calls.  Reads parameters, node features, the one-hot labels of the first M
 * (labelled) nodes and the edge list from a file of raw values (float32: W1 b1 W2 b2 x labels; then uint64: the E
 * source nodes, the E target nodes), runs `steps` steps (Adam lr 0.01, per-tensor clip 10 / 1e-6), prints the loss
 * of every step and the time per step.
 *
 *   gcn_step <input.bin> <steps> <nodes> <features> <hidden> <classes> <edges> <labelled>
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

static zg_hip_ctx *ctx;
static size_t N, E;
static const uint64_t *src_idx, *tgt_idx;
static size_t dims[3];
static float *W[2], *b[2], *Wg[2], *bg[2];

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

static float *device_floats(size_t n) {
    void *dev = NULL;
    CHECK(zg_hip_alloc(ctx, n * sizeof(float), &dev));
    return (float *)dev;
}
static float *upload(FILE *f, size_t n) {
    float *host = (float *)malloc(n * sizeof(float));
    if (fread(host, sizeof(float), n, f) != n) {
        fprintf(stderr, "input file too short\n");
        exit(1);
    }
    float *dev = device_floats(n);
    CHECK(zg_hip_memcpy_h2d(ctx, dev, host, n * sizeof(float)));
    free(host);
    return dev;
}
static float *zeros(size_t n) {
    float *p = device_floats(n);
    CHECK(zg_hip_mem_fill(ctx, p, n, 0.0f));
    return p;
}

/* C[M,N] = op(A) op(B) + beta * C through bmm_acc with one batch, as NDArray.bmm_acc_ sets it up */
static void bmm(const float *A, const float *B, float *C, size_t M, size_t Nc, size_t K, int ta, int tb, size_t lda,
                size_t ldb, float beta) {
    const uint64_t a[3] = {1, M, K}, bs[3] = {1, K, Nc}, c[3] = {1, M, Nc};
    CHECK(zg_hip_bmm_acc(ctx, A, a, B, bs, C, c, ta, tb, lda, ldb, Nc, 1.0f, beta));
}

static void unbroadcast_rows(const float *g, size_t rows, size_t cols, float *out) { /* out += column sums of g */
    const uint64_t xs[2] = {rows, cols}, ys[1] = {cols};
    const size_t scratch_len = zg_hip_unbroadcast_scratch_len(xs, 2, ys, 1);
    void *scratch = NULL;
    if (scratch_len) CHECK(zg_hip_mem_scratch(ctx, scratch_len * sizeof(float), &scratch));
    CHECK(zg_hip_unbroadcast(ctx, g, xs, 2, out, ys, 1, (float *)scratch, scratch_len, 1.0f, 1.0f));
}

typedef struct {
    const float *x;
    cached h, deg, y;
} saved;

/* deg^-1/2 with deg = 1 + in-degree, computed by every layer's forward (model.zig:116-224) */
static cached degree_norm(void) {
    cached deg = cache_alloc(N);
    CHECK(zg_hip_mem_fill(ctx, deg.ptr, N, 1.0f));
    cached ones_edges = cache_alloc(E);
    CHECK(zg_hip_mem_fill(ctx, ones_edges.ptr, E, 1.0f));
    cached contrib = cache_alloc(N);
    CHECK(zg_hip_mem_fill(ctx, contrib.ptr, N, 0.0f));
    CHECK(zg_hip_scatter_add(ctx, ones_edges.ptr, tgt_idx, E, contrib.ptr, N));
    cache_free(ones_edges);
    CHECK(zg_hip_add(ctx, contrib.ptr, N, deg.ptr, N, deg.ptr, N));
    cache_free(contrib);
    cached deg_norm = cache_alloc(N);
    CHECK(zg_hip_rsqrt_fwd(ctx, deg.ptr, deg_norm.ptr, N, 1e-12f));
    cache_free(deg);
    return deg_norm;
}

/* h = x W^T, y = aggregate(h) + b, relu in place after the first layer */
static saved conv_forward(int l, const float *x_in, int relu) {
    const size_t fan_in = dims[l], fan_out = dims[l + 1];
    saved s;
    s.x = x_in;
    s.h = cache_alloc(N * fan_out);
    bmm(x_in, W[l], s.h.ptr, N, fan_out, fan_in, 0, 1, fan_in, fan_in, 0.0f);
    s.deg = degree_norm();
    s.y = cache_alloc(N * fan_out);
    CHECK(zg_hip_mem_fill(ctx, s.y.ptr, N * fan_out, 0.0f));
    CHECK(zg_hip_scatter_gcn_deg_scaled(ctx, s.y.ptr, s.h.ptr, s.deg.ptr, src_idx, tgt_idx, fan_out, E, N));
    CHECK(zg_hip_add(ctx, b[l], fan_out, s.y.ptr, N * fan_out, s.y.ptr, N * fan_out));
    if (relu) CHECK(zg_hip_relu_fwd(ctx, s.y.ptr, s.y.ptr, N * fan_out));
    return s;
}

/* consumes g_y and what the forward saved; returns the input gradient (ptr null when none is needed) */
static cached conv_backward(int l, saved s, cached g_y, int need_input_grad) {
    const size_t fan_in = dims[l], fan_out = dims[l + 1];
    unbroadcast_rows(g_y.ptr, N, fan_out, bg[l]);
    cached g_h = cache_alloc(N * fan_out);
    CHECK(zg_hip_mem_fill(ctx, g_h.ptr, N * fan_out, 0.0f));
    cached g_deg = cache_alloc(N);
    CHECK(zg_hip_mem_fill(ctx, g_deg.ptr, N, 0.0f));
    CHECK(zg_hip_scatter_gcn_deg_scaled_bwd(ctx, g_y.ptr, s.h.ptr, s.deg.ptr, src_idx, tgt_idx, g_h.ptr, g_deg.ptr, fan_out,
                                            E, N));
    cache_free(g_deg); /* the degrees need no gradient: the chain stops at rsqrt (src/ndtensor.zig:1009) */
    cache_free(g_y);
    cache_free(s.y);
    cache_free(s.deg);
    cached g_x = {NULL, 0};
    if (need_input_grad) {
        g_x = cache_alloc(N * fan_in);
        CHECK(zg_hip_mem_fill(ctx, g_x.ptr, N * fan_in, 0.0f));
        bmm(g_h.ptr, W[l], g_x.ptr, N, fan_in, fan_out, 0, 0, fan_out, fan_in, 1.0f); /* dA += dC . B */
    }
    bmm(g_h.ptr, s.x, Wg[l], fan_out, fan_in, N, 1, 0, fan_out, fan_in, 1.0f);         /* dB += dC^T . A */
    cache_free(g_h);
    cache_free(s.h);
    return g_x;
}

int main(int argc, char **argv) {
    if (argc != 9) {
        fprintf(stderr, "usage: %s input.bin steps nodes features hidden classes edges labelled\n", argv[0]);
        return 2;
    }
    const int steps = atoi(argv[2]);
    N = (size_t)atol(argv[3]);
    dims[0] = (size_t)atol(argv[4]), dims[1] = (size_t)atol(argv[5]), dims[2] = (size_t)atol(argv[6]);
    E = (size_t)atol(argv[7]);
    const size_t M = (size_t)atol(argv[8]), C = dims[2];
    const float lr = 0.01f, beta1 = 0.9f, beta2 = 0.999f, epsilon = 1e-8f;
    FILE *f = fopen(argv[1], "rb");
    if (!f) {
        perror(argv[1]);
        return 2;
    }
    CHECK(zg_hip_init(0, &ctx));
    float *m[4], *v[4];
    for (int l = 0; l < 2; l++) {
        const size_t nw = dims[l + 1] * dims[l], nb = dims[l + 1];
        W[l] = upload(f, nw);
        b[l] = upload(f, nb);
        Wg[l] = zeros(nw), bg[l] = zeros(nb);
        m[2 * l] = zeros(nw), v[2 * l] = zeros(nw);
        m[2 * l + 1] = zeros(nb), v[2 * l + 1] = zeros(nb);
    }
    float *x = upload(f, N * dims[0]);
    float *labels = upload(f, M * C);
    /* the edge list lives where the host can write it and the kernels can read it */
    void *edges = NULL;
    CHECK(zg_hip_host_alloc(ctx, 2 * E * sizeof(uint64_t), &edges));
    if (fread(edges, sizeof(uint64_t), 2 * E, f) != 2 * E) {
        fprintf(stderr, "input file too short\n");
        return 1;
    }
    fclose(f);
    src_idx = (const uint64_t *)edges;
    tgt_idx = src_idx + E;

    uint64_t t = 0; /* Adam's counter: once per parameter tensor update (src/nn/optim.zig:189) */
    struct timespec t0, t1;
    const int warm = steps > 20 ? 10 : 0;
    for (int s = 0; s < steps; s++) {
        if (s == warm) {
            CHECK(zg_hip_sync(ctx));
            clock_gettime(CLOCK_MONOTONIC, &t0);
        }
        saved s1 = conv_forward(0, x, 1);
        saved s2 = conv_forward(1, s1.y.ptr, 0);
        cached out_m = cache_alloc(M * C); /* MaskLayer.forward: the labelled rows, one contiguous prefix */
        CHECK(zg_hip_memcpy_d2d(ctx, out_m.ptr, s2.y.ptr, M * C * sizeof(float)));
        cached probs = cache_alloc(M * C), loss = cache_alloc(1), g_m = cache_alloc(M * C), loss_grad = cache_alloc(1);
        CHECK(zg_hip_smce_fwd(ctx, out_m.ptr, labels, probs.ptr, loss.ptr, M, C));
        float loss_host = 0.0f;
        CHECK(zg_hip_memcpy_d2h(ctx, &loss_host, loss.ptr, sizeof(float)));
        printf("loss %.9g\n", loss_host);
        /* backward */
        CHECK(zg_hip_mem_fill(ctx, loss_grad.ptr, 1, 1.0f));
        CHECK(zg_hip_mem_fill(ctx, g_m.ptr, M * C, 0.0f));
        CHECK(zg_hip_smce_bwd(ctx, probs.ptr, labels, g_m.ptr, M, C));
        cached g2 = cache_alloc(N * C);
        CHECK(zg_hip_mem_fill(ctx, g2.ptr, N * C, 0.0f));
        CHECK(zg_hip_memcpy_d2d(ctx, g2.ptr, g_m.ptr, M * C * sizeof(float))); /* MaskLayer.backward */
        cache_free(probs);
        cache_free(loss);
        cache_free(loss_grad);
        cache_free(g_m);
        cache_free(out_m);
        cached g1 = conv_backward(1, s2, g2, 1);
        CHECK(zg_hip_relu_inplace_bwd(ctx, s1.y.ptr, g1.ptr, N * dims[1]));
        (void)conv_backward(0, s1, g1, 0);
        /* optim.step(), then zero_grad() */
        for (int l = 0; l < 2; l++) {
            CHECK(zg_hip_adam_step(ctx, W[l], Wg[l], m[2 * l], v[2 * l], dims[l + 1] * dims[l], ++t, lr, beta1, beta2, epsilon,
                                   1, 10.0f, 1e-6f));
            CHECK(zg_hip_adam_step(ctx, b[l], bg[l], m[2 * l + 1], v[2 * l + 1], dims[l + 1], ++t, lr, beta1, beta2, epsilon, 1,
                                   10.0f, 1e-6f));
        }
        for (int l = 0; l < 2; l++) {
            CHECK(zg_hip_mem_fill(ctx, Wg[l], dims[l + 1] * dims[l], 0.0f));
            CHECK(zg_hip_mem_fill(ctx, bg[l], dims[l + 1], 0.0f));
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
