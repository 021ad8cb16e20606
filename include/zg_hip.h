/*
 * zg_hip.h -- C ABI of the MI355X (gfx950) device backend for Zigrad.
 *
 * One entry point per device op that Zigrad reaches through
 * DeviceReference.dispatch (reference: src/device/device_reference.zig:15-27,
 * parameter structs in src/device/opspec.zig) plus the memory API of
 * src/device/device_reference.zig:29-131.  A Zig `HipDevice` struct binds these
 * one-to-one (see zig/hip_device.zig); the structural precedent on the reference
 * side is src/cuda/{cuda_utils,blas_conflux,nn_conflux}.h.
 *
 * Conventions
 *   - element type is fp32 throughout (every configuration of the reference's
 *     examples is fp32); `usize` of the reference is uint64_t here;
 *   - a reference slice `[]T` becomes (pointer, length); all data pointers are
 *     DEVICE pointers unless a parameter is documented as host memory;
 *     index arrays may live in device memory or in pinned host memory obtained
 *     from zg_hip_host_alloc (both are readable by the kernels);
 *   - shapes (x_shape, A_shape, ...) are HOST arrays, as in the reference where
 *     they are stack slices (src/ndarray.zig:884-888);
 *   - every call is asynchronous on the context's single stream, in order,
 *     except where stated (d2h copies block, as NDTensor.get needs:
 *     src/ndtensor.zig:524-528);
 *   - every function returns 0 on success and a ZG_HIP_E* code otherwise;
 *     zg_hip_last_error() gives the message.  The reference's ops return void
 *     and panic on failure (src/device/device_reference.zig:20-22); the Zig
 *     binding turns a non-zero return into @panic.
 *   - argument checks happen on the host before any launch; a rejected call
 *     launches nothing;
 *   - "in order" describes what a caller can observe, not when kernels are launched: some calls (float fills, a
 *     layer's products, its bias gradient, optimizer steps, the graph-convolution aggregation) are held inside the
 *     context for the calls that usually follow them and leave in fewer launches with the same values, and every
 *     other call launches what is held first (the comments at those entry points say what is held and for what);
 *   - OPERAND LIFETIME.  Because work is held, a call that returned ZG_HIP_OK may still name its operands: every
 *     pointer handed to a call (device operands, pinned host index arrays, a pinned or device alpha / lr_t) must stay
 *     valid AND unchanged until the next call on the context that launches what is held: zg_hip_sync, zg_hip_flush,
 *     zg_hip_stream, or any op that is not itself held.  Memory from this context's own allocators may be given back
 *     at once (the free calls know what is held).  A caller that mixes its own HIP calls with the library's -- its own
 *     hipMalloc / hipFree of operands, hipDeviceSynchronize followed by its own hipMemcpy of a result, kernels on a
 *     stream handle fetched EARLIER from zg_hip_stream -- must call zg_hip_flush (or zg_hip_stream again) first, or
 *     switch holding off for the context with zg_hip_set_holding(ctx, 0): then every call launches its own work
 *     before it returns and the in-order stream alone decides what is visible, as in a library that holds nothing.
 *     An error of held work (a failed launch) is reported by the call that launches it, not by the call that queued
 *     it; with holding off it is reported by the next call on the context;
 *   - a context belongs to one host thread at a time (the reference's devices are not shared between threads
 *     either); different contexts may be used from different threads.
 */
#ifndef ZG_HIP_H
#define ZG_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct zg_hip_ctx zg_hip_ctx;
typedef struct zg_hip_event zg_hip_event;
typedef struct zg_hip_graph zg_hip_graph;

enum {
    ZG_HIP_OK = 0,
    ZG_HIP_EINVAL = 1,   /* argument/shape check failed; nothing was launched */
    ZG_HIP_EOOM = 2,     /* device allocation failed (reference: Error.DeviceOOM, src/allocators/device_data.zig:44) */
    ZG_HIP_ERUNTIME = 3, /* a HIP runtime call failed */
    ZG_HIP_ECAPTURE = 4, /* the call synchronises, allocates from the driver or touches host memory and was made
                            while an execution graph was being captured (or a graph call was made out of order) */
};

/* kinds for zg_hip_mem_random (reference: RandType, src/device/device_common.zig:3) */
enum { ZG_RAND_UNIFORM = 0, ZG_RAND_NORMAL = 1, ZG_RAND_KAIMING = 2 };

/* ---------------------------------------------------------------------------------------------
 * context (replaces HostDevice.init/deinit/sync: src/device/host_device.zig:183-196, :960;
 * shape precedent: src/device/cuda_device.zig:126-160)
 * ------------------------------------------------------------------------------------------- */
const char *zg_hip_last_error(void);
int zg_hip_device_count(int *count);
int zg_hip_init(int device_id, zg_hip_ctx **out);
/* Launches what waits, waits for the stream and releases everything the context owns.  The context is gone afterwards
 * whatever is returned; a non-zero return reports an error of work that was still held. */
int zg_hip_deinit(zg_hip_ctx *ctx);
int zg_hip_sync(zg_hip_ctx *ctx);
/* Launches whatever earlier calls left waiting in the context and returns without waiting for the stream (no
 * counterpart in the reference, which holds nothing).  For callers that are about to touch operands or results with
 * HIP calls of their own; see OPERAND LIFETIME above. */
int zg_hip_flush(zg_hip_ctx *ctx);
/* enable = 0: from now on every call launches its own work before it returns (what waits now is launched first);
 * enable = 1 (the state of a new context): calls may leave work waiting for the calls that follow.  Values are the
 * same either way; holding only saves launches. */
int zg_hip_set_holding(zg_hip_ctx *ctx, int enable);
int zg_hip_total_memory(zg_hip_ctx *ctx, size_t *bytes);
/* the HIP stream every op is enqueued on, as an opaque pointer (hipStream_t).  What waits in the context is launched
 * first; NULL when that fails (zg_hip_last_error has the reason) or ctx is NULL. */
void *zg_hip_stream(zg_hip_ctx *ctx);

/* timing helpers on the context's stream (hipEvent_t underneath) */
int zg_hip_event_create(zg_hip_ctx *ctx, zg_hip_event **out);
int zg_hip_event_record(zg_hip_ctx *ctx, zg_hip_event *ev);
int zg_hip_event_elapsed_ms(zg_hip_event *start, zg_hip_event *stop, float *ms); /* blocks until `stop` completed */
int zg_hip_event_destroy(zg_hip_event *ev);

/* ---------------------------------------------------------------------------------------------
 * DataHandler primitives for src/allocators/caching_allocator.zig (contract: map/unmap/alloc/free/
 * page_size; host version src/device/host_device.zig:50-110, cuda version src/device/cuda_device.zig:21-81)
 * ------------------------------------------------------------------------------------------- */
int zg_hip_page_size(zg_hip_ctx *ctx, size_t *bytes);
int zg_hip_pool_map(zg_hip_ctx *ctx, size_t bytes, void **out);  /* one contiguous device region for a block pool */
int zg_hip_pool_unmap(zg_hip_ctx *ctx, void *ptr);
int zg_hip_alloc(zg_hip_ctx *ctx, size_t bytes, void **out);    /* mem_alloc: src/device/host_device.zig:890-898 */
int zg_hip_free(zg_hip_ctx *ctx, void *ptr);                    /* mem_free:  src/device/host_device.zig:900-903 */
/* Pinned host memory that the host reads and writes through the pointer and the kernels read and write in place (no
 * counterpart in the reference, whose one device is the host): what a binding serves every `usize` allocation from,
 * because the reference's callers fill and read index tensors with host loops over `.raw` (NDArray.gather,
 * src/ndarray.zig:607-624; the GCN's edge lists, examples/gcn/src/model.zig:204-205).  Blocks of up to 16 MiB that are
 * given back are kept (256 MiB at most, until zg_hip_clear_cache) and reused for requests of the same power-of-two
 * size class, so a tensor of indices per train step costs no driver call; a reused block is handed out only after the
 * stream has passed the point at which it was given back. */
int zg_hip_host_alloc(zg_hip_ctx *ctx, size_t bytes, void **out);
int zg_hip_host_free(zg_hip_ctx *ctx, void *ptr);

/* The library's own caching allocator (two block pools, small <= 1 MiB and large, over segments obtained on
 * demand, + grow-only scratch), the C++ counterpart of CachingAllocator(DataHandler)
 * (src/allocators/caching_allocator.zig:15-162): blocks are split on allocation and fused with free neighbours on
 * release (src/allocators/block_pool.zig:185-324), every operation in constant time.  `block` is the DeviceData.ctx
 * of the reference (src/allocators/device_data.zig:32-40): an opaque non-zero handle that zg_hip_mem_cache_free
 * takes back together with the pointer.  A zero-byte request yields (NULL, 0).  cache_configure sets the size of the
 * segments each pool grows by. */
int zg_hip_cache_configure(zg_hip_ctx *ctx, size_t small_pool_bytes, size_t large_pool_bytes);
int zg_hip_mem_cache_alloc(zg_hip_ctx *ctx, size_t bytes, void **out, uint64_t *block);
int zg_hip_mem_cache_free(zg_hip_ctx *ctx, void *ptr, uint64_t block);
int zg_hip_mem_scratch(zg_hip_ctx *ctx, size_t bytes, void **out); /* src/allocators/caching_allocator.zig:133-156 */
int zg_hip_clear_cache(zg_hip_ctx *ctx);
/* *yes = 1 when ptr lies in memory this context handed out as device memory (cache pools, zg_hip_alloc /
 * zg_hip_pool_map regions, the scratch buffer), else 0.  The reference's callers pass host scalars and device slices
 * through the same parameters (src/ndarray.zig:251 and src/nn/optim.zig:117 against src/ndtensor.zig:1146-1150); a
 * binding tells them apart with this range test.  A pure host-side lookup: nothing is launched and work that waits in
 * the context keeps waiting. */
int zg_hip_is_device_ptr(zg_hip_ctx *ctx, const void *ptr, int *yes);
/* host counters; nothing is launched and what waits keeps waiting */
int zg_hip_cache_stats(zg_hip_ctx *ctx, size_t *bytes_in_use, size_t *bytes_mapped, uint64_t *n_device_allocs);
/* Kernels launched by the library in this process so far (all contexts together), device-to-device copies included (no counterpart in the
 * reference; for tests and for reading profiles: how many launches an op sequence costs).  Work still waiting in the
 * context is not counted and is not sent out by this call. */
int zg_hip_launch_count(zg_hip_ctx *ctx, uint64_t *launches);

/* ---------------------------------------------------------------------------------------------
 * memory ops (src/device/host_device.zig:919-958)
 * ------------------------------------------------------------------------------------------- */
int zg_hip_memcpy_h2d(zg_hip_ctx *ctx, void *dst, const void *src_host, size_t bytes); /* mem_transfer .HtoD */
/* .DtoH, blocking.  Up to 4096 bytes (NDTensor.get of a scalar, src/ndtensor.zig:524-528) travel through pinned memory of
 * the context: a copy kernel on the stream, the wait for the stream, a host copy. */
int zg_hip_memcpy_d2h(zg_hip_ctx *ctx, void *dst_host, const void *src, size_t bytes);
/* mem_copy / .DtoD.  A waiting float fill of at most 2^20 elements that covers the destination and more, and is clear of
 * the source, leaves in the copy's launch (a gradient zero-filled, then rows copied into it). */
int zg_hip_memcpy_d2d(zg_hip_ctx *ctx, void *dst, const void *src, size_t bytes);
/* mem_fill (src/device/host_device.zig:876-884).  The fill is queued inside the context and launched together with
 * any other waiting fills (up to 16, one kernel) at the start of the next call on this context that is not a float fill
 * or a cache allocation: callers zero gradients tensor by tensor (examples/mnist/src/model.zig:57-62) and one launch per
 * tensor costs more than the fills.  Every later call on the context, zg_hip_sync, zg_hip_stream and a recording's
 * end included, therefore finds the memory filled; only work queued on the raw stream obtained EARLIER from
 * zg_hip_stream, with no call on the context in between, could overtake a waiting fill.  A waiting fill of +0.0 over
 * exactly the dense output of zg_hip_matmul / zg_hip_bmm_acc with beta = 1, the gradient of zg_hip_smce_bwd, the output
 * of zg_hip_scatter_gcn_deg_scaled, a gradient of zg_hip_scatter_gcn_deg_scaled_bwd or the destination of
 * zg_hip_scatter_add is not launched at all: the op writes what it would have added to the zeros (and a source of
 * zg_hip_scatter_add that is exactly a fill still waiting is not read: the fill's value is every contribution, and the
 * fill stays queued for later readers; such a count into a zeroed destination of at most 65536 elements whose offsets
 * were seen before waits with the small elementwise ops below); a waiting fill of any
 * value over exactly the output of a small elementwise op (see below) is taken over likewise, and one inside the output
 * of zg_hip_max_along, which writes every element and reads none, is dropped; one over exactly the gradient of an optimizer
 * step that is itself still waiting (zero_grad() after step()) is stored by the step's update kernel; and a waiting
 * fill that lies inside a cache block handed back with zg_hip_mem_cache_free is dropped (nobody can read it any more). */
int zg_hip_mem_fill(zg_hip_ctx *ctx, float *x, size_t n, float value);
int zg_hip_mem_fill_u8(zg_hip_ctx *ctx, void *x, size_t n, uint8_t value);
int zg_hip_mem_fill_u64(zg_hip_ctx *ctx, uint64_t *x, size_t n, uint64_t value);
int zg_hip_mem_sequence(zg_hip_ctx *ctx, float *x, size_t n, float initial, float step);
int zg_hip_mem_take(zg_hip_ctx *ctx, const float *src, size_t src_len, const uint64_t *idxs, size_t n, float *dst);
/* values are generated on the host (the reference hands mem_random a host std.Random,
 * src/device/host_device.zig:931-945) and copied up; `seed` stands in for that generator */
int zg_hip_mem_random(zg_hip_ctx *ctx, float *x, size_t n, int kind, uint64_t fan, uint64_t seed);

/* ---------------------------------------------------------------------------------------------
 * elementwise binary (src/device/host_device.zig:205-219, :975-1019; opspec.zig:19-57)
 * requires max(xl,yl) % min(xl,yl) == 0 and zl == max(xl,yl); z may alias x or y.  Empty operands: zl == 0 with x and
 * y each empty or one float (not both one float) does nothing, as the host's loops do; an empty operand against a
 * longer one is refused (the host's loop would not end).
 *
 * Small elementwise ops wait.  These four with operands of one length or one operand of a single float, the unary
 * forward and backward ops below, zg_hip_scale and the elementwise loss gradients, on at most 65536 elements, are not
 * launched by their own call: up to eight that follow each other with the same length leave in one launch, in which
 * thread i carries element i through the ops in call order (a caller's chain r + gamma * max_q * (1 - done) is one
 * launch, not four).  An op joins only when every element it shares with a waiting op is shared at the same index (the
 * same n floats, in place or not) and no waiting op writes a one-float operand; otherwise, and on any other call but
 * zg_hip_mem_cache_alloc and zg_hip_mem_cache_free (a caller allocates each result just before its op and frees the
 * temporaries afterwards; the pool keeps a freed block's memory), the waiting ops are launched first.  Waiting float
 * fills that meet none of an op's operands stay waiting.  Same values, bit for bit, as a launch per call.
 * ------------------------------------------------------------------------------------------- */
int zg_hip_add(zg_hip_ctx *ctx, const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
int zg_hip_sub(zg_hip_ctx *ctx, const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
int zg_hip_mul(zg_hip_ctx *ctx, const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
int zg_hip_div(zg_hip_ctx *ctx, const float *x, size_t xl, const float *y, size_t yl, float *z, size_t zl);
/* The same four ops with the one-float operand passed BY VALUE: z[i] = x[i] o s, or s o x[i] when scalar_is_lhs.
 * NDArray.add_scalar & co hand the op a scalar that lives on the caller's stack (src/ndarray.zig:247-257:
 * `.y = &.{s}`), which HostDevice reads in place (src/device/host_device.zig:975-1019) and a kernel cannot.  By value
 * the scalar is a kernel argument: no copy to the device, no wait, the call joins the small elementwise ops that wait
 * (above) and can be recorded into an execution graph.  z may alias x.  A binding calls these when an operand of
 * zg_hip_add & co has length 1 and zg_hip_is_device_ptr says it is not device memory. */
int zg_hip_add_scalar(zg_hip_ctx *ctx, const float *x, size_t n, float s, int scalar_is_lhs, float *z);
int zg_hip_sub_scalar(zg_hip_ctx *ctx, const float *x, size_t n, float s, int scalar_is_lhs, float *z);
int zg_hip_mul_scalar(zg_hip_ctx *ctx, const float *x, size_t n, float s, int scalar_is_lhs, float *z);
int zg_hip_div_scalar(zg_hip_ctx *ctx, const float *x, size_t n, float s, int scalar_is_lhs, float *z);

/* ---------------------------------------------------------------------------------------------
 * linear algebra (src/device/host_device.zig:224-346)
 * On no elements (n == 0) dot, sum and nrm2 write 0, as the BLAS calls behind the reference do; scale, axpy and
 * clip_nrm2 do nothing.  A product with k == 0 leaves C = beta C and does not look at A and B (they may be null);
 * with m == 0 or n == 0 there is nothing to do.
 * ------------------------------------------------------------------------------------------- */
int zg_hip_dot(zg_hip_ctx *ctx, const float *x, const float *y, size_t n, float *z);
int zg_hip_matvec(zg_hip_ctx *ctx, const float *A, const float *x, float *y, size_t m, size_t n, int trans_a,
                  float alpha, float beta);
/* Timing of the products, for benchmarks (no counterpart in the reference).  While on, the launches of every product
 * (zg_hip_matmul, zg_hip_bmm_acc, the fused Linear entry points: the product's kernel with whatever its epilogue
 * carries, plus the reduction or the strips when the product is cut) are bracketed by a pair of events on the
 * context's stream at the moment they are queued.  zg_hip_gemm_timing(ctx, 1) clears the count and starts,
 * zg_hip_gemm_timing(ctx, 0) stops; zg_hip_gemm_timing_read waits for the stream and returns the summed time between
 * the pairs and the number of products.  Nothing is bracketed while a graph is being recorded. */
int zg_hip_gemm_timing(zg_hip_ctx *ctx, int enable);
int zg_hip_gemm_timing_read(zg_hip_ctx *ctx, double *total_ms, uint64_t *products);

/* How a product of this shape would be launched by the staged kernels (no counterpart in the reference; for tests
 * and for reading profiles).  out[0] kind: 0 one launch, 1 k cut over several workgroups per tile and the partial
 * tiles added in a fixed order by a second kernel, 2 C cut into a block of whole 256 x 128 tiles plus strips that are
 * launched as products of their own, 3 the tail in pieces: a whole number of rounds of tiles computed whole and, in the
 * same launch, the tiles that would start one more (mostly empty) round cut along k into pieces, which a second kernel
 * adds tile by tile in a fixed order; out[1] tile: 0 = 256 x 128, 1 = 128 x 128, 2 = 64 x 64; out[2], out[3] number of k
 * ranges and k-tiles (of 16) per range; out[4], out[5] tile rows and columns of the main block (kind 2), or out[4] the
 * number of tiles computed whole (kind 3); out[6] the planner's estimate in microseconds.  Products served by the
 * unstaged small-product kernels, or by the one-launch kernel for deep products of k-contiguous operands on a few
 * blocks (384 <= k <= 2048, at most a CU's worth of 16 x 16 blocks of C), are not planned this way.
 * ctx may be null (256 compute units are assumed); nothing is launched. */
int zg_hip_gemm_plan(zg_hip_ctx *ctx, size_t m, size_t n, size_t k, size_t batches, int64_t *out);

/* row-major C = alpha*op(A)*op(B) + beta*C; C is not read when beta == 0.
 * Products that wait.  Two kinds of single (unbatched) product with a dense C (ldc == n) are not launched by the call
 * that asks for them but by the NEXT call on the context, whatever it is:
 *   - a layer's forward product, C = A B^T with beta == 0 (x.bmm_acc(W, trans_b), examples/mnist/src/model.zig:107):
 *     if the next call is zg_hip_add of a row of n values onto C in place (bias.add_(y), :108) the row is added in the
 *     product's epilogue and the product waits one more call; if the next call is zg_hip_relu_fwd of C in place
 *     (:38-46) the ReLU is applied in the epilogue too and the product is launched;
 *   - an input-gradient product, C += A B with beta == 1 onto a C whose zero fill is still waiting (ensure_grad(0) then
 *     BmmAccBwd, src/ndtensor.zig:221-228, :1107-1109): one following product that touches none of its operands (the
 *     weight gradient, :1126-1128) is launched ahead of it, or, when both products are small enough for the unstaged
 *     kernel and read the same dense A, waits with it; if the next call is zg_hip_relu_inplace_bwd on C
 *     (src/nn/nn.zig:44-50) the mask is applied in the epilogue and the product is launched, in one launch with the
 *     weight-gradient product and the layer's bias gradient (see zg_hip_unbroadcast) when those wait too.
 * Any other call (a read, a fill, a free, an allocation, another op, zg_hip_sync, the end of a recording) launches the
 * waiting product first, unchanged.  The values are those of the separate calls, bit for bit: the epilogue does the
 * same IEEE operations in the same order.  An argument error is reported by the call that asks for the product. */
int zg_hip_matmul(zg_hip_ctx *ctx, const float *A, const float *B, float *C, size_t m, size_t n, size_t k,
                  int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta);
/* shapes are host arrays of 3: {batches, rows, cols} of the logical (post-transpose) operands */
int zg_hip_bmm_acc(zg_hip_ctx *ctx, const float *A, const uint64_t *A_shape, const float *B,
                   const uint64_t *B_shape, float *C, const uint64_t *C_shape, int trans_a, int trans_b, size_t lda,
                   size_t ldb, size_t ldc, float alpha, float beta);
/* Fused Linear layer (the epilogue fusion the CUDA backend leaves open): the reference issues bmm_acc(trans_b) +
 * bias.add_ (examples/mnist/src/model.zig:104-110) + relu_ (:38-46) as three device ops, and in backward
 * relu_inplace_bwd (src/device/host_device.zig:543-547) + the dA product of BmmAccBwd (src/ndtensor.zig:1092-1136).
 * These run the same arithmetic in one launch: y[batch, fan_out] = act(x[batch, fan_in] . w[fan_out, fan_in]^T +
 * bias), bias may be null, relu != 0 applies max(0, .). */
int zg_hip_linear_fwd(zg_hip_ctx *ctx, const float *x, const float *w, const float *bias, float *y, size_t batch,
                      size_t fan_in, size_t fan_out, int relu);
/* gx[batch, fan_in] = (accumulate ? gx : 0) + gy[batch, fan_out] . w, then gx = 0 where act_in <= 0; act_in is the
 * ReLU output that fed the layer (null: no mask).  With accumulate == 0 gx is not read and needs no zero fill. */
int zg_hip_linear_bwd_input(zg_hip_ctx *ctx, const float *gy, const float *w, const float *act_in, float *gx,
                            size_t batch, size_t fan_in, size_t fan_out, int accumulate);
/* The whole backward of the layer for a final output gradient gy[batch, fan_out] (the two products of BmmAccBwd,
 * src/ndtensor.zig:1092-1136, the bias's unbroadcast, src/device/host_device.zig:709-780, and the ReLU backward of the
 * layer before): gw[fan_out, fan_in] += gy^T . x;  gb[fan_out] += column sums of gy (null: none);
 * gx[batch, fan_in] = gy . w, zero where act_in <= 0 (gx null: no input gradient; act_in null: no mask).
 * One launch for a small layer, the separate ops otherwise; the same values either way. */
int zg_hip_linear_bwd(zg_hip_ctx *ctx, const float *gy, const float *x, const float *w, const float *act_in, float *gw,
                      float *gb, float *gx, size_t batch, size_t fan_in, size_t fan_out);
int zg_hip_outer(zg_hip_ctx *ctx, const float *x, size_t xl, const float *y, size_t yl, float *A, float alpha);
/* B = A^T + alpha*B; B is not read when alpha == 0 (the reference hands in uninitialised B then:
 * src/ndarray.zig:794-802) */
int zg_hip_transpose(zg_hip_ctx *ctx, const float *A, float *B, size_t m, size_t n, float alpha);
/* alpha is read through the pointer: a host pointer when alpha_on_device == 0 (SGD, src/nn/optim.zig:114-118),
 * a device pointer otherwise (dot backward, src/ndtensor.zig:1146-1150) */
int zg_hip_axpy(zg_hip_ctx *ctx, const float *x, float *y, size_t n, const float *alpha, int alpha_on_device);
int zg_hip_sum(zg_hip_ctx *ctx, const float *x, size_t n, float *y); /* sum of |x|, as cblas_sasum */
int zg_hip_scale(zg_hip_ctx *ctx, float *x, size_t n, float alpha);
int zg_hip_nrm2(zg_hip_ctx *ctx, const float *x, size_t n, float *y);
int zg_hip_clip_nrm2(zg_hip_ctx *ctx, float *x, size_t n, float max_norm, float delta);

/* ---------------------------------------------------------------------------------------------
 * unary forward/backward (src/device/host_device.zig:353-598); y may alias x in the *_fwd ops
 * ------------------------------------------------------------------------------------------- */
int zg_hip_pow_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n, float e);
int zg_hip_pow_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, const float *y_g, size_t n, float e, float eps);
int zg_hip_sqrt_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n);
int zg_hip_sqrt_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, const float *y_g, size_t n, float eps);
int zg_hip_rsqrt_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n, float eps);
int zg_hip_rsqrt_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, const float *y_g, size_t n, float eps);
int zg_hip_exp_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n);
int zg_hip_exp_bwd(zg_hip_ctx *ctx, float *x_g, const float *y, const float *y_g, size_t n);
int zg_hip_relu_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n);
int zg_hip_relu_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, const float *y_g, size_t n);
int zg_hip_relu_inplace_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, size_t n);
int zg_hip_tanh_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n);
int zg_hip_tanh_bwd(zg_hip_ctx *ctx, float *x_g, const float *y, const float *y_g, size_t n);
int zg_hip_tanh_inplace_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, size_t n);
int zg_hip_sigm_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n);
int zg_hip_sigm_bwd(zg_hip_ctx *ctx, float *x_g, const float *y, const float *y_g, size_t n);
int zg_hip_sigm_inplace_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, size_t n);
int zg_hip_clamp_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t n, float lo, float hi);
int zg_hip_clamp_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, const float *y_g, size_t n, float lo, float hi);
/* x[isamax(x)]: the element of largest |x|, the first on ties (src/device/host_device.zig:573-580).  A NaN counts as
 * larger than anything and the first one wins, as mkl_rt, the BLAS the reference names, documents for i?amax. */
int zg_hip_max_fwd(zg_hip_ctx *ctx, const float *x, size_t n, float *y);
int zg_hip_max_bwd(zg_hip_ctx *ctx, const float *x, float *x_g, size_t n, const float *y, const float *y_g);

/* ---------------------------------------------------------------------------------------------
 * reductions (src/device/host_device.zig:709-874, src/device/reduce.zig)
 * ------------------------------------------------------------------------------------------- */
int zg_hip_sum_along(zg_hip_ctx *ctx, const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len,
                     size_t dim, float alpha, float beta);
int zg_hip_max_along(zg_hip_ctx *ctx, const float *x, const uint64_t *x_shape, size_t x_rank, float *y, size_t y_len,
                     size_t dim);
/* no reference op: first index of the maximum along dim (std.mem.indexOfMax per slice,
 * examples/mnist/src/main-simple.zig:124-125) */
int zg_hip_argmax_along(zg_hip_ctx *ctx, const float *x, const uint64_t *x_shape, size_t x_rank, uint64_t *y,
                        size_t y_len, size_t dim);
/* scratch sizing rule of NDArray.unbroadcast_ (src/ndarray.zig:701-719), in floats */
size_t zg_hip_unbroadcast_scratch_len(const uint64_t *x_shape, size_t x_rank, const uint64_t *y_shape,
                                      size_t y_rank);
/* unbroadcast (src/device/host_device.zig:709-780).  The form a Linear layer's bias gradient takes (y += sums over the
 * leading dimensions of x, alpha = beta = 1, at most 65536 elements of x) waits inside the context like a product
 * (see zg_hip_matmul): the layer's input-gradient and weight-gradient products follow it (src/ndtensor.zig:780-796,
 * 1092-1136) and, when they are small too, the three leave in one launch.  Any other call sends it out first. */
int zg_hip_unbroadcast(zg_hip_ctx *ctx, const float *x, const uint64_t *x_shape, size_t x_rank, float *y,
                       const uint64_t *y_shape, size_t y_rank, float *scratch, size_t scratch_len, float alpha,
                       float beta);
int zg_hip_broadcast(zg_hip_ctx *ctx, const float *x, size_t xl, float *y, size_t yl, float alpha, float beta);

/* ---------------------------------------------------------------------------------------------
 * indexing (src/device/host_device.zig:1039-1087, :1356-1403; src/ndarray.zig:593-633;
 * src/ndtensor.zig:1437-1513).  All accumulating ops add contributions to one destination element
 * in the order of the input index array, so results do not depend on scheduling.
 * ------------------------------------------------------------------------------------------- */
/* offsets of NDArray.gather computed on the device; shapes are host arrays of `rank`; `indices`, `offsets`
 * device-readable.  Out-of-range indices are reported through *status (host, optional, blocking when given):
 * 0 ok, 1 InvalidIndexShape, 2 IndexOutOfBounds */
int zg_hip_gather_offsets(zg_hip_ctx *ctx, const uint64_t *src_shape, const uint64_t *idx_shape, size_t rank,
                          const uint64_t *indices, size_t dim, uint64_t *offsets, int *status);
/* the whole of NDArray.gather (src/ndarray.zig:593-633) in one launch: the offsets as above (kept: the backward
 * scatters through them) and dst[i] = src[offsets[i]] */
int zg_hip_gather(zg_hip_ctx *ctx, const float *src, const uint64_t *src_shape, const uint64_t *idx_shape, size_t rank,
                  const uint64_t *indices, size_t dim, uint64_t *offsets, float *dst, int *status);
int zg_hip_scatter_add(zg_hip_ctx *ctx, const float *src, const uint64_t *offsets, size_t n, float *dst,
                       size_t dst_len);
int zg_hip_index_select_fwd(zg_hip_ctx *ctx, const float *src, size_t src_len, const uint64_t *indices, size_t n_idx,
                            size_t stride, float *dst);
int zg_hip_index_select_bwd(zg_hip_ctx *ctx, const float *y_grad, const uint64_t *indices, size_t n_idx,
                            size_t stride, float *x_grad, size_t x_len);
/* n_nodes = number of rows of dst/h (the reference derives it from the slices' lengths).
 * Like the products (see zg_hip_matmul), the aggregation works with the calls around it: a waiting zero fill of exactly
 * dst (or of exactly grad_h / grad_deg in the backward) is taken over and the sums are written instead of added to
 * zeros; and the forward's kernel is launched by the NEXT call on the context: zg_hip_add of a row of `stride` values
 * onto dst in place (y._add(bias), examples/gcn/src/model.zig:110) and zg_hip_relu_fwd of dst in place (:36) become the
 * kernel's tail, any other call launches it first, unchanged.  Same values, bit for bit.  The backward launches the
 * feature gradient at once and holds the two launches of the degree gradient for the next call: the reference's layer
 * computes grad_deg into a buffer it gives back unread (the degrees are data of the graph, src/ndtensor.zig:1009), and
 * a zg_hip_mem_cache_free of the block that holds all of grad_deg while they wait drops them; any other call launches
 * them first. */
int zg_hip_scatter_gcn_deg_scaled(zg_hip_ctx *ctx, float *dst, const float *h, const float *deg,
                                  const uint64_t *src_indices, const uint64_t *tgt_indices, size_t stride,
                                  size_t n_edge, size_t n_nodes);
int zg_hip_scatter_gcn_deg_scaled_bwd(zg_hip_ctx *ctx, const float *grad_output, const float *h, const float *deg,
                                      const uint64_t *src_indices, const uint64_t *tgt_indices, float *grad_h,
                                      float *grad_deg, size_t stride, size_t n_edge, size_t n_nodes);

/* CSR forms (src/device/host_device.zig:1325-1353).  scatter_add_csr: dst[j] += src[i] for j in [row_ptr[i],
 * row_ptr[i + 1]), row_ptr non-decreasing with n_segments + 1 entries.  segment_sum_csr: dst[i] = the sum of
 * src[row_offsets[i] .. row_offsets[i + 1]) (written, not accumulated). */
int zg_hip_scatter_add_csr(zg_hip_ctx *ctx, const float *src, const uint64_t *row_ptr, size_t n_segments, float *dst,
                           size_t dst_len);
int zg_hip_segment_sum_csr(zg_hip_ctx *ctx, const float *src, size_t src_len, const uint64_t *row_offsets,
                           size_t n_segments, float *dst);

/* Kept plans.  When the index arrays of zg_hip_scatter_add, zg_hip_index_select_bwd, zg_hip_scatter_gcn_deg_scaled or
 * zg_hip_scatter_gcn_deg_scaled_bwd lie in zg_hip_host_alloc memory (where the reference's callers write them with
 * host loops, examples/gcn/src/model.zig:204-205), the context keeps the destination ordering it computed, a host
 * copy of the arrays' contents and a device copy for the kernels.  A later call whose arrays hold the same values
 * (compared on the host, byte for byte, when the call is made) runs the same apply kernels on the kept ordering
 * instead of computing it again: same values, five to six launches fewer per ordering.  At most 16 orderings are
 * kept (least recently used goes first), for arrays of up to 65536 entries (longer ones cost more to compare than
 * to analyse).  A recorded graph keeps the orderings it used, and zg_hip_graph_run returns
 * ZG_HIP_EINVAL when one of those arrays no longer holds what it held at the recording.  Shorter index arrays in
 * device memory are analysed on every call.
 * Arrays of 262144 to 2^24 entries, in device memory or in zg_hip_host_alloc memory, are kept differently: under the
 * ADDRESSES of the arrays, with 32-bit copies of their contents beside the ordering, and every call starts with a
 * kernel that compares the arrays with the copies ON THE GPU.  Unchanged arrays skip the rebuild (the kernels of the
 * build are launched and return at once), changed ones are ordered again in place; either way the call works on the
 * arrays as they are when its kernels run, whoever rewrote them, so a recorded graph stays valid when the arrays are
 * rewritten between replays.  An array that turns out to change on most calls is dropped from the cache and analysed
 * on every call like a short one (the address is tried again 1024 calls later).  These entries count in `hits` when
 * the address was found, whether or not the contents had changed.
 * `hits` / `builds` count calls served from a kept ordering / orderings computed and kept; no counterpart in the
 * reference. */
int zg_hip_plan_cache_stats(zg_hip_ctx *ctx, uint64_t *hits, uint64_t *builds);

/* Edge plans.  The three ops above sort the edge list by destination on every call, because the reference hands
 * them bare index slices (examples/gcn/src/model.zig:116-224 builds them per forward).  For an edge list that does
 * not change between calls (the dataset's graph, examples/gcn/src/dataset.zig:110-127) the analysis can be done
 * once: a plan holds both orderings (by target, by source) and device copies of the two index arrays; the planned
 * ops launch the same kernels on it and return the same values as zg_hip_scatter_add (offsets = targets),
 * zg_hip_scatter_gcn_deg_scaled and zg_hip_scatter_gcn_deg_scaled_bwd.  The index arrays may be device or
 * zg_hip_host_alloc memory and may be reused after create returns.  Create and free are refused while recording. */
typedef struct zg_hip_edge_plan zg_hip_edge_plan;
int zg_hip_edge_plan_create(zg_hip_ctx *ctx, const uint64_t *src_indices, const uint64_t *tgt_indices, size_t n_edge,
                            size_t n_nodes, zg_hip_edge_plan **out);
int zg_hip_edge_plan_free(zg_hip_ctx *ctx, zg_hip_edge_plan *plan);
/* accumulate != 0: add into the outputs, as the unplanned ops do; accumulate == 0: the outputs are written (every
 * element, zeros where no edge arrives), so the caller needs no zero fill.  grad_deg may be null when the degrees need
 * no gradient (they are data of the graph; the reference's chain stops there too, src/ndtensor.zig:1009). */
int zg_hip_scatter_add_planned(zg_hip_ctx *ctx, const float *src, const zg_hip_edge_plan *plan, float *dst,
                               int accumulate);
/* bias (null: none) and relu (0: none) are the tail of a graph-convolution layer, applied to every row after its
 * edges: dst[t, :] = max(dst[t, :] + bias, 0), the `y._add(self.bias)` of examples/gcn/src/model.zig:110 and the `relu_` of :36 */
int zg_hip_scatter_gcn_deg_scaled_planned(zg_hip_ctx *ctx, float *dst, const float *h, const float *deg,
                                          const zg_hip_edge_plan *plan, const float *bias, int relu, size_t stride,
                                          int accumulate);
int zg_hip_scatter_gcn_deg_scaled_bwd_planned(zg_hip_ctx *ctx, const float *grad_output, const float *h,
                                              const float *deg, const zg_hip_edge_plan *plan, float *grad_h,
                                              float *grad_deg, size_t stride, int accumulate);

/* ---------------------------------------------------------------------------------------------
 * losses: the host loops of src/nn/loss.zig:94-305 as device ops (new op names; the reference
 * dereferences .raw on the host and has no opspec for them)
 * ------------------------------------------------------------------------------------------- */
int zg_hip_smce_fwd(zg_hip_ctx *ctx, const float *logits, const float *target, float *probs, float *loss,
                    size_t rows, size_t cols);
int zg_hip_smce_bwd(zg_hip_ctx *ctx, const float *probs, const float *target, float *grad, size_t rows, size_t cols);
/* (An empty matrix: zg_hip_smce_bwd, zg_hip_softmax_fwd and zg_hip_softmax_bwd do nothing, like the host's loops over
 * no rows; the forward losses, which divide by the number of rows or elements, refuse it with ZG_HIP_EINVAL.) */
/* smce_fwd followed by the loss's backward with upstream gradient 1 (loss.backward() on the scalar loss,
 * src/nn/loss.zig:150-159): grad (+)= (probs - target)/rows.  Same values as the two calls; a batch of at most
 * 256 rows x 32 columns (64 x 256, 16 x 4096) takes one launch.  accumulate == 0: grad is written, not read. */
int zg_hip_smce_fwd_bwd(zg_hip_ctx *ctx, const float *logits, const float *target, float *probs, float *loss,
                        float *grad, size_t rows, size_t cols, int accumulate);
/* integer-label form: one pass over the logits forward (online softmax), lse[rows] kept for backward */
int zg_hip_smce_label_fwd(zg_hip_ctx *ctx, const float *logits, const uint64_t *labels, float *lse, float *loss,
                          size_t rows, size_t cols);
/* No counterpart in the reference: zg_hip_smce_label_fwd for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It calls no allocator of any kind: the per-row loss
 * terms and the partial sums live in a fixed array in the library's device image (1 MiB + 8 KiB per GPU, held until
 * the process ends) instead of the context's grow-only workspace.  At most 262144 rows; more is rejected with
 * ZG_HIP_EINVAL before any launch.  Same kernels and the same values as zg_hip_smce_label_fwd.  All calls on one GPU
 * share the array: calls that overlap on one GPU (two contexts, two streams) race; calls on one context are ordered
 * by its stream.  Work that earlier calls left waiting in the context (see zg_hip_mem_fill, zg_hip_matmul) is launched
 * first, as by every call; it needs no memory either: what a waiting product uses was reserved by the call that
 * queued it. */
int zg_hip_smce_label_fwd_noalloc(zg_hip_ctx *ctx, const float *logits, const uint64_t *labels, float *lse,
                                  float *loss, size_t rows, size_t cols);
/* accumulate != 0: grad += (p - onehot)/rows (the reference's `+=`, src/nn/loss.zig:157);
 * accumulate == 0: grad is overwritten (valid when the caller knows grad is a fresh zero buffer) */
int zg_hip_smce_label_bwd(zg_hip_ctx *ctx, const float *logits, const uint64_t *labels, const float *lse,
                          float *grad, size_t rows, size_t cols, int accumulate);
int zg_hip_softmax_fwd(zg_hip_ctx *ctx, const float *x, float *y, size_t rows, size_t cols);
int zg_hip_softmax_bwd(zg_hip_ctx *ctx, const float *y, const float *y_g, float *x_g, size_t rows, size_t cols);
int zg_hip_smooth_l1_fwd(zg_hip_ctx *ctx, const float *pred, const float *target, size_t n, float beta, float *loss);
int zg_hip_smooth_l1_bwd(zg_hip_ctx *ctx, const float *pred, const float *target, float *grad, size_t n, float beta);
/* smooth_l1_fwd followed by the backward of the scalar loss (upstream gradient 1): grad (+)= d loss / d pred; one
 * launch for up to 4096 elements.  accumulate == 0: grad is written, not read. */
int zg_hip_smooth_l1_fwd_bwd(zg_hip_ctx *ctx, const float *pred, const float *target, float *grad, size_t n, float beta,
                             float *loss, int accumulate);
int zg_hip_mse_fwd(zg_hip_ctx *ctx, const float *pred, const float *target, size_t n, float *loss);
int zg_hip_mse_bwd(zg_hip_ctx *ctx, const float *pred, const float *target, float *grad, size_t n);

/* ---------------------------------------------------------------------------------------------
 * optimizers: src/nn/optim.zig:100-122 (SGD.update) and :177-234 (Adam.update) as one op per
 * parameter tensor.  `clip` != 0 applies the reference's per-tensor clip_nrm2 to grad first
 * (grad is modified in place, as in the reference).
 * A step is not launched by its own call: it waits while the calls that follow are more steps with the same settings
 * on tensors that do not overlap the waiting ones (an optimizer walks its parameter list), and the run then leaves
 * through the parameter-list kernels below (the clip factors of all tensors in two launches, then the updates); a
 * zero fill of exactly a waiting step's gradient (zero_grad() after step()) is stored by its update kernel; any other
 * call on the context launches what is waiting first.  Same values, bit for bit, as a launch per call.
 * ------------------------------------------------------------------------------------------- */
int zg_hip_sgd_step(zg_hip_ctx *ctx, float *param, float *grad, size_t n, float lr, int clip, float max_norm,
                    float delta);
/* t: the per-tensor-update counter AFTER the reference's `self.t += 1` (src/nn/optim.zig:189) */
int zg_hip_adam_step(zg_hip_ctx *ctx, float *param, float *grad, float *m, float *v, size_t n, uint64_t t, float lr,
                     float beta1, float beta2, float epsilon, int clip, float max_norm, float delta);

/* lr_t of Adam for counter value t, computed in fp32 exactly as zg_hip_adam_step does on the host
 * (src/nn/optim.zig:190-191). */
int zg_hip_adam_lr_t(float lr, float beta1, float beta2, uint64_t t, float *lr_t);
/* zg_hip_adam_step with lr_t read from memory when the kernel executes.  `lr_t` points to device memory or to
 * zg_hip_host_alloc memory; the host may rewrite it between replays of a captured graph (not while a replay that
 * reads it is still running).  This is what lets one captured step serve every later step. */
int zg_hip_adam_step_at(zg_hip_ctx *ctx, float *param, float *grad, float *m, float *v, size_t n, const float *lr_t,
                        float beta1, float beta2, float epsilon, int clip, float max_norm, float delta);

/* The optimizer step over a whole parameter list, as Optimizer.step() walks it (src/nn/optim.zig:100-122, :177-234):
 * tensors of up to 131072 elements share launches (one workgroup per tensor, 16 tensors per launch), larger ones
 * take the per-tensor kernels; values are those of the per-tensor calls.  The lists are host arrays of n_tensors
 * entries.  zero_grads != 0 also leaves every gradient zero: optim.step() followed by model.zero_grad()
 * (examples/mnist/src/main-simple.zig:70-71, examples/mnist/src/model.zig:57-62) without the fills.
 * Adam: lr_t[i] is tensor i's step size (zg_hip_adam_lr_t with that tensor's counter value); with
 * lr_t_in_memory != 0 it is an array in device or zg_hip_host_alloc memory that the kernels read when they run
 * (see zg_hip_adam_step_at), otherwise a host array read during the call. */
int zg_hip_sgd_step_multi(zg_hip_ctx *ctx, size_t n_tensors, float *const *params, float *const *grads,
                          const size_t *lens, float lr, int clip, float max_norm, float delta, int zero_grads);
int zg_hip_adam_step_multi(zg_hip_ctx *ctx, size_t n_tensors, float *const *params, float *const *grads,
                           float *const *ms, float *const *vs, const size_t *lens, const float *lr_t,
                           int lr_t_in_memory, float beta1, float beta2, float epsilon, int clip, float max_norm,
                           float delta, int zero_grads);

/* ---------------------------------------------------------------------------------------------
 * input staging: the step before the hot path.  The reference uploads every batch with a blocking
 * mem_transfer(.HtoD) (src/device/device_reference.zig:101-105, as used by NDTensor.from_slice in
 * examples/mnist/src/dataset.zig:51-52).  These three calls let a training loop upload batch k+1 from pinned
 * host memory on a second stream (default priority) while the kernels of batch k run:
 *   staged_h2d         asynchronous copy on the copy stream; `src_host` must come from zg_hip_host_alloc and
 *                      must not be rewritten until zg_hip_staging_wait returned (or a later sync)
 *   staging_after_compute   copies issued from now on wait for all work issued to the compute stream so far
 *                      (call it before overwriting a device buffer that earlier ops still read)
 *   compute_after_staging   ops issued from now on wait for every copy issued so far
 *   staging_wait       blocks the host until every staged copy has finished (the pinned source may be reused)
 * ------------------------------------------------------------------------------------------- */
int zg_hip_staged_h2d(zg_hip_ctx *ctx, void *dst, const void *src_host, size_t bytes);
int zg_hip_staging_after_compute(zg_hip_ctx *ctx);
int zg_hip_compute_after_staging(zg_hip_ctx *ctx);
int zg_hip_staging_wait(zg_hip_ctx *ctx);

/* ---------------------------------------------------------------------------------------------
 * execution graphs: the ExecutionGraph of the reference's second device, src/device/cuda_device.zig:558-611
 * (open = begin stream capture, save = end capture and instantiate, run = launch, free).
 * Between open and save every op call is recorded instead of executed.  Calls that synchronise, allocate
 * from the driver or copy to/from host memory return ZG_HIP_ECAPTURE (run one eager step first so the
 * caching allocator and the internal workspace have their final size).  zg_hip_mem_cache_free inside a
 * capture parks the block with the graph instead of returning it to the pool, so the addresses recorded in
 * the graph stay private to it until zg_hip_graph_free.  Launch-bound steps (tens of 2-microsecond kernels)
 * replay without per-op host work.
 * ------------------------------------------------------------------------------------------- */
int zg_hip_graph_open(zg_hip_ctx *ctx);
int zg_hip_graph_save(zg_hip_ctx *ctx, zg_hip_graph **out);
int zg_hip_graph_run(zg_hip_ctx *ctx, zg_hip_graph *graph);
int zg_hip_graph_free(zg_hip_ctx *ctx, zg_hip_graph *graph);

#ifdef __cplusplus
}
#endif
#endif
