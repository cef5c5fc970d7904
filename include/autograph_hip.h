/*
 * autograph_hip.h - C ABI of the MI355X (gfx950) device backend for autograph's
 * dense-contraction hot path.
 *
 * The reference has no FFI layer of its own: its device backend is the krnl crate,
 * reached from the `#[cfg(feature = "device")]` branch of every op.  Each entry point
 * below replaces one of those device branches and takes exactly the plain values that
 * branch extracts before dispatching a kernel (buffer, element offset, dims, signed
 * element strides, option integers).  Citations are file:line in the reference tree.
 *
 * Conventions
 *   - Every function returns 0 on success, a negative AGH_E* code for argument errors
 *     (detected before anything is launched, like the reference's `bail!`s) and a
 *     positive hipError_t value when HIP fails.  agh_last_error_string() describes the
 *     last failure on the calling thread.  Nothing throws or aborts across the ABI.
 *   - All device work is enqueued on ONE in-order stream owned by the library
 *     (krnl's per-device queue).  Launch entry points return without waiting;
 *     agh_memcpy_d2h and agh_sync wait.
 *   - Pointers named x/y/a/b/c/dx/dy are DEVICE pointers from agh_malloc.  Offsets and
 *     strides are in ELEMENTS (not bytes); strides may be negative or zero.
 *   - bf16 data are raw 16-bit patterns (uint16_t).
 *   - Outputs are caller-allocated and fully overwritten unless stated otherwise.
 *     Kernels keep no pointer after they finish; the caller frees.
 *   - Entry points may be called from any thread; calls are serialised internally.
 */
#ifndef AUTOGRAPH_HIP_H
#define AUTOGRAPH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AGH_OK 0
#define AGH_EINVAL (-1)   /* bad shape / stride / option value */
#define AGH_ENOINIT (-2)  /* agh_init has not succeeded */
#define AGH_ENULL (-3)    /* null pointer where data is required */
#define AGH_ERANGE (-4)   /* size does not fit the kernel's index range */

/* Epilogue activation of the fused Dense entry points. */
#define AGH_ACT_NONE 0
#define AGH_ACT_RELU 1

/* ------------------------------------------------------------------ runtime ---- */

/* Device::builder().index(i).build()  (tests/integration_tests.rs:27-30).  Selects the
 * GPU, creates the stream.  Idempotent for the same index. */
int agh_init(int device_index);
/* Frees the library's own workspace and stream.  Buffers from agh_malloc stay valid
 * until freed by the caller. */
int agh_shutdown(void);
const char *agh_last_error_string(void);
/* Name, compute-unit count and memory size of the active device (krnl DeviceInfo). */
int agh_device_info(char *name, size_t name_len, int *compute_units, size_t *total_mem_bytes);

/* Buffer allocation: Tensor::uninit (src/tensor.rs:1377-1389), one per op output in the reference
 * (src/tensor/linalg.rs:412-419, src/tensor/ops.rs:855-878).  Served by a caching allocator: agh_free
 * does not wait and does not return the block to the driver, it keeps it (by size class: at most 25 %
 * larger than asked) for the next agh_malloc.  Reuse is safe because all work is issued in order: a
 * block freed while kernels that use it are still queued is only touched by work launched after them
 * (a block last used inside an unjoined branch makes the main stream wait for the branch stream when
 * it is handed out again).  Cached blocks go back to the driver at agh_shutdown, at
 * agh_cache_release, when the driver runs out of memory, or when the cache exceeds its limit
 * (64 GiB, or AGH_CACHE_LIMIT_MB at agh_init). */
int agh_malloc(void **ptr, size_t bytes);
int agh_free(void *ptr);
/* Waits for all queued work and returns every cached block to the driver, and the library's own
 * workspace too unless a graph from agh_graph_end is still alive.  The reference has no counterpart
 * (krnl frees a buffer when it is dropped). */
int agh_cache_release(void);
/* Bytes and blocks held for reuse, blocks currently handed out (any pointer may be null). */
int agh_cache_stats(size_t *cached_bytes, size_t *cached_blocks, size_t *live_blocks);
/* Bytes of the library's own workspace (split-K partials, reordered filter banks; both streams' blocks) and the number of
 * outgrown workspace blocks kept alive for live graphs.  None of this memory is the caller's; the figures let a caller
 * that must not allocate verify that a call sequence did not grow it. */
int agh_workspace_stats(size_t *workspace_bytes, size_t *retired_blocks);
/* into_device / to_device (src/tensor.rs:1775-1833): host -> device, enqueued on the current stream
 * (the branch stream inside a branch, like every launch).
 * The host range must stay valid until the next agh_sync unless it is pageable memory. */
int agh_memcpy_h2d(void *dst, const void *src, size_t bytes);
/* into_array / into_vec (src/tensor.rs:1923-1934): blocks until the bytes are on the host.  Issued
 * on the current stream; outside a branch it first waits for branches that have not been joined, so
 * data produced there are complete. */
int agh_memcpy_d2h(void *dst, const void *src, size_t bytes);
int agh_memcpy_d2d(void *dst, const void *src, size_t bytes);
/* Tensor::zeros / fill for byte patterns (src/tensor.rs:1394-1416). */
int agh_memset(void *dst, int byte_value, size_t bytes);
/* Same copy without the wait (for use inside a captured graph, or when the caller syncs). */
int agh_memcpy_d2h_async(void *dst, const void *src, size_t bytes);
/* Pinned host memory for transfers that must not stage through a bounce buffer. */
int agh_host_alloc(void **ptr, size_t bytes);
int agh_host_free(void *ptr);
/* device.wait() (src/tensor/linalg.rs:549). */
int agh_sync(void);
/* The hipStream_t all work is enqueued on (for callers that record their own events). */
void *agh_stream(void);

/* Launch-bound sequences (a LeNet5 forward pass is a dozen tiny kernels) can be recorded once
 * and replayed as one hipGraph: between agh_graph_begin and agh_graph_end every launch entry
 * point and agh_memcpy_d2h_async is captured instead of executed.  No entry point that
 * allocates or waits (agh_malloc, agh_sync, agh_memcpy_d2h, a first split-K GEMM that has to grow the
 * workspace) may be called while capturing (they return an error): run the sequence once eagerly first.
 * agh_free is allowed while capturing (a host-side temporary may be dropped at any moment): the block is
 * set aside and goes back to the cache in agh_graph_end; a block that recorded work touches must of course
 * stay allocated for as long as the graph is replayed.  The library's workspace (split-K partials,
 * reordered filter banks) is named by the captured nodes: while any graph from agh_graph_end is alive, a
 * workspace block that has to grow is retired, not freed, so replays stay valid after larger eager calls;
 * retired blocks are released when the last graph is destroyed or at agh_shutdown.  agh_graph_launch
 * first joins any branch that is still open on the second stream (its work may use the workspace a
 * captured arm names).
 * The reference has no counterpart (krnl dispatches kernel by kernel). */
int agh_graph_begin(void);
int agh_graph_end(void **graph_exec);
int agh_graph_launch(void *graph_exec);
int agh_graph_destroy(void *graph_exec);

/* Independent work.  Everything issued between agh_branch_begin and agh_branch_end goes to a second
 * in-order stream: it starts after all work issued before the begin, and runs concurrently with what
 * the caller issues after the end.  agh_branch_join makes all later work wait for every branch issued
 * so far; agh_sync waits for both streams (inside a branch too: work issued after it still goes to the
 * second stream and is still joined).  Several begin/end pairs may precede one join (their work
 * runs in order among itself).  The CALLER guarantees that a branch and the work issued between its
 * end and the join touch disjoint outputs (e.g. the weight gradient and the input gradient of one
 * layer, autograd.rs:607-627: two `dot` calls on the same `output_grad`).  Works under graph capture:
 * branches become parallel arms of the graph, and a capture must be joined before agh_graph_end.
 * The branch state belongs to the library, not to the calling thread: while one thread is between begin and
 * end, entry points called from any thread go to the second stream.
 * The reference has no counterpart (krnl has one queue per device). */
int agh_branch_begin(void);
int agh_branch_end(void);
int agh_branch_join(void);

/* Timing helpers: hipEvent pairs recorded on the library's stream. */
int agh_event_create(void **event);
int agh_event_destroy(void *event);
int agh_event_record(void *event);
int agh_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for `stop` */

/* --------------------------------------------------------------------- gemm ---- */

/* fn gemm(alpha, a, b, beta, c)  (src/tensor/linalg.rs:249-360), reached from
 * Tensor::dot (:410-421) and ScalarTensor::dot (:453-466).
 *   c[off_c + i*rsc + j*csc] = alpha * sum_x a[off_a + i*rsa + x*csa] * b[off_b + x*rsb + j*csb]
 *                              + beta * c[...]            for i < m, j < n
 * Accumulation is f32 on the matrix cores; bf16 results are rounded once, to nearest
 * even (linalg.rs:244, :217).  beta == 0 never reads c (linalg.rs:215).  a and b may
 * alias each other; c must not overlap a or b, and its m*n elements must be distinct
 * addresses (rsc, csc nonzero and non-overlapping).  m, n or k == 0 is allowed (k == 0
 * yields beta*c).  dims must be < 2^31. */
int agh_gemm_f32(int64_t m, int64_t k, int64_t n, float alpha,
                 const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                 const void *b, int64_t off_b, int64_t rsb, int64_t csb,
                 float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc);
int agh_gemm_bf16(int64_t m, int64_t k, int64_t n, float alpha,
                  const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                  const void *b, int64_t off_b, int64_t rsb, int64_t csb,
                  float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc);

/* agh_gemm_bf16 for callers that cannot allocate: code under hipGraph capture before any eager run, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments,
 * same kernels and bit-identical results, but the split-K partial sums (the only memory the GEMM uses
 * beyond its operands) go to a fixed AGH_NOALLOC_SCRATCH_BYTES buffer that is part of the library image,
 * so the call never reaches hipMalloc / hipFree or any allocating routine.  A shape whose split-K plan
 * needs more scratch than that returns AGH_ERANGE and launches nothing.  Every call on the GPU shares the
 * one buffer: calls are ordered by the library's streams, but a call issued inside a branch
 * (agh_branch_begin) overlaps the main stream's and would race on it, so inside a branch a call whose
 * plan needs the scratch returns AGH_EINVAL.  Nothing in the buffer has to start at zero (every partial that is read
 * was written by the same call). */
#define AGH_NOALLOC_SCRATCH_BYTES 16777216
int agh_gemm_bf16_noalloc(int64_t m, int64_t k, int64_t n, float alpha,
                          const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                          const void *b, int64_t off_b, int64_t rsb, int64_t csb,
                          float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc);

/* Dense forward fused into one launch: `input.dot(&weight)` then `add_assign(bias)`
 * (src/learn/neural_network/layer.rs:1134-1143, autograd.rs:571-599) then the Relu
 * layer that follows it (layer.rs:1254-1267, rule x >= 0 ? x : 0 at :1526-1532).
 * bias (may be null) has n elements at bias[off_bias + j*bias_stride] and is added to
 * every row.  The epilogue rounds in the order the three separate reference ops do:
 * T(dot) -> T(bias + .) -> relu, so bf16 results equal the unfused sequence bit for bit
 * given the same f32 dot. */
int agh_gemm_f32_bias_act(int64_t m, int64_t k, int64_t n, float alpha,
                          const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                          const void *b, int64_t off_b, int64_t rsb, int64_t csb,
                          float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc,
                          const void *bias, int64_t off_bias, int64_t bias_stride, int act);
int agh_gemm_bf16_bias_act(int64_t m, int64_t k, int64_t n, float alpha,
                           const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                           const void *b, int64_t off_b, int64_t rsb, int64_t csb,
                           float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc,
                           const void *bias, int64_t off_bias, int64_t bias_stride, int act);

/* A batch of `batch` independent GEMMs in one launch; matrix i of each operand starts
 * batch_stride_* elements after matrix i-1 (0 = shared by the whole batch), bias/act as in
 * the fused entry points (bias may be null, act AGH_ACT_NONE).  This is how the conv2_im2col
 * chain (src/learn/neural_network/layer.rs:968-1004) writes its result straight in NCHW
 * layout: per image, C is the [oh*ow, oc] product seen column-major (rsc = 1, csc = oh*ow),
 * which removes the reference's `permuted_axes([0,3,1,2]).to_standard_layout()` copy. */
int agh_gemm_f32_batched(int64_t batch, int64_t m, int64_t k, int64_t n, float alpha,
                         const void *a, int64_t off_a, int64_t rsa, int64_t csa, int64_t batch_stride_a,
                         const void *b, int64_t off_b, int64_t rsb, int64_t csb, int64_t batch_stride_b,
                         float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc, int64_t batch_stride_c,
                         const void *bias, int64_t off_bias, int64_t bias_stride, int act);
int agh_gemm_bf16_batched(int64_t batch, int64_t m, int64_t k, int64_t n, float alpha,
                          const void *a, int64_t off_a, int64_t rsa, int64_t csa, int64_t batch_stride_a,
                          const void *b, int64_t off_b, int64_t rsb, int64_t csb, int64_t batch_stride_b,
                          float beta, void *c, int64_t off_c, int64_t rsc, int64_t csc, int64_t batch_stride_c,
                          const void *bias, int64_t off_bias, int64_t bias_stride, int act);

/* ------------------------------------------------------------ im2col / col2im ---- */

/* Im2ColConv2 device branch (src/tensor/ops.rs:842-880; semantics from the host impl
 * :741-813).  x: [bs,c,ih,iw] standard layout.  y: [bs*oh*ow, c*fh*fw] row-major with
 * o = (i + 2p - d(f-1) - 1)/s + 1 (src/ops.rs:35);
 *   y[(b,ho,wo),(ci,fi,fj)] = x[b,ci,-ph+fi*dh+sh*ho,-pw+fj*dw+sw*wo], 0 outside x. */
int agh_im2col_conv2_f32(const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                         int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                         int64_t sh, int64_t sw, int64_t dh, int64_t dw);
int agh_im2col_conv2_bf16(const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                          int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                          int64_t sh, int64_t sw, int64_t dh, int64_t dw);

/* Col2ImConv2 device branch (src/tensor/ops.rs:992-1030).  x: [bs*ih*iw, c*fh*fw] where
 * (ih,iw) is the PATCH GRID (options.shape).  y: [bs,c,oh,ow] with
 * o = (i-1)s + d(f-1) + 1 - 2p (src/ops.rs:75), fully overwritten.  Sums follow the
 * reference's HOST loop (:913-960): accumulator of type T starting at +0, contributions
 * added in (hi, wi) ascending order, every bf16 add rounded - so results are bit-identical
 * to the host path (the reference's own device kernel accumulates in f32 instead). */
int agh_col2im_conv2_f32(const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                         int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                         int64_t sh, int64_t sw, int64_t dh, int64_t dw);
int agh_col2im_conv2_bf16(const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                          int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                          int64_t sh, int64_t sw, int64_t dh, int64_t dw);

/* The input-gradient edge of conv2_im2col in one launch: `output_grad.dot(&weight_matrix)?.col2im_conv2(..)`
 * (src/learn/neural_network/layer.rs:976-988).  dy: the gradient matrix [bs*ih*iw, oc] in standard layout
 * ((ih, iw) the PATCH GRID, as for col2im), w: the filter bank [oc, c, fh, fw] in standard layout, dx:
 * [bs, c, oh, ow], fully overwritten.  Every patch entry is an f32 dot over oc rounded once to T, as
 * agh_gemm_<T> produces it, and the entries are summed like agh_col2im_conv2_<T> (type T, host order): the
 * result differs from the two separate calls only by the order of the f32 adds inside a dot product.  The
 * patch matrix [bs*ih*iw, c*fh*fw] is never written.  The filter bank must fit in LDS as f32
 * (oc*c*fh*fw <= 16384), else AGH_ERANGE: use agh_gemm_<T> + agh_col2im_conv2_<T>. */
int agh_conv2_backward_input_f32(const void *dy, const void *w, void *dx, int64_t bs, int64_t c,
                                 int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw,
                                 int64_t ph, int64_t pw, int64_t sh, int64_t sw, int64_t dh, int64_t dw);
int agh_conv2_backward_input_bf16(const void *dy, const void *w, void *dx, int64_t bs, int64_t c,
                                  int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw,
                                  int64_t ph, int64_t pw, int64_t sh, int64_t sw, int64_t dh, int64_t dw);

/* ---------------------------------------------------------- direct convolution ---- */

/* Conv2 forward without a materialised patch matrix: for layers whose input image and filter
 * bank fit in LDS, and, on the matrix cores as an implicit GEMM, for unit stride and dilation with
 * input channels a multiple of 16 (bf16) or 8 (f32), output channels a multiple of 64 and rows of
 * whole 16-byte vectors (returns AGH_ERANGE otherwise: use im2col + gemm).  Same result as the
 * conv2_im2col chain (src/learn/neural_network/layer.rs:950-1005) up to f32 summation order;
 * the reference's host has the analogous conv_direct path (layer/conv_direct.rs:23-83).
 * x: [bs,ic,ih,iw], w: [oc,ic,fh,fw], bias: null or [oc], added PER OUTPUT CHANNEL (bias[o] to every
 * y[b,o,:,:]).  The reference's conv2 calls `output.add_assign(bias)` (layer.rs:944-946), whose broadcast
 * (autograd.rs:571-599) aligns a [oc] vector with the TRAILING axis of [bs,oc,oh,ow] and so only accepts
 * ow == oc; no reference test or benchmark gives Conv2 a bias, so the per-channel reading is this
 * library's and is not pinned by the reference.
 * act: the Relu layer that follows (layer.rs:1254-1267), pool2x2 != 0: also the MaxPool2 with
 * filter [2,2] and stride [2,2] that follows (layer.rs:1193-1216) with its first-strict-max rule.
 * y: [bs,oc,oh,ow], or [bs,oc,oh/2,ow/2] with the pool.  Rounding order as the separate
 * layers: T(conv) -> T(bias + .) -> relu -> pool. */
int agh_conv2_direct_f32(const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic,
                         int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                         int64_t sh, int64_t sw, int64_t dh, int64_t dw, int act, int pool2x2);
int agh_conv2_direct_bf16(const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic,
                          int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                          int64_t sh, int64_t sw, int64_t dh, int64_t dw, int act, int pool2x2);

/* The LeNet5 of the reference's benchmark (benches/neural-network-benches/src/
 * autograph_backend.rs:88-162) as ONE launch: conv 1->6 5x5, relu, pool 2x2, conv 6->16 5x5, relu,
 * pool 2x2, flatten, dense 256->128, relu, dense 128->84, relu, dense 84->10 + bias, with all
 * activations in LDS and rounded to T after every layer like the layer-by-layer path.
 * x: [bs,1,28,28], w1: [6,1,5,5], w2: [16,6,5,5], wd1: [256,128], wd2: [128,84], wd3: [84,10]
 * (Dense weights are [inputs, outputs], layer.rs:482-486), b3: [10], logits: [bs,10] - a device
 * buffer, or pinned host memory from agh_host_alloc so the result needs no separate copy. */
int agh_lenet5_forward_f32(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                           const void *wd3, const void *b3, void *logits, int64_t bs);
int agh_lenet5_forward_bf16(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                            const void *wd3, const void *b3, void *logits, int64_t bs);

/* The same forward pass for a training step (benches/neural-network-benches/src/autograph_backend.rs:70-86): one
 * launch that also writes what the backward edges read (layer.rs:950-1005, :1193-1216, :1253-1267, autograd.rs:607-627):
 * c1 [bs,6,24,24] and c2 [bs,16,8,8], the convolution outputs BEFORE the relu; p1 [bs,6,12,12] and p2 [bs,16,4,4] after
 * relu and pooling; d1 [bs,128] and d2 [bs,84], the dense outputs before the relu, a1 and a2 after it.  Every value
 * is rounded to T where the layer-by-layer path rounds it; convolutions and dense layers sum in f32 in another order
 * than the GEMM kernels, so results agree with that path up to f32 summation order. */
int agh_lenet5_forward_train_f32(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                                 const void *wd3, const void *b3, void *c1, void *p1, void *c2, void *p2, void *d1,
                                 void *a1, void *d2, void *a2, void *logits, int64_t bs);
int agh_lenet5_forward_train_bf16(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                                  const void *wd3, const void *b3, void *c1, void *p1, void *c2, void *p2, void *d1,
                                  void *a1, void *d2, void *a2, void *logits, int64_t bs);

/* The input-gradient chain of the same training step in one launch (the backward edges of
 * src/learn/neural_network/autograd.rs:239-261 in their order: criterion.rs:79-103, autograd.rs:607-627, layer.rs:1253-1267,
 * :1193-1216, :950-1005): from the logits and the u8 labels, the activations agh_lenet5_forward_train_<T> wrote (c1, c2, d1,
 * d2) and the weights, it writes what the weight gradients multiply: g_logits [bs,10] = dy / bs * (softmax - one-hot),
 * g_d2 [bs,84] and g_d1 [bs,128] (gradients of the dense pre-activations), gm2 [bs*64, 16] and gm1 [bs*576, 6] (gradients
 * of the convolution outputs, as the standard-layout [bs*h*w, c] matrices of layer.rs:976-1003).  dW is then
 * a2^T . g_logits, a1^T . g_d2, flatten(p2)^T . g_d1, gm2^T . im2col(p1) and gm1^T . im2col(x); db3 the axis-0 sum of
 * g_logits.  Values are rounded to T where the separate calls (agh_cross_entropy_backward, agh_gemm, agh_relu_backward,
 * agh_max_pool2_relu_backward, agh_conv2_backward_input) round them; the dense dot products sum in f32 in another
 * order than the GEMM kernels.  wd1 must be 16-byte aligned, wd2 8-byte aligned. */
int agh_lenet5_backward_f32(const void *logits, const void *target, float dy, const void *c1, const void *c2,
                            const void *d1, const void *d2, const void *w2, const void *wd1, const void *wd2,
                            const void *wd3, void *g_logits, void *g_d2, void *g_d1, void *gm2, void *gm1, int64_t bs);
int agh_lenet5_backward_bf16(const void *logits, const void *target, float dy, const void *c1, const void *c2,
                             const void *d1, const void *d2, const void *w2, const void *wd1, const void *wd2,
                             const void *wd3, void *g_logits, void *g_d2, void *g_d1, void *gm2, void *gm1, int64_t bs);

/* The dense layers' weight gradients, the bias gradient and the loss of that step in one launch (autograd.rs:607-627,
 * :490-542, criterion.rs:205-226): dwd3 [84,10] = a2^T . g_logits, dwd2 [128,84] = a1^T . g_d2, dwd1 [256,128] =
 * f^T . g_d1 with f = flatten(p2) [bs,256], each dot summed in f32 over the batch and rounded once to T (as agh_gemm
 * rounds it); db3 [10] = the rows of g_logits added one at a time in T (agh_sum_axis0); *loss = the summed cross-entropy
 * of `logits` against the u8 labels, rows added in order (agh_cross_entropy_loss), written as one f32 to device or pinned
 * host memory; loss may be null (then logits and target are not read). */
int agh_lenet5_dense_weight_grads_f32(const void *a2, const void *a1, const void *f, const void *g_logits,
                                      const void *g_d2, const void *g_d1, void *dwd3, void *dwd2, void *dwd1, void *db3,
                                      const void *logits, const void *target, void *loss, int64_t bs);
int agh_lenet5_dense_weight_grads_bf16(const void *a2, const void *a1, const void *f, const void *g_logits,
                                       const void *g_d2, const void *g_d1, void *dwd3, void *dwd2, void *dwd1, void *db3,
                                       const void *logits, const void *target, void *loss, int64_t bs);

/* The two convolutions' weight gradients of that step without their patch matrices (layer.rs:990-1003:
 * output_grad^T . im2col(input)): dw2 [16,6,5,5] from gm2 [bs*64,16] and p1 [bs,6,12,12], dw1 [6,1,5,5] from gm1
 * [bs*576,6] and x [bs,1,28,28].  Per image the sums run in f32 over the output positions; the images' partial sums
 * (in the library's workspace) are added in image order and rounded once to T, as a split-K agh_gemm rounds. */
int agh_lenet5_conv_weight_grads_f32(const void *x, const void *p1, const void *gm1, const void *gm2, void *dw1, void *dw2,
                                     int64_t bs);
int agh_lenet5_conv_weight_grads_bf16(const void *x, const void *p1, const void *gm1, const void *gm2, void *dw1, void *dw2,
                                      int64_t bs);

/* ---------------------------------------------------------------- max pool ---- */

/* MaxPool2 device branch (src/tensor/ops.rs:1117-1133; rule from the host impl
 * :1062-1084).  x: [bc, ih, iw] (bc = bs*c planes), y: [bc, oh, ow], o = (i - size)/s + 1
 * (src/ops.rs:99).  The first element of the window is taken, a later one replaces it
 * only if strictly greater; the result is a bit copy of that element. */
int agh_max_pool2_f32(const void *x, void *y, int64_t bc, int64_t ih, int64_t iw,
                      int64_t h, int64_t w, int64_t sh, int64_t sw);
int agh_max_pool2_bf16(const void *x, void *y, int64_t bc, int64_t ih, int64_t iw,
                       int64_t h, int64_t w, int64_t sh, int64_t sw);

/* MaxPool2Backward device branch (src/tensor/ops.rs:1252-1264; host rule :1173-1201).
 * dx_inout holds the forward input x on entry ([bc, ih, iw]) and the input gradient on
 * return; dy is [bc, oh, ow].  Per window: every cell is zeroed and `0 + dy` lands on the
 * first strict maximum; cells no window covers keep x.  Overlapping windows
 * (sh < h or sw < w) are applied in the host's (ho, wo) order, one plane per thread. */
int agh_max_pool2_backward_f32(void *dx_inout, const void *dy, int64_t bc, int64_t ih, int64_t iw,
                               int64_t h, int64_t w, int64_t sh, int64_t sw);
int agh_max_pool2_backward_bf16(void *dx_inout, const void *dy, int64_t bc, int64_t ih, int64_t iw,
                                int64_t h, int64_t w, int64_t sh, int64_t sw);

/* Relu followed by MaxPool2 in one pass (layer.rs:1253-1267 then :1193-1216, as LeNet5 chains them,
 * benches/neural-network-benches/src/autograph_backend.rs:114-115, :123-124): y = max_pool2(relu(x)), bit-identical
 * to agh_relu_* followed by agh_max_pool2_*; relu(x) is not written. */
int agh_relu_max_pool2_f32(const void *x, void *y, int64_t bc, int64_t ih, int64_t iw,
                           int64_t h, int64_t w, int64_t sh, int64_t sw);
int agh_relu_max_pool2_bf16(const void *x, void *y, int64_t bc, int64_t ih, int64_t iw,
                            int64_t h, int64_t w, int64_t sh, int64_t sw);

/* The backward of that pair in one pass: dx = relu_backward(x, max_pool2_backward(relu(x), dy)), bit-identical
 * to agh_relu_*, agh_max_pool2_backward_* (in place on relu(x)) and agh_relu_backward_* in a row
 * (layer.rs:205-220, :1542-1565).  x: [bs, c, ih, iw], the input of the relu; dy: [bs, c, oh, ow]; dx (not
 * aliasing x): [bs, c, ih, iw], or with nhwc != 0 [bs, ih, iw, c], which is the standard-layout matrix
 * [bs*ih*iw, c] the convolution backward multiplies (autograd.rs:429-445), so that copy is saved too.
 * Windows must not overlap (sh >= h, sw >= w), else AGH_EINVAL. */
int agh_max_pool2_relu_backward_f32(const void *x, const void *dy, void *dx, int64_t bs, int64_t c,
                                    int64_t ih, int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw, int nhwc);
int agh_max_pool2_relu_backward_bf16(const void *x, const void *dy, void *dx, int64_t bs, int64_t c,
                                     int64_t ih, int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw, int nhwc);

/* -------------------------------------------------------------------- relu ---- */

/* relu / relu_mut (x == y allowed) and relu_backward / relu_backward_mut (dx == dy
 * allowed) kernels (src/learn/neural_network/layer.rs:1542-1565) over n contiguous
 * elements. */
int agh_relu_f32(const void *x, void *y, int64_t n);
int agh_relu_bf16(const void *x, void *y, int64_t n);
int agh_relu_backward_f32(const void *x, const void *dy, void *dx, int64_t n);
int agh_relu_backward_bf16(const void *x, const void *dy, void *dx, int64_t n);

/* ---- around the contraction path: what a training step needs besides the ops above ----
 * All follow the HOST arithmetic of the reference: every operation the host performs in the
 * element type is rounded to the element type, sums run in the host's order. */

/* `assign` with BinaryOp::Identity and alpha = 1: strided copy of up to 4 dimensions between views
 * of the same element type (src/tensor/ops.rs:257-318; device kernels assign{2,4}_<X>_<Y> :1353-1438).
 * This is `into_standard_layout` / `to_standard_layout_shared` (the NHWC<->NCHW copies of
 * layer.rs:1000-1004 and autograd.rs:396-445) and the broadcast of a bias.  Index space d0..d3 (pad
 * with 1), element strides signed, a stride 0 on x broadcasts. */
int agh_assign_f32(const void *x, int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3,
                   void *y, int64_t off_y, int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3,
                   int64_t d0, int64_t d1, int64_t d2, int64_t d3);
int agh_assign_bf16(const void *x, int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3,
                    void *y, int64_t off_y, int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3,
                    int64_t d0, int64_t d1, int64_t d2, int64_t d3);

/* `scaled_add`: y = alpha * x + y on contiguous buffers, product and sum each one operation in the
 * element type; alpha is cast to the element type first (src/tensor/ops.rs:294-296; plain SGD is
 * scaled_add(-learning_rate), optimizer.rs:419-424). */
int agh_scaled_add_f32(void *y, float alpha, const void *x, int64_t n);
int agh_scaled_add_bf16(void *y, float alpha, const void *x, int64_t n);

/* `scaled_add` on views (src/tensor/ops.rs:192-204 -> `assign(BinaryOp::Add, alpha, rhs, self)`, :257-318, eval
 * :1319-1330; device kernels :1400-1438): y[i] = T(T(alpha) * x[i]) + y[i] over the index space d0..d3 (pad with 1),
 * signed element strides, a stride 0 on x broadcasts (`rhs.broadcast(self.raw_dim())`, :287-291).  This is also
 * `add_assign` (alpha = 1, :245-255), i.e. the un-fused `output.add_assign(&bias)` of Dense::forward
 * (layer.rs:1138-1140, autograd.rs:571-599: y [m, n] strides (n, 1), x = bias [n] as strides (0, 1)), and gradient
 * accumulation into a view.  The elements of y must be distinct addresses (no stride 0 along a dimension > 1, else
 * AGH_EINVAL); x may alias y only element for element. */
int agh_scaled_add_strided_f32(void *y, int64_t off_y, int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3, float alpha,
                               const void *x, int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3,
                               int64_t d0, int64_t d1, int64_t d2, int64_t d3);
int agh_scaled_add_strided_bf16(void *y, int64_t off_y, int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3, float alpha,
                                const void *x, int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3,
                                int64_t d0, int64_t d1, int64_t d2, int64_t d3);

/* SGD with momentum: in f32, v = momentum*v + dw; w -= learning_rate*v; both cast back
 * (optimizer.rs:430-465, kernel :509-512). */
int agh_sgd_momentum_f32(void *w, const void *dw, float learning_rate, float momentum, void *velocity, int64_t n);
int agh_sgd_momentum_bf16(void *w, const void *dw, float learning_rate, float momentum, void *velocity, int64_t n);

/* Sum over axis 0 of a row-major [rows, cols] array into y[cols]: zero, then one add in the element
 * type per row, rows ascending (src/tensor/reduce.rs:59-62 on the host; the bias gradient,
 * autograd.rs:490-542). */
int agh_sum_axis0_f32(const void *x, void *y, int64_t rows, int64_t cols);
int agh_sum_axis0_bf16(const void *x, void *y, int64_t rows, int64_t cols);

/* Cross-entropy loss summed over the batch, f32 arithmetic, rows in order
 * (src/learn/criterion.rs:205-226); targets are u8 class indices.  `loss` is one float in device
 * memory or in memory from agh_host_alloc. */
int agh_cross_entropy_loss_f32(const void *x, const void *target_u8, int64_t bs, int64_t classes, float *loss);
int agh_cross_entropy_loss_bf16(const void *x, const void *target_u8, int64_t bs, int64_t classes, float *loss);
/* Its gradient: dx = T((dy / bs) * (softmax(x) - onehot(t))), f32 arithmetic
 * (src/learn/neural_network/criterion.rs:79-103). */
int agh_cross_entropy_backward_f32(const void *x, const void *target_u8, float dy, void *dx, int64_t bs, int64_t classes);
int agh_cross_entropy_backward_bf16(const void *x, const void *target_u8, float dy, void *dx, int64_t bs, int64_t classes);

/* `Accuracy::accuracy` device branch (src/learn/criterion.rs:101-118, kernel :269-296; host rule :30-47): the number
 * of rows of x [bs, classes] whose target score is strictly greater than every other score of the row (ties and
 * NaNs do not count; a target >= classes does not count, where the host panics).  Targets are u8 class indices.
 * `correct` is one uint32 in device memory or in memory from agh_host_alloc. */
int agh_accuracy_f32(const void *x, const void *target_u8, int64_t bs, int64_t classes, void *correct);
int agh_accuracy_bf16(const void *x, const void *target_u8, int64_t bs, int64_t classes, void *correct);

#ifdef __cplusplus
}
#endif
#endif /* AUTOGRAPH_HIP_H */
