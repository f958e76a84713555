/*
 * dcgan_hip.h -- C ABI of the MI355X (gfx950) backend for dcgan-cuda's convolution hot path.
 *
 * One entry point per operator of the reference's GPU kernel table (src/gpu/kernels.cu:23-61)
 * that a DCGAN training iteration reaches, plus the memory calls behind the reference's
 * tensor_alloc / tensor_write / tensor_read (src/memory/alloc.cu, src/memory/copy.hxx).
 * Plain pointers and sizes only: every `float*` is a DEVICE pointer unless the comment says
 * host.  All tensors are fp32; activations NHWC, filters HWIO, matrices row-major -- the
 * reference's layouts.  `stream` is a hipStream_t passed as void* (NULL = the default stream);
 * calls are asynchronous with respect to the host unless stated otherwise.
 *
 * Every function returns 0 on success or a non-zero code (a hipError_t value, or DH_EINVAL for
 * arguments the kernels cannot take); dh_last_error() describes the last failure of the calling
 * thread.  The host shim turns non-zero into std::runtime_error, the reference's convention
 * (src/memory/alloc.cu:6-14).
 *
 * Threads: the reference drives its GPU from one host thread (src/gpu/runner.cu:10-18) and so
 * does the host mirror here.  Calls from several host threads are allowed when they use
 * different streams (each stream has a scratch arena of its own) and the same device; calls on
 * one stream, the dh_profile_* and dh_debug_* hooks, and dh_init must not overlap with other calls.
 *
 * Each declaration cites the reference interface it stands in for.
 */
#ifndef DCGAN_HIP_H
#define DCGAN_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DH_EINVAL 10001
#define DH_ENOTSUP 10002 /* a paired launch that this shape cannot take: issue the two single calls instead */

/* Epilogue activations that the convolution entry points can fuse. */
enum { DH_ACT_NONE = 0, DH_ACT_RELU = 1, DH_ACT_LEAKY = 2, DH_ACT_TANH = 3, DH_ACT_SIGMOID = 4 };

/* ---- runtime / memory ---------------------------------------------------------------------- */

/* Library version string. */
const char* dh_version(void);
/* Message of the last failed call on this thread ("" if none). */
const char* dh_last_error(void);
/* Select the GPU and create the library's state on it.  Optional: the first call of any other
 * function initialises device 0.  (The reference has no explicit init: its first cudaMalloc,
 * src/memory/alloc.cu:20, creates the context.) */
int dh_init(int device);
/* Name, compute-unit count, engine clock (kHz) and memory size of the current device. */
int dh_device_info(char* name, size_t name_len, int* compute_units, int* clock_khz,
                   size_t* memory_bytes);
/* tensor_alloc / tensor_free in GPU mode: src/memory/alloc.cu:16-37 (cudaMalloc / cudaFree). */
int dh_malloc(void** ptr, size_t bytes);
int dh_free(void* ptr);
/* tensor_write / tensor_read in GPU mode: src/memory/copy.hxx:29-46 (blocking cudaMemcpy).  Like the
 * reference's, these copies are ordered against the DEFAULT stream only; a caller that runs kernels on
 * a stream of its own (dh_stream_create) waits for that stream before it copies results back. */
int dh_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes);
/* The same for the inputs a training loop feeds before every run (src/ops/graph.cu:139-147 writes each
 * fed input with tensor_write): the host buffer is copied into a pinned staging buffer of the library
 * (16 of them, used in turn) and from there to the device in `stream` order (by a kernel that reads the
 * pinned buffer across the bus: it starts sooner than a copy command), so src_host may be reused on
 * return and kernels queued on `stream` afterwards see the data -- but the call does not wait for the
 * work queued before it, as the blocking copy does.  Copies above 64 MiB wait for `stream` and are then
 * blocking. */
int dh_memcpy_h2d_staged(void* dst_device, const void* src_host, size_t bytes, void* stream);
int dh_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes);
int dh_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes, void* stream);
/* tensor_fill with zero (src/memory/copy.hxx:7-27) without the host staging buffer. */
int dh_memset0(void* ptr, size_t bytes, void* stream);
/* cudaDeviceSynchronize of src/gpu/runner.cu:16, moved out of the per-node loop. */
int dh_sync(void);
/* Streams are created non-blocking: work on them is ordered against the default stream and against
 * each other only through dh_stream_wait_event (the reference has one stream and no events). */
int dh_stream_create(void** stream);
int dh_stream_destroy(void* stream);
int dh_stream_sync(void* stream);
int dh_stream_wait_event(void* stream, void* event);
/* HIP events for timing on the stream the kernels run on. */
int dh_event_create(void** event);
int dh_event_destroy(void* event);
int dh_event_record(void* event, void* stream);
int dh_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */
/* Split-K partial sums live in a scratch arena per device and stream that grows on demand (at most
 * 8 streams per device may run kernels that need one); reserving the largest size up front, for the
 * default stream, keeps hipMalloc out of the steady state; dh_workspace_bytes is the sum over streams.  (Replaces the 3-4
 * cudaMalloc/cudaFree per call of src/gpu/conv2d_gemm.hh:514-553.) */
int dh_workspace_reserve(size_t bytes);
size_t dh_workspace_bytes(void);

/* Pooled device memory for tensors: what tensor_alloc / tensor_free call in place of the reference's
 * cudaMalloc / cudaFree per tensor (src/memory/alloc.cu:16-37; one per operator output at every
 * Op::compile, src/ops/conv2d.cu:49-79, and again after an input changes shape, src/ops/graph.cu:104-120).
 * Blocks are carved from a few large slabs the library keeps (256-byte aligned; freed neighbours merge),
 * so a training loop -- and a recompile at another shape that fits what is held -- makes no hipMalloc or
 * hipFree.  A freed block may be handed out again at once: correct for callers that queue all work on one
 * stream (the stream orders the old tensor's last use before the new one's first); others synchronise or
 * order their streams before freeing.  dh_pool_reserve makes sure that ONE idle range of at least
 * `bytes` is held (a dh_pool_alloc of up to that size that follows makes no hipMalloc, however fragmented the
 * rest is), dh_pool_trim returns idle slabs to the driver (after a device synchronisation), dh_pool_stats
 * reports hipMalloc calls made so far, bytes held, bytes handed out and their peak (any may be NULL). */
int dh_pool_alloc(void** ptr, size_t bytes);
int dh_pool_free(void* ptr);
int dh_pool_reserve(size_t bytes);
int dh_pool_trim(void);
int dh_pool_stats(size_t* hipmalloc_calls, size_t* bytes_held, size_t* bytes_in_use, size_t* peak_in_use);

/* Per-kernel timing (no counterpart in the reference, whose only timer is the per-run wall clock of
 * src/ops/graph.cu:150-169).  on = 1 brackets the launches of the convolution kernels by HIP events
 * on the stream they are launched on; on = 2 also those of the reduction, dense and element-wise
 * kernels (some 150 launches per training iteration: the events then slow the iteration itself).
 * dh_profile_read() waits for them and writes one line per kernel tag:
 * "name<TAB>launches<TAB>total ms<TAB>total algorithmic work<TAB>total issued FLOPs", the work being
 * FLOPs, or bytes for the memory-bound kernels, whose tags start with "hbm:"; the last column is what
 * the matrix cores were issued for the convolution launches (live k-slabs as full tiles: skipped
 * padding taps are not in it, the padding of partial tiles is), 0 where that is not accounted. */
int dh_profile_enable(int on);
int dh_profile_reset(void);
int dh_profile_read(char* buf, size_t buf_len);

/* Test hook: on != 0 routes every convolution through the general kernel (element-wise bounds
 * checks, any channel count or alignment) even where the 16-byte buffer-load kernel applies. */
int dh_debug_force_generic_conv(int on);

/* Test and tuning hook: splits > 0 makes every convolution cut its contraction into that many
 * splits (at most one per 16-deep k-slab) instead of choosing by occupancy; 0 restores the choice.
 * The partial sums are added in split order by a second kernel, so results are reproducible. */
int dh_debug_force_splitk(int splits);

/* Test and tuning hook: width 64 or 128 makes every forward / input-gradient launch of the buffer-load
 * kernel whose result has more than 64 columns use 128 x width tiles; 0 restores the library's choice
 * (by rule for launches the device holds at once, by measurement for larger ones, see dh_conv2d_fwd).
 * Without a split the tile width does not change any sum: results are identical to the bit. */
int dh_debug_force_tile_width(int width);

/* ---- convolutions: fp32 implicit GEMM on MFMA, no im2col buffer ------------------------------ */

/* conv2d forward, optionally with the bias add and activation that follow it fused in.
 * Replaces gpu::kernel_conv2d (src/gpu/conv2d.cu:13-62) [+ mvrow_add, src/gpu/matmul.cu:28-38,
 * + vect_relu_leaky etc., src/gpu/relu.cu:26-55].  Also serves conv2d_transpose's input
 * gradient (src/gpu/conv2d.cu:214-259).
 *   x [N,H,W,C]  k [kh,kw,C,O]  y [N,Ho,Wo,O]
 *   y[b,i,j,o] = act(bias[o] + sum_{di,dj,c} x[b, sh*i+di-pad_top, sw*j+dj-pad_left, c] * k[di,dj,c,o])
 * pad_top / pad_left are the pads BEFORE the image (the reference's pad_total / 2).
 * bias may be NULL; alpha is the leaky slope. */
int dh_conv2d_fwd(const float* x, const float* k, float* y,
                  int N, int H, int W, int C, int kh, int kw, int O,
                  int sh, int sw, int pad_top, int pad_left, int Ho, int Wo,
                  const float* bias, int act, float alpha, void* stream);

/* conv2d input gradient == conv2d_transpose forward, optionally with bias + activation fused.
 * Replaces gpu::kernel_conv2d_input_grad (src/gpu/conv2d.cu:70-117) and
 * gpu::kernel_conv2d_transpose (src/gpu/conv2d.cu:167-212).
 *   dy [N,Ho,Wo,O]  k [kh,kw,C,O]  dx [N,H,W,C]
 *   dx[b,h,w,c] = act(bias[c] + sum over (i,di): sh*i+di-pad_top == h, (j,dj) likewise, o of
 *                 dy[b,i,j,o] * k[di,dj,c,o])
 * pad_top / pad_left are those of the forward convolution this is the adjoint of. */
int dh_conv2d_dx(const float* dy, const float* k, float* dx,
                 int N, int Ho, int Wo, int O, int kh, int kw, int C,
                 int sh, int sw, int pad_top, int pad_left, int H, int W,
                 const float* bias, int act, float alpha, void* stream);

/* conv2d filter gradient.  Replaces gpu::kernel_conv2d_kernel_grad (src/gpu/conv2d.cu:119-165)
 * and, with the roles of the activations exchanged, gpu::kernel_conv2d_transpose_kernel_grad
 * (src/gpu/conv2d.cu:264-307).
 *   x [N,H,W,C]  dy [N,Ho,Wo,O]  dk [kh,kw,C,O]
 *   dk[di,dj,c,o] = sum_{b,i,j} x[b, sh*i+di-pad_top, sw*j+dj-pad_left, c] * dy[b,i,j,o]
 * Split-K partial sums are reduced in a fixed order: results are reproducible run to run. */
int dh_conv2d_dk(const float* x, const float* dy, float* dk,
                 int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw,
                 int sh, int sw, int pad_top, int pad_left, void* stream);

/* Two instances of the same product in ONE launch: the same filter applied to two sets of
 * activations of identical shape -- the discriminator on the real and on the generated batch
 * (dcgan/main.cu:304-307 builds it twice over shared variables).  At batch 64 a single instance
 * leaves the machine short of workgroups and has to split its contraction; two instances together
 * need half the splits.
 *   dh_conv2d_fwd_pair: y1 = conv(x1, k), y2 = conv(x2, k)           (+ the same bias / activation)
 *   dh_conv2d_dx_pair:  dx1 = dx(dy1, k), dx2 = dx(dy2, k)           (+ the same bias / activation)
 *   dh_conv2d_dk_pair:  dk = dk(x1, dy1) + dk(x2, dy2), the sum the reference forms with an `add`
 *                       node when a filter receives gradient along two paths (src/ops/graph.cu:295-308)
 * They need the buffer-load kernel (channel counts divisible by 4 and, for the channels the product
 * contracts over -- the input's for fwd, dy's for dx -- by 16; 16-byte aligned tensors below 2 GiB)
 * and return DH_ENOTSUP otherwise; results agree with the single calls to rounding
 * (the contraction may be split differently).  dh_conv2d_dk_pair also takes the thin-input filter
 * gradient (at most 80 filter elements per output channel, at most 64 output channels: the image
 * layer); dh_conv2d_dk_pair_supported tells a caller that plans its launches ahead whether a geometry
 * is one the paired filter gradient takes (1) or not (0), 16-byte aligned tensors assumed. */
int dh_conv2d_fwd_pair(const float* x1, const float* x2, const float* k, float* y1, float* y2, int N, int H, int W,
                       int C, int kh, int kw, int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo,
                       const float* bias, int act, float alpha, void* stream);
int dh_conv2d_dx_pair(const float* dy1, const float* dy2, const float* k, float* dx1, float* dx2, int N, int Ho,
                      int Wo, int O, int kh, int kw, int C, int sh, int sw, int pad_top, int pad_left, int H, int W,
                      const float* bias, int act, float alpha, void* stream);
int dh_conv2d_dk_pair(const float* x1, const float* dy1, const float* x2, const float* dy2, float* dk, int N, int H,
                      int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw, int pad_top, int pad_left,
                      void* stream);
int dh_conv2d_dk_pair_supported(int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw);
/* 1 when dh_conv2d_fwd_pair has a kernel for the geometry (16-byte aligned tensors assumed): input channels
 * divisible by 16 and output channels by 4 with every tensor below 2 GiB, or the image layer's shape (a 5-row
 * filter of 15 values per row, at most 64 output channels, rows of at most 32 output pixels). */
int dh_conv2d_fwd_pair_supported(int N, int H, int W, int C, int kh, int kw, int O, int sh, int sw, int pad_top,
                                 int pad_left, int Ho, int Wo);

/* ---- bias and activations: coalesced, vectorised, one pass over HBM ----------------------------- */

/* out[r,c] = z[r,c] + b[c].  conv2d_bias_add lowers to this (src/ops/conv2d-bias-add.cu:35-38);
 * replaces gpu::mvrow_add (src/gpu/matmul.cu:28-38, :106-119). */
int dh_bias_add(const float* z, const float* b, float* out, size_t rows, size_t cols, void* stream);
/* db[c] = sum_r dz[r,c].  conv2d_bias_add_grad lowers to this
 * (src/ops/conv2d-bias-add-grad.cu:29-31); replaces gpu::mat_sum_cols (src/gpu/sum.cu:112-151). */
int dh_bias_grad(const float* dz, float* db, size_t rows, size_t cols, void* stream);
/* The first half of dh_bias_grad only: parts[q*cols + c] = sum of column c over the q-th range of rows,
 * for the dh_bias_grad_part_count(rows, cols) ranges the matrix is cut into (`parts` must hold that
 * many times cols floats).  The sum over q, in the order dh_bias_grad uses, is left to the consumer:
 * dh_adam_step_multi takes a gradient in this form (no counterpart in the reference, whose
 * mat_sum_cols is one kernel per column block, src/gpu/sum.cu:112-151). */
size_t dh_bias_grad_part_count(size_t rows, size_t cols);
int dh_bias_grad_parts(const float* dz, float* parts, size_t rows, size_t cols, void* stream);
/* dh_bias_grad for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same kernels, same
 * summation order and bit-identical result, but the row-range sums go to a fixed buffer that is part
 * of the library's code object instead of the stream's growing arena: the call allocates and frees
 * nothing.  The buffer is dh_bias_grad_static_max_bytes() = 2 MiB per GPU, held until the process
 * ends; every bias gradient of the DCGAN fits at any batch size.  The call fails with DH_EINVAL when
 * dh_bias_grad_part_count(rows, cols) * cols floats exceed the buffer.  Every call on a GPU shares
 * that GPU's buffer (each range sum is written before it is read, so nothing needs clearing): calls
 * that overlap on one GPU -- from different streams or threads -- race; calls on one stream are
 * ordered by the stream.  dh_init must have run on the device before a stream capture begins: the first
 * library call on a device otherwise initialises it (and looks the buffer's address up) inside that call. */
int dh_bias_grad_static(const float* dz, float* db, size_t rows, size_t cols, void* stream);
size_t dh_bias_grad_static_max_bytes(void);
/* out[r] = sum_c a[r,c].  Replaces gpu::mat_sum_rows (src/gpu/sum.cu:69-108). */
int dh_mat_sum_rows(const float* a, float* out, size_t rows, size_t cols, void* stream);
/* Replace vect_relu / vect_relu_leaky (src/gpu/relu.cu:26-55), vect_sigmoid / vect_tanh
 * (src/gpu/sigmoid.cu:22-50). */
int dh_relu(const float* x, float* out, size_t n, void* stream);
int dh_relu_leaky(const float* x, float* out, size_t n, float alpha, void* stream);
int dh_tanh(const float* x, float* out, size_t n, void* stream);
int dh_sigmoid(const float* x, float* out, size_t n, void* stream);
/* Replace vect_relu_grad / vect_relu_leaky_grad (src/gpu/relu.cu:36-66), vect_sigmoid_grad and
 * vect_tanh_grad (src/gpu/sigmoid.cu:32-40, :114-122).  relu_grad passes dout where z > 0,
 * leaky_relu_grad scales dout by alpha where z < 0; tanh/sigmoid gradients take the forward
 * OUTPUT. */
int dh_relu_grad(const float* z, const float* dout, float* out, size_t n, void* stream);
int dh_leaky_relu_grad(const float* z, const float* dout, float* out, float alpha, size_t n, void* stream);
int dh_tanh_grad(const float* tanh_out, const float* dout, float* out, size_t n, void* stream);
int dh_sigmoid_grad(const float* sig_out, const float* dout, float* out, size_t n, void* stream);
/* out = a + b.  Replaces gpu::vect_add (src/gpu/sum.cu:207-214). */
int dh_add(const float* a, const float* b, float* out, size_t n, void* stream);
/* Fused backward step of a conv layer's bias/activation pair: dz = act'(.) * dout and
 * db[c] = sum_r dz[r,c] in one pass.  `act_ref` is z for relu/leaky (the forward output works
 * equally: same sign) and the forward output for tanh/sigmoid.  db may be NULL.
 * Fuses leaky_relu_grad + mat_sum_cols of the reference's backward node list. */
int dh_act_bias_grad(const float* act_ref, const float* dout, float* dz, float* db,
                     size_t rows, size_t cols, int act, float alpha, void* stream);
/* The same with the column sums left as row-range sums (see dh_bias_grad_parts). */
int dh_act_bias_grad_parts(const float* act_ref, const float* dout, float* dz, float* parts,
                           size_t rows, size_t cols, int act, float alpha, void* stream);

/* ---- losses --------------------------------------------------------------------------------------- */

/* *out = mean_i( x>=0 ? x - x*y + log(1+exp(-x)) : -x*y + log(1+exp(x)) ); out is a device scalar.
 * Replaces gpu::sigmoid_cross_entropy (src/gpu/sigmoid.cu:61-100). */
int dh_sigmoid_cross_entropy(const float* y, const float* logits, float* out, size_t n, void* stream);
/* out[i] = (sigmoid(x[i]) - y[i]) / n.  Replaces src/gpu/sigmoid.cu:103-111. */
int dh_sigmoid_cross_entropy_grad(const float* y, const float* logits, float* out, size_t n, void* stream);
/* Both of the above for one vector of logits, or for two (y2 / logits2 non-null) together with the sum of the
 * two losses, in ONE launch: loss_k = dh_sigmoid_cross_entropy(y_k, logits_k), grad_k =
 * dh_sigmoid_cross_entropy_grad(y_k, logits_k), *loss_sum = *loss1 + *loss2 -- the same values to the bit.  Any
 * of loss1, grad1, loss2, grad2, loss_sum may be NULL.  For a runner that matches the loss node, its gradient
 * node and the `add` that joins the discriminator's two losses (dcgan/main.cu:304-307; kernels
 * src/gpu/sigmoid.cu:61-111, src/gpu/sum.cu:207-214): five one-workgroup launches become one. */
int dh_sigmoid_cross_entropy_head(const float* y1, const float* logits1, float* loss1, float* grad1, const float* y2,
                                  const float* logits2, float* loss2, float* grad2, float* loss_sum, size_t n, void* stream);
/* Mean squared error and its gradient 2/n*(y_hat - y), the loss the reference's conv-gradient tests
 * use (tests/test_conv2d_grad.cu:96).  Replace gpu::mse / mse_grad (src/gpu/sum.cu:15-65). */
int dh_mse(const float* y, const float* y_hat, float* out, size_t rows, size_t cols, void* stream);
int dh_mse_grad(const float* y, const float* y_hat, float* out, size_t n, void* stream);
/* *out = number of rows whose first-maximum column agrees in y and y_hat (ties -> lowest index).
 * Replaces gpu::argmax_acc (src/gpu/sum.cu:154-204). */
int dh_argmax_acc(const float* y, const float* y_hat, float* out, size_t rows, size_t cols, void* stream);

/* ---- dense layers --------------------------------------------------------------------------------- */

/* out (m x p) = a (m x n) * b (n x p) [+ bias (p)].  Replace gpu::matmul / matmul_add
 * (src/gpu/matmul.cu:12-26, :40-56). */
int dh_gemm_nn(const float* a, const float* b, const float* bias, float* out,
               size_t m, size_t n, size_t p, void* stream);
/* dh_gemm_nn followed by an activation (DH_ACT_*) in the write-out: mat_mul_add and the relu of a dense layer
 * (src/api/layers.cu dense_layer: mat_mul_add then the activation op) as one launch. */
int dh_gemm_nn_act(const float* a, const float* b, const float* bias, float* out, size_t m, size_t n, size_t p,
                   int act, float alpha, void* stream);
/* out (m x p) = tr(a) * b, a is (n x m), b is (n x p).  Replaces tmat_mat_mul (src/gpu/matmul.cu:58-71). */
int dh_gemm_tn(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream);
/* out = tr(a1) * b1 + tr(a2) * b2 as ONE contraction over both (the weight gradients of a dense layer that runs
 * on two batches and whose sum is all the optimiser reads).  Takes the shapes dh_gemm_tn_pair_supported
 * answers 1 for (a single output column, p == 1, with m >= 64 and n <= 64) and returns DH_ENOTSUP otherwise. */
int dh_gemm_tn_pair(const float* a1, const float* b1, const float* a2, const float* b2, float* out, size_t m, size_t n,
                    size_t p, void* stream);
int dh_gemm_tn_pair_supported(size_t m, size_t n, size_t p);
/* out (m x p) = a * tr(b), a is (m x n), b is (p x n).  Replaces mat_tmat_mul (src/gpu/matmul.cu:73-86). */
int dh_gemm_nt(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream);

/* ---- optimisers: single pass, HBM-bandwidth bound --------------------------------------------------- */

/* m = a*m + b*g.  Replaces gpu::moment_update (src/gpu/update.cu:24-32). */
int dh_moment_update(float* m, const float* g, float a, float b, size_t n, void* stream);
/* v = a*v + b*g*g.  Replaces gpu::moment_update2 (src/gpu/update.cu:35-43). */
int dh_moment_update2(float* v, const float* g, float a, float b, size_t n, void* stream);
/* p -= lrt * m / (sqrt(v) + eps); lrt = lr*sqrt(1-beta2^t)/(1-beta1^t) is formed by the caller on
 * the host in float, as the reference does (src/gpu/update.cu:81-96). */
int dh_adam_update(float* p, const float* m, const float* v, float lrt, float eps, size_t n, void* stream);
/* The three kernels above in one pass (28 B/param instead of 40):
 *   m = m_decay*m + m_gain*g;  v = v_decay*v + v_gain*g*g;  p -= lrt * m / (sqrt(v) + eps)
 * with the same arithmetic, in the same order, as the three separate calls
 * (the reference passes beta and 1 - beta, src/api/adam-optimizer.cu:48-49). */
int dh_adam_step(float* p, float* m, float* v, const float* g, float m_decay, float m_gain,
                 float v_decay, float v_gain, float lrt, float eps, size_t n, void* stream);

/* The same step for several variables in ONE launch (a DCGAN optimiser step updates 10 variables,
 * most of them bias vectors of a few hundred elements).  Item i uses the gradient g1, or g1 + g2
 * when g2 is not null: that sum is what the reference forms with a separate `add` node when a
 * variable receives gradient along two paths (src/ops/graph.cu:295-308, src/cpu/ops.hxx:933-938).
 * lrt is per item because every variable keeps its own step counter (src/ops/adam-update.cu:45).
 * A gradient may also be handed over as the row-range sums dh_bias_grad_parts / dh_act_bias_grad_parts
 * leave behind: g1_parts > 1 says that g1 holds g1_parts vectors of n elements whose sum is the gradient
 * (likewise g2_parts).  They are added here exactly as dh_bias_grad would have added them, so the
 * result is the same to the bit and the bias gradient's second kernel is never launched. */
typedef struct dh_adam_item
{
    float* p;
    float* m;
    float* v;
    const float* g1;
    const float* g2;
    size_t n;
    float lrt;
    size_t g1_parts; /* 0 or 1: g1 is the gradient itself */
    size_t g2_parts;
} dh_adam_item;
int dh_adam_step_multi(const dh_adam_item* items, int count, float m_decay, float m_gain, float v_decay,
                       float v_gain, float eps, void* stream);
/* var += *coeff * dv with coeff a DEVICE scalar.  Replaces gpu::vect_update (src/gpu/update.cu:14-21). */
int dh_sgd_update(float* var, const float* dv, const float* coeff_device, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif
