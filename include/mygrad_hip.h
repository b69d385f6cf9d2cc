/* libmygrad_hip.so -- C ABI of the MI355X (gfx950) conv_nd / max_pool kernels.
 *
 * Every function returns an mg_status (0 = OK, negative = error) and never
 * aborts or throws; mg_last_error() gives the message of the calling thread's
 * last failure.  All tensor arguments are DEVICE pointers obtained from
 * mg_malloc() (plain pointers, C-contiguous row-major, NCHW-style).  Work is
 * enqueued on one library-owned HIP stream; mg_sync() or a device-to-host copy
 * fences it.  The library is not re-entrant: entry points take one global lock.
 *
 * "Reference" below is MyGrad (paths relative to its checkout).
 */
#ifndef MYGRAD_HIP_H
#define MYGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MG_MAX_ND 3 /* spatial / pooled rank handled by the kernels */

typedef enum {
  MG_OK = 0,
  MG_ERR_BAD_ARG = -1,     /* null pointer, non-positive extent, inconsistent shapes */
  MG_ERR_UNSUPPORTED = -2, /* dtype / rank / size outside what the kernels handle */
  MG_ERR_NO_DEVICE = -3,   /* no usable gfx950 device */
  MG_ERR_OOM = -4,         /* device or pinned-host allocation failed */
  MG_ERR_HIP = -5,         /* any other HIP runtime failure */
  MG_ERR_NOT_INIT = -6     /* mg_init() has not succeeded */
} mg_status;

/* MG_F16 (IEEE binary16) is a storage type only: mg_cast and mg_accumulate take it, every other
 * entry point computes in float32 or float64 and refuses it (MG_ERR_UNSUPPORTED). */
typedef enum { MG_F32 = 0, MG_F64 = 1, MG_F16 = 2 } mg_dtype;

/* Shapes of one convolution  x:(N,C,X...) * w:(F,C,W...) -> out:(N,F,G...).
 * Axes are right-aligned: a rank-nd problem fills the LAST nd entries of each
 * array and leaves the leading ones at X=W=G=stride=dil=1, pad=0.  G is passed
 * in, G[k] <= (X[k]+2*pad[k]-((W[k]-1)*dil[k]+1))/stride[k]+1 (floor), so the
 * caller decides between the reference's exact-integer rule
 * (src/mygrad/nnet/layers/conv.py:63-74) and the flooring placement of its
 * window helper (src/mygrad/nnet/layers/utils.py:221-222). */
typedef struct {
  int32_t dtype; /* mg_dtype of x, w, out, grad, dx, dw alike */
  int32_t nd;    /* 1..MG_MAX_ND */
  int64_t N, C, F;
  int64_t X[MG_MAX_ND], W[MG_MAX_ND], G[MG_MAX_ND];
  int64_t stride[MG_MAX_ND], pad[MG_MAX_ND], dil[MG_MAX_ND];
} mg_conv_desc;

/* Shapes of one max-pool over the trailing nd axes of x:(lead, X...) ->
 * out:(lead, G...), window P, step S, no padding, no dilation; `lead` is the
 * product of the un-pooled leading axes (1 if there are none).  Right-aligned
 * like mg_conv_desc.  G[k] <= (X[k]-P[k])/S[k]+1 (floor). */
typedef struct {
  int32_t dtype;    /* mg_dtype of x, out, grad */
  int32_t dx_dtype; /* mg_dtype of dx: same as dtype, or MG_F64 for f32 input (the
                       reference builds dx in float64, pooling.py:147) */
  int32_t nd;       /* 1..MG_MAX_ND */
  int32_t reserved;
  int64_t lead;
  int64_t X[MG_MAX_ND], P[MG_MAX_ND], S[MG_MAX_ND], G[MG_MAX_ND];
} mg_pool_desc;

/* Shapes of one batch normalisation of x:(N, C, S...) over every axis but axis 1;
 * S is the product of the axes after the second (1 if there are none).  gamma and beta
 * are (C,) when announced. */
typedef struct {
  int32_t dtype;     /* mg_dtype of every tensor */
  int32_t has_gamma; /* 0: no scaling (the reference's empty-array gamma, batchnorm.py:48-49) */
  int32_t has_beta;  /* 0: no shift (batchnorm.py:50-51) */
  int32_t reserved;
  int64_t N, C, S;
  double eps;        /* added to the variance under the root, >= 0 */
} mg_bn_desc;

/* A sliding-window view of x:(lead, X...) over its trailing nd axes: window W placed every
 * S elements, its own elements D apart; G[k] <= (X[k] - ((W[k]-1)*D[k]+1)) / S[k] + 1 placements
 * per axis (src/mygrad/nnet/layers/utils.py:201-228).  Right-aligned like mg_conv_desc. */
typedef struct {
  int32_t elem_bytes; /* 1, 2, 4 or 8: the copy moves bytes, any dtype of that size */
  int32_t nd;         /* 1..MG_MAX_ND */
  int64_t lead;
  int64_t X[MG_MAX_ND], W[MG_MAX_ND], S[MG_MAX_ND], D[MG_MAX_ND], G[MG_MAX_ND];
} mg_window_desc;

typedef struct {
  char name[64];      /* hipDeviceProp_t::gcnArchName */
  int32_t compute_units;
  int32_t clock_khz;
  int32_t wavefront;
  int32_t lds_bytes_per_block;
  int64_t hbm_bytes;
  int32_t l2_bytes;
  int32_t memory_clock_khz;
  int32_t memory_bus_bits;
  int32_t reserved;
} mg_device_info_t;

/* ---- runtime (no reference counterpart: the reference is host-only NumPy) ---- */
int mg_init(int device);           /* idempotent; picks the device, creates the stream */
int mg_shutdown(void);             /* frees the stream, workspace and cached plans */
const char *mg_last_error(void);   /* message of this thread's last failing call */
const char *mg_last_plan(void);    /* diagnostics: the kernel family, tile and split that the most recent mg_conv_* or
                                      mg_maxpool_* call ran on; valid until the next call into the library */
int mg_device_info(mg_device_info_t *info);

/* Device memory.  A block given back with mg_free is kept by the library and handed out again
 * by a later mg_malloc of a like size (no driver call, no wait for the device): work that the
 * library enqueued on the block before mg_free runs before anything its next owner enqueues,
 * because there is one stream.  A caller that touches a block from a stream of its own must
 * wait for that work before mg_free.  MYGRAD_HIP_POOL=0 (read by mg_init) switches the reuse
 * off; at most a quarter of the device's memory is kept idle. */
int mg_malloc(void **dptr, size_t nbytes);
int mg_free(void *dptr);
int mg_host_alloc(void **hptr, size_t nbytes); /* pinned host memory (hipHostMalloc); blocks given back are reused like device blocks, at most 8 GiB kept idle */
int mg_host_free(void *hptr);
int mg_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes); /* stream-ordered, returns when src may be reused */
int mg_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes); /* returns when dst holds the data */
int mg_memcpy_d2d(void *dst_dev, const void *src_dev, size_t nbytes);  /* stream-ordered; a plain 16-byte-per-lane
                                                                          copy kernel when everything is 16-byte aligned */
int mg_memset_zero(void *dst_dev, size_t nbytes);                      /* stream-ordered fill kernel */
int mg_sync(void);

/* HIP events on the library stream, for timing kernels from the host. */
int mg_event_create(void **event);
int mg_event_record(void *event);
int mg_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronizes on `stop` */
int mg_event_destroy(void *event);

/* Per-launch kernel timing.  After mg_timing_enable(1) every kernel the library
 * launches is bracketed by a pair of HIP events on the library stream;
 * mg_timing_read() waits for the stream, returns up to `capacity` (tag, ms)
 * records in launch order, sets *count to the number recorded and starts over.
 * Tags: 1 conv forward, 2 conv dgrad, 3 conv wgrad, 4 wgrad split-K reduction,
 * 5 filter packing, 6 max-pool forward, 7 max-pool backward, 8 device copy,
 * 9 element-wise kernel, 10 whole-array sum. */
int mg_timing_enable(int on);
int mg_timing_read(int32_t *tags, float *ms, int capacity, int *count);
/* Suspends (1) or resumes (0) the recording without waiting for the stream and without
 * dropping what was recorded: an event costs a few microseconds of stream time, so a caller
 * that times a long run may record a sample of its steps and let the others run untouched. */
int mg_timing_pause(int paused);

/* Device diagnostic, no counterpart in the reference: the rate at which the
 * matrix cores retire one MFMA instruction shape when nothing else is in their way
 * (independent accumulators in registers, no memory traffic), in TFLOP/s over the
 * whole device.  kind: 0 = v_mfma_f32_16x16x4_f32, 1 = v_mfma_f64_16x16x4_f64,
 * 2 = v_mfma_f64_4x4x4_4b_f64.  waves_per_simd: 1..8 wavefronts issuing on every
 * SIMD.  It is the ceiling the convolution kernels' MFMA loops are measured against
 * besides the published peak (bench.py --probe-mfma). */
int mg_probe_mfma(int kind, int waves_per_simd, double *tflops);

/* Device diagnostic, no counterpart in the reference: one launch that stores (store_big
 * != 0) or loads (store_big == 0) every 16-byte piece of `big` (big_bytes, a multiple of
 * 16) while the opposite stream runs over `small` at 1 / share of that volume -- piece i of
 * big goes with piece i / share of small, which therefore needs ceil(big_bytes / share)
 * bytes (16 with share 0: no second stream).  *ms receives the launch's duration by HIP
 * events.  It measures what the memory system sustains for a given mix of loads and
 * stores, the ceiling of the bandwidth-bound kernels (bench.py --calibrate-mix). */
int mg_probe_stream(void *big_dev, void *small_dev, size_t big_bytes, int share, int store_big, float *ms);

/* ---- convolution ---- */

/* out[n,f,g] = sum_{c,t} w[f,c,t] * x[n,c,g*stride+t*dil-pad] (zero outside x).
 * Replaces ConvND.__call__, src/mygrad/nnet/layers/conv.py:81-103 (np.pad +
 * sliding_window_view + np.tensordot + moveaxis copy). */
int mg_conv_fwd(const mg_conv_desc *desc, const void *x, const void *w, void *out);

/* dx[n,c,i] = sum over (f,t,g) with g*stride+t*dil-pad == i of grad[n,f,g]*w[f,c,t].
 * Replaces ConvND.backward_var(grad, 0), src/mygrad/nnet/layers/conv.py:114-138
 * (tensordot + Python col2im loop + crop). */
int mg_conv_dgrad(const mg_conv_desc *desc, const void *grad, const void *w, void *dx);

/* dw[f,c,t] = sum_{n,g} grad[n,f,g] * x[n,c,g*stride+t*dil-pad].
 * Replaces ConvND.backward_var(grad, 1), src/mygrad/nnet/layers/conv.py:140-155.
 * Split over the (n,g) sum with a fixed-order second stage: run-to-run identical. */
int mg_conv_wgrad(const mg_conv_desc *desc, const void *grad, const void *x, void *dw);

/* ---- max-pool ---- */

/* out[lead,g] = max_a x[lead, g*S+a]; NaN propagates; among equal maxima the
 * value of the first (row-major in the window) is returned.
 * Replaces MaxPoolND.__call__, src/mygrad/nnet/layers/pooling.py:93-98. */
int mg_maxpool_fwd(const mg_pool_desc *desc, const void *x, void *out);

/* dx[lead,i] = sum, in ascending row-major window order starting from +0.0 and
 * accumulated in double, of grad[lead,g] over the windows g whose first-occurrence
 * argmax is i (first NaN wins); rounded once to dx_dtype.  Atomic-free.
 * Replaces MaxPoolND.backward_var, src/mygrad/nnet/layers/pooling.py:100-149
 * (argmax :111, np.add.at :147-148). */
int mg_maxpool_bwd(const mg_pool_desc *desc, const void *x, const void *grad, void *dx);

/* The same pair with the argmax remembered between the passes instead of recomputed:
 * the forward pass also writes argmax[lead,g] (one byte per window, lead * prod(G) bytes:
 * the row-major offset (a0*P1 + a1)*P2 + a2 inside the window of the first-occurrence
 * maximum, the first NaN if any), and the backward pass routes grad from those bytes
 * without reading x.  Same results, bit for bit, as mg_maxpool_fwd / mg_maxpool_bwd while
 * x is unchanged between the two calls.  A window of more than 256 elements is refused
 * (unsupported): use the pair above.
 * mg_maxpool_fwd_argmax replaces MaxPoolND.__call__, src/mygrad/nnet/layers/pooling.py:93-98,
 * and performs the argmax of :109-111 early; mg_maxpool_bwd_argmax replaces the rest of
 * MaxPoolND.backward_var, pooling.py:113-149 (index arithmetic and np.add.at). */
int mg_maxpool_fwd_argmax(const mg_pool_desc *desc, const void *x, void *out, void *argmax);
int mg_maxpool_bwd_argmax(const mg_pool_desc *desc, const void *argmax, const void *grad, void *dx);

/* Backward pass of a pooling over four or five axes that ran as two mg_maxpool_fwd_argmax calls:
 * `inner` over the last three axes (its leading index runs over the un-pooled axes and the leading
 * pooled ones), then `outer` over the leading pooled axes of its result (nd = 2 or 3, the last axis
 * being the inner stage's merged grid with a window of one element placed at every position).
 * grad:(outer lead, outer grid) is routed to dx:(inner lead, inner X...) through both records, every
 * element adding its windows in the row-major order of the whole windows: what np.add.at does for
 * a pooling over all the axes at once, MaxPoolND.backward_var, src/mygrad/nnet/layers/pooling.py:136-148,
 * bit for bit (routing the two stages one after the other adds the same terms in another order). */
int mg_maxpool_bwd_argmax_staged(const mg_pool_desc *inner, const mg_pool_desc *outer, const void *inner_argmax,
                                 const void *outer_argmax, const void *grad, void *dx);

/* The same for six or seven pooled axes, which run as three mg_maxpool_fwd_argmax calls: `third` pools the
 * two foremost axes over the merged grid of the first two stages, as `outer` does over the first
 * stage's.  grad:(third lead, third grid); same order of additions (pooling.py:136-148). */
int mg_maxpool_bwd_argmax_staged3(const mg_pool_desc *inner, const mg_pool_desc *outer, const mg_pool_desc *third,
                                  const void *inner_argmax, const void *outer_argmax, const void *third_argmax, const void *grad,
                                  void *dx);

/* ---- element-wise and whole-array kernels either side of conv / pool ----
 * dtype: 0 float32, 1 float64; n elements, C-contiguous, same shape; device pointers,
 * 16-byte aligned (what mg_malloc returns). */

/* out[i] = a[i] * b[i].  Replaces the body of Multiply.__call__ (np.multiply on
 * same-shape operands, src/mygrad/math/arithmetic/ops.py:45-46) and both branches of
 * Multiply.backward_var (grad * other, ops.py:48-53). */
int mg_multiply(int dtype, int64_t n, const void *a, const void *b, void *out);

/* out = a * b with NumPy's broadcasting (np.multiply in Multiply.__call__, ops.py:45-46, and
 * grad * other in backward_var, ops.py:48-53, before reduce_broadcast sums it back).  `out` is
 * C-contiguous of `shape` (nd axes, 1 to 6: merge neighbouring axes that both operands treat
 * alike first; fewer than 2^31 elements); a_strides / b_strides are the operands' strides in
 * elements along those axes, 0 along an axis the operand is broadcast on, and 1 or 0 along the
 * last axis.  One pass: an operand is read where it lies, never spread out in memory. */
int mg_multiply_broadcast(int dtype, int nd, const int64_t *shape, const int64_t *a_strides, const int64_t *b_strides, const void *a,
                          const void *b, void *out);

/* out[i] = x[i] * (x[i] > 0) as one IEEE multiply by 1 or 0: negative x gives -0.0, NaN
 * stays NaN.  Replaces ReLu.__call__, src/mygrad/nnet/activations/relu.py:11-14. */
int mg_relu_fwd(int dtype, int64_t n, const void *x, void *out);

/* dx[i] = grad[i] * (x[i] > 0).  Replaces ReLu.backward_var, relu.py:16-17 (the mask the
 * reference stores in self.back is recomputed from x). */
int mg_relu_bwd(int dtype, int64_t n, const void *x, const void *grad, void *dx);

/* The same pair with the mask kept between the passes, as the reference keeps it
 * (self.back, src/mygrad/nnet/activations/relu.py:11-17): the forward pass also writes one bit
 * per element, bit i % 8 of mask[i / 8] = (x[i] > 0), (n + 7) / 8 bytes; the backward pass
 * multiplies grad by those bits and does not read x (so it uses the x of the forward pass
 * even if x has changed since, like the reference). */
int mg_relu_fwd_mask(int dtype, int64_t n, const void *x, void *out, void *mask);
int mg_relu_bwd_mask(int dtype, int64_t n, const void *mask, const void *grad, void *dx);

/* *out (one element on the device) = sum of x, added in a fixed tree and carried in double,
 * rounded once.  Replaces Sum.__call__ with axis=None (np.sum,
 * src/mygrad/math/sequential/ops.py:120-121; src/mygrad/operation_base.py Sequential). */
int mg_sum_all(int dtype, int64_t n, const void *x, void *out);

/* mg_sum_all for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same
 * kernels, same chunking, the same result bit for bit, but the chunk sums go to a fixed 32 KiB
 * array in the library's device image (resolved per device by mg_init) instead of the library's
 * growing workspace, and no timing events are recorded: the call allocates nothing on the host
 * side of HIP or on the device.  n above MG_SUM_STATIC_MAX_N is refused (MG_ERR_UNSUPPORTED).
 * Every call on a device shares that device's array: calls that overlap on one device (two
 * host threads are serialised by the library's lock, but two processes' or streams' kernels
 * are not) race.  Nothing needs clearing between calls: each call writes every chunk sum it
 * reads. */
#define MG_SUM_STATIC_MAX_N ((int64_t)1 << 31)
int mg_sum_all_static(int dtype, int64_t n, const void *x, void *out);

/* out[i] = *value (one element on the device).  Replaces Sum.backward_var with axis=None
 * (np.full(a.shape, grad), sequential/ops.py:123-126). */
int mg_fill_from(int dtype, int64_t n, const void *value, void *out);

/* ---- gradient bookkeeping between operations, on the device ----
 * What Operation.backward does to a gradient that backward_var returned before it becomes, or
 * joins, var.grad (src/mygrad/operation_base.py:216-228), and how Tensor.backward seeds the
 * terminal tensor (src/mygrad/tensor_base.py:1308-1334), for gradients that never leave the
 * device.  Buffers from mg_malloc (32-byte aligned for the first two). */

/* out[i] = (to_dtype) x[i]: `backed.astype(var.dtype)`, operation_base.py:223-224 (the float64
 * gradient of a float32 max_pool input, pooling.py:147).  Either type may be MG_F16: float16
 * operands of conv_nd / max_pool are widened to float32 for the kernels and the result is
 * rounded to float16 once, to nearest even (from float64 in one step, not through float32). */
int mg_cast(int from_dtype, int to_dtype, int64_t n, const void *x, void *out);

/* acc[i] = (acc_dtype)(acc[i] + inc[i]), the sum formed in the wider of the two types:
 * `var._grad += backed`, operation_base.py:227-228, with NumPy's rule for a narrower `acc`.
 * Either type may be MG_F16. */
int mg_accumulate(int acc_dtype, int inc_dtype, int64_t n, void *acc, const void *inc);

/* out[i] = value: `np.full_like(self.data, fill_value=1.0)`, the seed of Tensor.backward()
 * without an argument, tensor_base.py:1330-1334. */
int mg_fill_value(int dtype, int64_t n, double value, void *out);

/* ---- batch normalisation ---- */

/* mean[c], var[c] = mean and (biased) variance of x[:, c, ...]; y = (x - mean) /
 * sqrt(var + eps) [* gamma] [+ beta].  The sums run over a fixed partition in double and
 * are rounded once; the element-wise steps are rounded in dtype in the reference's order.
 * mean and var, (C,) each, are outputs the caller keeps for mg_batchnorm_bwd.
 * Replaces BatchNorm.__call__, src/mygrad/nnet/layers/batchnorm.py:26-74. */
int mg_batchnorm_fwd(const mg_bn_desc *desc, const void *x, const void *gamma, const void *beta, void *y, void *mean,
                     void *var);

/* With xn = (x - mean) / sqrt(var + eps) recomputed from x (the reference keeps it in
 * self.x_norm, batchnorm.py:64):
 *   dx     = ((grad - mean_c(grad)) - xn * sum_c(grad * xn) / (N*S)) / sqrt(var + eps) [* gamma]
 *            (BatchNorm.backward_var index 0, batchnorm.py:78-99)
 *   dgamma = sum_c(grad * xn)   (index 1 with gamma, batchnorm.py:101-102)
 *   dbeta  = sum_c(grad)        (index 2, or 1 without gamma, batchnorm.py:104-106)
 * Any of dx, dgamma, dbeta may be null (not wanted), not all three. */
int mg_batchnorm_bwd(const mg_bn_desc *desc, const void *x, const void *grad, const void *gamma, const void *mean,
                     const void *var, void *dx, void *dgamma, void *dbeta);

/* ---- sums over some of the axes ----
 * x is seen as (outer, n, inner), C-contiguous (the caller merges neighbouring axes that are
 * all summed or all kept).  over_middle = 1: out[o, i] = sum_m x[o, m, i], out:(outer, inner).
 * over_middle = 0: out[m] = sum_{o, i} x[o, m, i], out:(n).  Carried in double over a fixed
 * partition, rounded once; run-to-run identical.  More than one kept and one summed group on
 * each side takes several calls.
 * Replaces np.sum(a, axis=...) in Sum.__call__ (Sequential.__call__,
 * src/mygrad/operation_base.py:400-452, src/mygrad/math/sequential/ops.py:120-121) and the
 * sums of reduce_broadcast (src/mygrad/_utils/__init__.py:131-168) behind a broadcasting
 * Multiply. */
int mg_sum_over(int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, void *out);

/* The same sums of x * y for two arrays of one shape, in one pass over both: the product is
 * rounded to dtype before it is added, so the result is that of mg_multiply followed by
 * mg_sum_over.  Replaces grad * other followed by reduce_broadcast's sums in
 * Multiply.backward_var for an operand that was broadcast
 * (src/mygrad/math/arithmetic/ops.py:48-53, src/mygrad/_utils/__init__.py:131-168). */
int mg_sum_product_over(int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, const void *y, void *out);

/* ---- transposition ----
 * out = x.transpose(perm) made C-contiguous: x has `nd` axes of extents shape[], output axis i
 * is input axis perm[i]; elements of 4 or 8 bytes, fewer than 2^31 of them; at most 6 axes
 * after those of length one are dropped and runs that stay together are merged.
 * Brings the operands of an Einstein summation into the order (batch, rows, contracted) /
 * (batch, contracted, columns) that the matrix-product entry points take, and the result back
 * into the order the subscripts ask for: part of what np.einsum does in EinSum.__call__ and
 * EinSum.backward_var, src/mygrad/linalg/ops.py:79-110 and :112-262. */
int mg_permute(int elem_bytes, int nd, const int64_t *shape, const int32_t *perm, const void *x, void *out);

/* Copy between a dense array of `shape` (C-contiguous) and an array of `extent` elements
 * addressed through `strides` (in elements, not negative): element (i_0, ...) of the dense side
 * pairs with offset sum_k i_k * strides[k] of the other.  scatter = 0: out (dense) takes its
 * values from x at those offsets; scatter = 1: x (dense) is written to out at those offsets,
 * which must differ between elements, the rest of out is left as it is.  At most 6 axes.
 * With the sum of several of a tensor's strides as one stride this takes out, and writes back,
 * the diagonals behind a label that occurs twice in one operand of an Einstein summation:
 * np.einsum("ii->i") in EinSum.__call__ and the as_strided view that EinSum.backward_var
 * writes through, src/mygrad/linalg/ops.py:220-262. */
int mg_strided_copy(int elem_bytes, int nd, const int64_t *shape, const int64_t *strides, int64_t extent, int scatter, const void *x,
                    void *out);

/* ---- matrix product ---- */

/* out[b] = a @ x[b], a:(M, K) shared by the batch, x:(batch, K, N), out:(batch, M, N), all
 * C-contiguous.  Runs as the convolution of x with M one-tap filters (the same implicit-GEMM
 * kernels; the reduction has length K).  A stack of left operands times one right operand,
 * (batch, M, K) @ (K, N), is the same call with batch = 1 and M := batch * M.
 * Replaces np.matmul in MatMul.__call__, src/mygrad/math/misc/ops.py:91-93. */
int mg_matmul(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *a, const void *x, void *out);

/* da = sum_b grad[b] @ x[b]^T (M, K): MatMul.backward_var index 0 (np.matmul(grad,
 * b.swapaxes(-1, -2)) summed over the broadcast batch, ops.py:107-114); fixed summation order. */
int mg_matmul_da(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *grad, const void *x, void *da);

/* dx[b] = a^T @ grad[b] (batch, K, N): MatMul.backward_var index 1 (np.matmul(a.swapaxes(-1, -2),
 * grad), ops.py:116-124). */
int mg_matmul_dx(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *grad, const void *a, void *dx);

/* out[p] = op(a[p]) @ op(b[p]) for p < batch: op(a[p]):(M, K), op(b[p]):(K, N), out[p]:(M, N);
 * with trans_a the matrix a[p] is stored as (K, M), with trans_b the matrix b[p] as (N, K); the
 * stacks are C-contiguous.  One launch for the whole stack (a wavefront per 16 x 16 tile of one
 * product), meant for stacks of matrices too small to fill the device one pair at a time; the
 * two gradients are the same call with the transpositions set.  Replaces np.matmul on two
 * stacks in MatMul.__call__ and the products of MatMul.backward_var,
 * src/mygrad/math/misc/ops.py:91-126. */
int mg_matmul_batched(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, int trans_a, int trans_b, const void *a, const void *b,
                      void *out);

/* ---- repeat and the window view ---- */

/* out[o, j, i] = a[o, src(j), i] with a seen as (outer, n, inner) around the repeated axis
 * (outer = inner = 1 for the flattened axis=None case) and out as (outer, total, inner).
 * src_of == NULL: every entry `repeats` times, src(j) = j / repeats, total = n * repeats.
 * Otherwise src_of[total] (int32, on the device) names the source entry of each output entry
 * (np.repeat(arange(n), repeats)).  Moves bytes: elem_bytes in {1, 2, 4, 8}, any dtype.
 * Replaces Repeat.__call__ (np.repeat), src/mygrad/tensor_manip/tiling/ops.py:16-22. */
int mg_repeat_fwd(int elem_bytes, int64_t outer, int64_t n, int64_t inner, int64_t repeats, int64_t total,
                  const int32_t *src_of, const void *a, void *out);

/* da[o, s, i] = sum of grad[o, j, i] over the run of output entries j that came from s, in
 * ascending j starting from +0.0, every addition rounded in dtype.  offsets == NULL: runs of
 * `repeats` (the reference sums a windowed view of grad, tiling/ops.py:36-56); otherwise
 * offsets[n + 1] (int64, on the device), run s = [offsets[s], offsets[s+1]), offsets[n] = total
 * (the reference's np.add.at over repeated flat indices, tiling/ops.py:58-72: same order, same
 * arithmetic).  dtype: 0 float32, 1 float64. */
int mg_repeat_bwd(int dtype, int64_t outer, int64_t n, int64_t inner, int64_t repeats, int64_t total,
                  const int64_t *offsets, const void *grad, void *da);

/* out:(G..., lead, W...) contiguous, out[g, l, w] = x[l, g*S + w*D]: the C-contiguous copy of
 * sliding_window_view(x, W, S, D), src/mygrad/nnet/layers/utils.py:7-228 (the view itself is a
 * host-side stride trick and moves nothing). */
int mg_window_gather(const mg_window_desc *desc, const void *x, void *out);

#ifdef __cplusplus
}
#endif
#endif /* MYGRAD_HIP_H */
