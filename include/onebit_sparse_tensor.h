/*
 * C ABI of libonebitmul for MI355X (gfx950): one-bit 2:4 sparse GEMM  D = alpha * A * B + beta * C.
 *
 * Drop-in for the reference header include/onebit_sparse_tensor.h (one declaration, line 5) and its
 * implementation csrc/kernel_lib.cu:23-97. Plain pointers and ints only; no runtime headers are needed
 * to call it. All pointers are DEVICE pointers unless stated otherwise.
 *
 * Operand formats (identical to the reference):
 *   a  one bit per kept value of A, (m x k/2) column-major with packed stride m, LSB first:
 *      bit (r, j) = bit (r + j*m) % 8 of byte (r + j*m) / 8; 1 -> +1.0, 0 -> -1.0
 *      (csrc/kernel_lib.cu:28,37; csrc/kernel.h:13-14; csrc/warp.h:41-50; written by
 *      onebit_sparse_mul/__init__.py:139-143 as a (k/2, m/8) uint8 tensor)
 *   e  int16 metadata, m x k/16 elements, nibble g of an element = idx0 | idx1 << 2 of dense group g,
 *      stored in the reordered layout of onebit_sparse_mul/_semi_structured_conversions.py:21-48,173-177
 *      (csrc/kernel_lib.cu:41)
 *   b  fp16, (k x n) row-major, packed stride n (csrc/kernel_lib.cu:38)
 *   c  (m x n) row-major source, d  (m x n) row-major destination (csrc/kernel_lib.cu:39-40)
 * Shape constraints: m % 64 == 0, k % 32 == 0 (where the reference metadata layout is a bijection),
 * n >= 1. Work is enqueued on a HIP stream and the call returns without synchronising, as the reference
 * does (csrc/kernel_lib.cu:86).
 */
#ifndef ONEBIT_SPARSE_TENSOR_H_
#define ONEBIT_SPARSE_TENSOR_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes for c / d */
#define ONEBIT_DTYPE_F32 0
#define ONEBIT_DTYPE_F16 1

/* metadata layouts of e */
#define ONEBIT_META_REFERENCE 0 /* onebit_sparse_mul/_semi_structured_conversions.py:21-48 (default) */
#define ONEBIT_META_CUTLASS   1 /* CUTLASS reorder_meta (tests/unit/warp_test.h:377-379) */
#define ONEBIT_META_LOGICAL   2 /* plain row-major (m, k/16) */

/* status codes of the int-returning entry points */
#define ONEBIT_OK             0
#define ONEBIT_ERR_ARGUMENT   1 /* null pointer, unsupported shape / dtype / layout */
#define ONEBIT_ERR_HIP        2 /* a HIP runtime call failed (no device, launch failure, out of memory) */

/*
 * Replaces: void onebit_sparse_matmul(void*,void*,void*,void*,void*,int,int,int)
 *           include/onebit_sparse_tensor.h:5, csrc/kernel_lib.cu:23-97.
 * d = 1 * A * b + 0 * c with fp32 c/d (csrc/kernel.h:17-18, csrc/kernel_lib.cu:60-61), metadata in the
 * reference layout, enqueued on the default stream. c is not read (beta = 0) and may equal d, as the torch
 * binding passes it (onebit_sparse_mul/torch_kernel_cuda.cpp:23-24). On any error it prints one line to
 * stderr and calls exit(EXIT_FAILURE), which is the reference's error convention (csrc/kernel_lib.cu:11-20).
 */
void onebit_sparse_matmul(void *a, void *b, void *c, void *d, void *e, int m, int n, int k);

/*
 * Extended form of the entry point above (same operands; csrc/kernel_lib.cu:23-97 with the values it
 * hard-codes at :60-62 and the dtypes of csrc/kernel.h:17-18 turned into arguments): alpha/beta epilogue
 * (csrc/kernel.h:27-31), fp16 or fp32 c and d, metadata layout, explicit stream (hipStream_t passed as
 * void*, NULL = default stream). Returns a status code and never exits.
 * The reordered copy of (a, e) is written on every call to a library-owned workspace kept per device and per
 * stream (grown with a device synchronization when a larger weight arrives; the old buffer is freed, so a HIP graph
 * captured before a larger call on the same stream must be captured again, and a call that would have to grow a
 * buffer while its stream is being captured is refused): calls on different streams may overlap on the GPU. On the
 * host, a call holds a per-device lock from taking that workspace until both kernels are enqueued, so threads that
 * submit to one GPU through this entry point take turns (a few microseconds each). The prepared form below skips the
 * reorder pass and holds the lock only while it looks up its own buffers.
 */
int onebit_sparse_matmul_ex(const void *a, const void *b, const void *c, void *d, const void *e, int m, int n, int k,
                            float alpha, float beta, int c_dtype, int d_dtype, int meta_layout, void *stream);

/*
 * Prepared-operand form: the weight side (a, e) is reordered once into a caller-owned device buffer and
 * reused by every later product. Replaces the host-side metadata reordering that the reference does in
 * Python before the call (onebit_sparse_mul/_semi_structured_conversions.py:171-177) and that CUTLASS
 * does with reorder_meta (tests/unit/warp_test.h:377-379).
 */
size_t onebit_sparse_prepared_bytes(int m, int k);
int onebit_sparse_prepare(const void *a, const void *e, int m, int k, int meta_layout, void *prepared, void *stream);
int onebit_sparse_matmul_prepared(const void *prepared, const void *b, const void *c, void *d, int m, int n, int k,
                                  float alpha, float beta, int c_dtype, int d_dtype, void *stream);

/*
 * The prepared product for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments, kernels and results
 * as onebit_sparse_matmul_prepared; the only difference is where the two internal buffers live that some shapes need
 * (fp32 partial sums when K is split over workgroups, a copy of B with padded rows when B's rows are not 16-byte
 * aligned): in a fixed array of ONEBIT_STATIC_SCRATCH_BYTES bytes that is part of the library's device code, of
 * which every GPU the library runs on holds one copy until the process ends. The call never calls hipMalloc, hipFree
 * or any allocating routine. A shape whose buffers do not fit is refused with ONEBIT_ERR_ARGUMENT and a message
 * that names the sizes (onebit_sparse_describe_launch of the tuning header tells which shapes need buffers: plan[2] > 1 or plan[3] = 1).
 * The buffers are written in full by the call's own kernels before they are read, so the contents a previous call
 * left behind do no harm; but every call on one GPU uses the same array, so two such calls that overlap in time on
 * one GPU (different streams, or different threads) race. Calls on one stream are ordered and safe.
 * Cost: the array is part of the library's code object, so every process that loads libonebitmul.so holds
 * ONEBIT_STATIC_SCRATCH_BYTES (64 MiB) of device memory on each GPU it uses the library on, from the first call of any
 * entry point on that GPU until the process ends, whether or not it ever calls this one.
 */
#define ONEBIT_STATIC_SCRATCH_BYTES (64u << 20)
int onebit_sparse_matmul_prepared_static(const void *prepared, const void *b, const void *c, void *d, int m, int n,
                                         int k, float alpha, float beta, int c_dtype, int d_dtype, void *stream);

/*
 * Linear-layer form of the prepared product, for the forward pass of BinaryLinear_2_4
 * (onebit_sparse_mul/__init__.py:116-128), whose activations are token-major:
 *     y[t][r] = sum over k of W[r][k] * x[t][k]  (+ bias[r] when bias is not NULL)
 * x: fp16, tokens x k, row-major, 16-byte aligned; y: tokens x m, row-major, fp16 or fp32 (y_dtype); bias: m values,
 * fp16 or fp32 (bias_dtype), or NULL. Same result as onebit_sparse_matmul_prepared on B = transpose(x) followed by
 * a transpose of D and the bias addition, without those passes: the kernels read x and write y where they lie.
 */
int onebit_sparse_linear_prepared(const void *prepared, const void *x, const void *bias, void *y, int tokens, int m,
                                  int k, int bias_dtype, int y_dtype, void *stream);

/*
 * Grouped linear-layer form: `count` independent products y_i = x_i W_i^T (+ bias_i) that share the token count, each
 * with its own prepared weight (m_i x k_i), activations x_i (tokens x k_i), bias_i (m_i values or NULL) and result y_i
 * (tokens x m_i); the x_i may be one and the same buffer. `problems` is a HOST array, read before the call returns.
 * For the callers of BinaryLinear_2_4.forward that issue several projections of one layer back to back (q / k / v,
 * gate / up: onebit_sparse_mul/__init__.py:118-128 called once per projection): with tokens <= 64 every 16 problems are
 * one launch of the split-K kernel, whose workgroups are numbered over the concatenated row groups of the problems, so
 * that the launch and the start of the memory stream are paid once instead of per projection (decode-sized products
 * take a few microseconds each, half of which is that). Results are identical to `count` calls of
 * onebit_sparse_linear_prepared without a K split over workgroups (same sums in the same order per element). With
 * tokens > 64 it is exactly such a sequence of calls. bias_dtype and y_dtype hold for all problems. No counterpart in
 * the reference (one launch per product, csrc/kernel_lib.cu:86); allocates nothing.
 */
typedef struct onebit_linear_problem {
  const void *prepared; /* from onebit_sparse_prepare, m x k */
  const void *x;        /* fp16, tokens x k, row-major, 16-byte aligned */
  const void *bias;     /* m values (bias_dtype) or NULL */
  void *y;              /* tokens x m, row-major (y_dtype) */
  int m, k;
} onebit_linear_problem;
int onebit_sparse_linear_prepared_grouped(const onebit_linear_problem *problems, int count, int tokens, int bias_dtype,
                                          int y_dtype, void *stream);

/*
 * Packs a dense fp16 weight (m x k, row-major, device) into the stored operands a (m*k/16 bytes) and e
 * (m*k/8 bytes) on the GPU. Replaces the tensor-op pipeline of BinaryLinear_2_4.pack
 * (onebit_sparse_mul/__init__.py:130-145 with _semi_structured_conversions.py:54-179,286-314): prune != 0 first
 * keeps the two largest magnitudes of every aligned group of four (among equal magnitudes the lower index is
 * pruned), prune == 0 takes the weight's non-zero pattern as it is.
 */
int onebit_sparse_pack(const void *weight, int m, int k, int prune, void *a, void *e, int meta_layout, void *stream);

/* Message of the last failure on the calling thread ("" if none). Host pointer, valid until the next call. */
const char *onebit_sparse_last_error(void);

/* Opt-in cache for callers of the one-call entry points (onebit_sparse_matmul, onebit_sparse_matmul_ex) whose
 * weights do not change, which is inference: with entries > 0 the library keeps the reordered copy of up to that
 * many weights per device, keyed by (a, e, m, k, meta_layout), in its own device memory, and a call with a known
 * key skips the reorder kernel (decode 11008 x 4096 x 16: one kernel instead of two). The caller promises that the
 * memory at a and e is neither modified nor freed and reused while its entry exists; after changing or freeing
 * weights call onebit_sparse_clear_weight_cache(). entries <= 0 (the default, the reference's behaviour: nothing is
 * retained between calls) switches the cache off and clears it. Least recently used entries are evicted (with a
 * device synchronization). A first use allocates with hipMalloc: not inside a stream capture. */
int onebit_sparse_set_weight_cache(int entries);
int onebit_sparse_clear_weight_cache(void);

/* Frees every library-owned buffer (the reordered operands of the one-call entry points, K-split partial sums and
 * padded copies of B, kept per device and per stream and otherwise held until the process ends) after synchronizing
 * the devices that hold any. The weight cache and the static workspace are not touched. Not inside a stream capture;
 * HIP graphs captured earlier must not be replayed afterwards. No counterpart in the reference (its launcher allocates
 * and frees a workspace on every call, csrc/kernel_lib.cu:73-76). */
int onebit_sparse_release_buffers(void);

#ifdef __cplusplus
}
#endif

#endif /* ONEBIT_SPARSE_TENSOR_H_ */
