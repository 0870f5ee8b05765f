/*
 * ttamd.h — C ABI of the MI355X (gfx950) GEMM backend for tinytensor.
 *
 * This is the drop-in boundary: everything a `BackendAMD : tinytensor::BackendBase`
 * adapter needs for the GEMM hot path (matmul, batched matmul, nn::Linear, conv2d lowered
 * to GEMM and their backward GEMMs).  Plain pointers and sizes only; every pointer named
 * "device pointer" is memory obtained from ttamd_malloc (or any hipMalloc'ed memory of the
 * same device).  Each entry cites the reference interface it stands in for
 * (paths relative to the tinytensor source tree, v1.0.6).
 *
 * Conventions
 *   - dtype codes follow tinytensor::ScalarType (include/tt/scalar.h:21-29).
 *   - Strides and offsets are in ELEMENTS, as in tinytensor::Tensor::stride()/offset()
 *     (include/tt/tensor.h:245-255).  Strides must be >= 0; 0 (expanded dims) is allowed.
 *   - GEMM shapes use the reference's letters: lhs [B,N,K] . rhs [B,K,M] -> out [B,N,M]
 *     (tinytensor/tensor/backend/cpu/matmul.cpp:25-33).
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the default
 *     stream, which is what the reference's GPU backend uses,
 *     tinytensor/tensor/backend/cuda/kernel_launch.cuh:19-29).  Calls do not synchronise;
 *     ttamd_memcpy_d2h and ttamd_device_synchronize do.
 *   - Every function returns a ttamd_status.  The adapter maps TTAMD_ERR_INVALID_ARGUMENT,
 *     TTAMD_ERR_INVALID_DEVICE, TTAMD_ERR_UNSUPPORTED_DTYPE and TTAMD_ERR_OUT_OF_MEMORY to
 *     `throw TTException` (include/tt/exception.h:15-25) and TTAMD_ERR_LAUNCH to TT_ERROR
 *     (print + exit(1), include/tt/exception.h:28-36), mirroring
 *     cuda/kernel_launch.cuh:25-28 and cuda/backend_cuda.cpp:53-63.
 */
#ifndef TTAMD_H_
#define TTAMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ttamd_status {
    TTAMD_OK = 0,
    TTAMD_ERR_INVALID_ARGUMENT = 1, /* shape/stride/pointer contract violated        -> TTException */
    TTAMD_ERR_INVALID_DEVICE = 2,   /* device id out of range                        -> TTException */
    TTAMD_ERR_UNSUPPORTED_DTYPE = 3,/* bool (matmul rejects it) or unknown code      -> TTException */
    TTAMD_ERR_OUT_OF_MEMORY = 4,    /* hipMalloc failed                              -> TTException */
    TTAMD_ERR_LAUNCH = 5            /* kernel launch / runtime failure               -> TT_ERROR    */
} ttamd_status;

typedef enum ttamd_dtype {
    TTAMD_BOOL = 0,
    TTAMD_U8 = 1,
    TTAMD_I16 = 2,
    TTAMD_I32 = 3,
    TTAMD_I64 = 4,
    TTAMD_F32 = 5,
    TTAMD_F64 = 6
} ttamd_dtype;

/* A 3-D strided view of device memory: what a tinytensor::Tensor carries
 * (storage pointer, offset(), stride(); include/tt/tensor.h:245-255). */
typedef struct ttamd_view3 {
    const void *data;  /* device pointer to element 0 of the storage */
    int64_t offset;    /* element offset of the view's first element */
    int64_t stride[3]; /* element strides: batch, row, column        */
} ttamd_view3;

/* A 4-D strided view (NCHW order of dims, arbitrary strides). */
typedef struct ttamd_view4 {
    const void *data;
    int64_t offset;
    int64_t stride[4];
} ttamd_view4;

/* Epilogue fused into the GEMM's store phase.  All fields 0/NULL = plain C = A.B, which is
 * what BackendBase::batched_matmul computes.  The other modes serve the callers either side
 * of the GEMM: nn::Linear's `+ bias->expand()` (tinytensor/nn/linear.cpp:45-48), the ReLU
 * that follows it in an MLP, conv2d's per-channel bias (cpu/conv.cpp:115-124), and the
 * element-wise steps that autograd places around the backward GEMMs of a Linear layer.
 * Order of application to each element v of A.B:
 *   v += bias;  v *= 0 where relu_grad_input < 0 (a product: NaN or infinite v stays NaN);  v = max(v, 0) if relu;
 *   v += out if accumulate;
 *   out = v;  relu_out = max(v, 0);  colsum_out[column] += v.
 * rhs_colsum_out does not depend on the product. */
typedef struct ttamd_epilogue {
    const void *bias; /* device pointer, same dtype as the GEMM, or NULL                      */
    int32_t bias_mode;/* 0 none, 1 = bias[column] (Linear), 2 = bias[row] (conv channel)      */
    int32_t relu;     /* 1: out = max(out, 0) after the bias                                  */
    int32_t accumulate;/* 1: out += result instead of out = result (grad accumulation)        */
    int32_t reserved; /* 0                                                                    */
    /* Linear followed by ReLU in one launch: `out` keeps the Linear result, which autograd saves as the ReLU's
     * input (autograd/unary_ops.cpp:562-567), and relu_out (dense [B,N,M] like out, or NULL) receives max(out, 0).
     * Not together with `relu`. */
    void *relu_out;
    /* TensorRelu::backward (autograd/unary_ops.cpp:568-573: grad_output * where(input < 0, 0, 1)) applied by the
     * GEMM that computes grad_output: dense [B,N,M] like out, the ReLU's saved input, or NULL.  (A masked zero
     * comes out as +0 where the reference's product leaves -0 under a negative value; the two compare equal.) */
    const void *relu_grad_input;
    /* Sum of `out` over its rows, [B,M] (or NULL): the gradient of a Linear layer's bias, which nn/linear.cpp:45-48
     * adds as an expanded view, so its gradient sums the batch dimension.  Per-tile partial sums are added in a fixed
     * order by a second small kernel (deterministic; not the reference's row-by-row order).  f32/f64; not together
     * with `accumulate`.  Written whenever the result has columns (no rows: zeros; K = 0: rows x bias). */
    void *colsum_out;
    /* Sum of the right operand over its rows (k), [B,M] (or NULL): when the product is a Linear layer's weight
     * gradient x^T . dy (TensorBatchedMatmul::backward, autograd/binary_ops.cpp:173-179), the right operand is dy and
     * its column sums are the bias gradient (nn/linear.cpp:45-48), taken from the vectors the product stages anyway
     * where its kernel can, else by a launch of its own.  The right operand must be dense row-major; f32/f64.  Added
     * in a fixed order (deterministic; not the reference's row-by-row order).  Written whenever the right operand has
     * columns (K = 0: zeros; a left operand without rows: no product, the sums all the same). */
    void *rhs_colsum_out;
} ttamd_epilogue;

/* ---- library / device ------------------------------------------------------------------ */

/* BackendBase::get_device_count (tinytensor/tensor/backend_base.h:321). */
ttamd_status ttamd_device_count(int *count);

/* Human-readable text for the last non-OK status returned on this thread
 * (the message the adapter puts into the TTException). */
const char *ttamd_last_error_string(void);

/* Name of the GPU architecture the loaded code object targets ("gfx950"). */
const char *ttamd_target_arch(void);

/* ---- storage: DeviceMemory<T> of the GPU peer (cuda/data_types.cuh:28-101) ------------- */

/* Allocation with per-device byte counters (BackendBase::current_memory_allocated /
 * total_memory_allocated, backend_base.h:317-318). */
ttamd_status ttamd_malloc(int device, size_t bytes, void **out);
ttamd_status ttamd_free(int device, void *ptr, size_t bytes);
ttamd_status ttamd_memory_allocated(int device, uint64_t *current_bytes, uint64_t *total_bytes);
/* The library keeps freed device blocks (by size class) and hands them out again instead of paying
 * hipMalloc + hipFree (25-70 us per pair, and a device-wide wait) for every result tensor; the counters above
 * count what the caller holds, not what is cached.  A cached block may still be in use by kernels enqueued before
 * its free, so the cache follows streams: ttamd_malloc_on_stream / ttamd_free_on_stream name the stream the block
 * is about to be used on / was last used on (ttamd_malloc / ttamd_free mean the default stream, the reference's
 * model: cuda/kernel_launch.cuh:19-29).  A block goes back out at once to a request for a stream it was allocated
 * or freed for (stream order), to a request for another stream only after events recorded on its own streams have
 * completed, and to anyone after ttamd_device_synchronize.  A caller that uses a block on a third stream
 * synchronises that stream before the free.  TTAMD_ALLOC_CACHE=0 switches the cache off.  ttamd_empty_cache waits
 * for the device and returns every cached block to the driver; ttamd_memory_cached reports the bytes currently
 * cached.  Several host threads: a request that considers a block of another stream records and queries events, and
 * a request that the driver cannot serve synchronises the device before it tries again; either would invalidate a
 * graph capture that ANOTHER thread has open in global capture mode, so threads that capture use thread-local or
 * relaxed capture mode, or keep other threads from allocating meanwhile.  No counterpart in the reference, whose
 * DeviceMemory<T> calls cudaMalloc / cudaFree directly (cuda/data_types.cuh:28-101). */
ttamd_status ttamd_malloc_on_stream(int device, size_t bytes, void *stream, void **out);
ttamd_status ttamd_free_on_stream(int device, void *ptr, size_t bytes, void *stream);

/* No counterpart in the reference.  Call before destroying a stream that was ever passed to ttamd_malloc_on_stream or
 * ttamd_free_on_stream: waits for the stream's work (hipStreamSynchronize) and removes the handle from the allocator's
 * books, so that no later request records or queries an event on a stream that no longer exists.  Blocks allocated
 * for the stream stay valid. */
ttamd_status ttamd_stream_release(int device, void *stream);
ttamd_status ttamd_empty_cache(int device);
ttamd_status ttamd_memory_cached(int device, uint64_t *cached_bytes);

/* Blocking copies: BackendBase::from_vec (backend_base.h:35-48) and to_vec (:55-60). */
ttamd_status ttamd_memcpy_h2d(int device, void *dst_device, const void *src_host, size_t bytes);
ttamd_status ttamd_memcpy_d2h(int device, void *dst_host, const void *src_device, size_t bytes);
ttamd_status ttamd_memset_zero(int device, void *dst_device, size_t bytes, void *stream);
ttamd_status ttamd_device_synchronize(int device);

/* BackendBase::identity applied to a strided view = Tensor::contiguous()/clone()
 * (tinytensor/tensor/tensor.cpp:583-596; CPU form cpu/unary.cpp:26-58, index map common/util.h:18-34).
 * Copies the view (ndim <= 8, element strides >= 0) into dense row-major `out`.  The GEMM entry points
 * do not need it; it serves the callers around them (reshape of a non-dense view). */
ttamd_status ttamd_contiguous(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, const int64_t *stride,
                              const void *data, int64_t offset, void *out, void *stream);

/* ---- the hot path ---------------------------------------------------------------------- */

/* BackendBase::batched_matmul (backend_base.h:130; CPU: cpu/matmul.cpp:25-74,
 * GPU peer: cuda/matmul.cu:26-78).  out[b] = lhs[b] . rhs[b] for b < B, out dense row-major
 * [B,N,M].  lhs/rhs may be any non-negative-stride view (permuted, expanded, offset): the
 * kernels read the view in place, no contiguous copy is made.  f32/f64 run on MFMA; u8/i16/
 * i32/i64 wrap modulo 2^n like the reference's SIMD lanes.  `epilogue` may be NULL. */
ttamd_status ttamd_batched_matmul(int device, ttamd_dtype dtype, int B, int N, int K, int M,
                                  const ttamd_view3 *lhs, const ttamd_view3 *rhs, void *out,
                                  const ttamd_epilogue *epilogue, void *stream);

/* Two independent products in one call: what TensorBatchedMatmul::backward (autograd/binary_ops.cpp:173-179) asks of
 * the backend -- dA = dC . B^T and dB = A^T . dC, two batched_matmul calls on permuted views -- and with it the backward
 * of nn::Linear (nn/linear.cpp:42-50).  Each product has ttamd_batched_matmul's contract (operands, epilogue, errors);
 * neither may read the other's result.  Both run as ONE grid when each is a dense fp32 product of 128 to 256 tiles of
 * 64 x 64 with a reduction of 512 or more, `first` with both operands contiguous along k (dC and B^T of dense dC, B),
 * `second` with the left operand contiguous along m and the right along n (A^T and dC of dense A, dC), no colsum_out:
 * a Linear layer of 784 to 1024 features at batch 1024, whose two products alone would each leave the chip one
 * workgroup per CU.  Every element is then summed in k order from 0 (the separate calls add two halves of the
 * reduction): equal on integer-valued data, equal to rounding otherwise, and the same bits on every call.  Anything
 * else runs as two ttamd_batched_matmul calls, first then second. */
typedef struct ttamd_product {
    int B, N, K, M;
    const ttamd_view3 *lhs, *rhs;
    void *out;
    const ttamd_epilogue *epilogue; /* may be NULL */
} ttamd_product;
ttamd_status ttamd_batched_matmul_pair(int device, ttamd_dtype dtype, const ttamd_product *first,
                                       const ttamd_product *second, void *stream);

/* ttamd_batched_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results; the difference is where the partial tiles of a split reduction live: in a fixed 8 MiB
 * array inside the library's code object (one copy per GPU, held until the process ends) instead of the per-stream
 * buffer that ttamd_batched_matmul grows with hipMalloc.  The call makes no hipMalloc / hipFree.  A product whose
 * partial tiles exceed the array (possible for some f64 shapes with fewer than 128 output tiles of 64 x 64) is refused
 * with TTAMD_ERR_INVALID_ARGUMENT and a message naming the sizes.  All calls on one GPU share that GPU's array:
 * calls that may overlap in time on one GPU race.  Calls on one stream are ordered by the stream.  A call that needs
 * the array on a different stream than the last call that used it is refused (TTAMD_ERR_INVALID_ARGUMENT) unless
 * ttamd_device_synchronize has run in between; several host threads launching on one stream are the caller's to
 * serialise.  The first call on a device looks up the array's device address; make that call outside a capture. */
ttamd_status ttamd_batched_matmul_noalloc(int device, ttamd_dtype dtype, int B, int N, int K, int M,
                                          const ttamd_view3 *lhs, const ttamd_view3 *rhs, void *out,
                                          const ttamd_epilogue *epilogue, void *stream);

/* BackendBase::conv2d (backend_base.h:269-275; CPU: cpu/conv.cpp:36-134).  input [B,C,H,W],
 * weight [O,C,k,k] (square kernel), bias [O] or NULL, zero padding; out dense [B,O,Ho,Wo] with
 * Ho = (H + 2*padding - k)/stride + 1.  Implicit GEMM: no im2col buffer is materialised. */
ttamd_status ttamd_conv2d_forward(int device, ttamd_dtype dtype, const ttamd_view4 *input, const ttamd_view4 *weight,
                                  const void *bias, void *out, int B, int C, int H, int W, int O, int k, int stride,
                                  int padding, void *stream);

/* BackendBase::conv2d_backward (backend_base.h:277-284; CPU: cpu/conv.cpp:136-294).
 * grad_out dense [B,O,Ho,Wo] (the reference reads it as dense storage, conv.cpp:199).
 * Writes grad_input [B,C,H,W], grad_weight [O,C,k,k] and, when grad_bias != NULL,
 * grad_bias [O] = sum of grad_out over batch and space (conv.cpp:289).  grad_input is a
 * gather over output positions (no scatter-add, so no write race); grad_weight reduces over
 * the batch inside one GEMM.  `workspace`/`workspace_bytes`: device scratch (never zero bytes
 * for B > 0) holding the weight transposed to [C, O*k*k] for grad_input (for a strided layer:
 * packed per stride class, plus the classes' dense results), the per-split partial tiles of
 * grad_weight and the per-part sums of grad_bias; query the size with ttamd_conv2d_backward_workspace. */
ttamd_status ttamd_conv2d_backward_workspace(ttamd_dtype dtype, int B, int C, int H, int W, int O, int k, int stride,
                                             int padding, size_t *bytes);
ttamd_status ttamd_conv2d_backward(int device, ttamd_dtype dtype, const void *grad_out, const ttamd_view4 *input,
                                   const ttamd_view4 *weight, void *grad_input, void *grad_weight, void *grad_bias,
                                   int B, int C, int H, int W, int O, int k, int stride, int padding, void *workspace,
                                   size_t workspace_bytes, void *stream);

/* No counterpart in the reference: which kernel family the calling thread's last ttamd_conv2d_forward (which = 0) or
 * the grad_input (which = 1) or grad_weight (which = 2) part of its last ttamd_conv2d_backward launched.  0x100: the
 * implicit-GEMM MFMA kernels; 0x200 + 16 * waves + patch buffers: the persistent kernel that keeps the weight block in
 * LDS (fp32, unit stride, channel counts that are multiples of 8, rows of whole 16-byte vectors), 0x200 for
 * grad_weight: the kernel that stages both operands in LDS; 0: neither (another dtype, a direct kernel) or no call
 * yet.  which = 3: how the partial tiles of that grad_weight were added up -- 0: there were none, 1: by a launch of
 * their own, 2: by workgroups appended to grad_input's launch.  For tests and profiles that mean to cover a particular
 * kernel. */
int ttamd_conv2d_last_kernel(int which);

/* BackendBase::max_pool2d / min_pool2d / avg_pool2d (backend_base.h:286-311; CPU: cpu/conv.cpp:296-349 over
 * cpu/kernel/conv.hpp:121-161).  input [B,C,H,W] (any strides), square window k, zero-contribution padding;
 * out dense [B,C,Ho,Wo] of the input's dtype, except avg of an integer input, which is f32
 * (common/reduce.h:63-69).  The window is folded in the reference's order with its arithmetic
 * (avg: out = x / (k*k) + out), so results are bit-identical to the CPU device's. */
typedef enum { TTAMD_POOL_MAX = 0, TTAMD_POOL_MIN = 1, TTAMD_POOL_AVG = 2 } ttamd_pool_op;
ttamd_status ttamd_pool2d_forward(int device, ttamd_dtype dtype, int op, const ttamd_view4 *input, void *out, int B,
                                  int C, int H, int W, int k, int stride, int padding, void *stream);
/* BackendBase::*_pool2d_backward (backend_base.h:288-311; CPU: cpu/conv.cpp:351-426 over conv.hpp:171-275); f32/f64.
 * grad_out and result dense [B,C,Ho,Wo]; writes every element of grad_input [B,C,H,W] (dense).  max/min: an
 * output's gradient is split evenly over the in-bounds window elements equal to the result. */
ttamd_status ttamd_pool2d_backward(int device, ttamd_dtype dtype, int op, const void *grad_out, const ttamd_view4 *input,
                                   const void *result, void *grad_input, int B, int C, int H, int W, int k, int stride,
                                   int padding, void *stream);

/* ---- elementwise / reduction ops that an MLP training step needs around its GEMMs ------------
 * (BackendBase::add, sub, mul, div, pow, maximum, minimum, lt, le, gt, ge, eq, ne: backend_base.h:109-131;
 * relu & friends: :136-260; where: :263; sum: :148-149; full: :51.  CPU forms: cpu/binary.cpp:26-84,
 * cpu/unary.cpp:26-82, cpu/kernel/reduce.hpp:15-48, functors in common/kernel/binary.hpp, unary.hpp.)
 * Operands are strided views (ndim <= 8, element strides >= 0) of ONE shape: the frontend broadcasts with
 * expand() before it calls the backend.  Results are dense row-major.  dtype = operand dtype; comparison
 * results are bool (one byte, 0/1).  Integer arithmetic wraps; integer division by zero yields 0. */
typedef enum ttamd_binary_op {
    TTAMD_BIN_ADD = 0, TTAMD_BIN_SUB, TTAMD_BIN_MUL, TTAMD_BIN_DIV, TTAMD_BIN_POW, TTAMD_BIN_MAXIMUM, TTAMD_BIN_MINIMUM,
    TTAMD_BIN_LT, TTAMD_BIN_LE, TTAMD_BIN_GT, TTAMD_BIN_GE, TTAMD_BIN_EQ, TTAMD_BIN_NE
} ttamd_binary_op;
typedef enum ttamd_unary_op {
    TTAMD_UN_RELU = 0, TTAMD_UN_NEGATE, TTAMD_UN_ABS, TTAMD_UN_SQRT, TTAMD_UN_EXP, TTAMD_UN_LOG, TTAMD_UN_SIGMOID, TTAMD_UN_TANH
} ttamd_unary_op;
ttamd_status ttamd_binary(int device, ttamd_dtype dtype, int op, int ndim, const int64_t *shape, const void *lhs,
                          int64_t lhs_offset, const int64_t *lhs_stride, const void *rhs, int64_t rhs_offset,
                          const int64_t *rhs_stride, void *out, void *stream);
ttamd_status ttamd_unary(int device, ttamd_dtype dtype, int op, int ndim, const int64_t *shape, const void *src,
                         int64_t offset, const int64_t *stride, void *out, void *stream);
/* BackendBase::to (backend_base.h:74; CPU: cpu/cast.cpp:27-110): out[i] = static_cast<to>(view[i]), dense result of
 * dtype `to`; a bool result is 1 for every non-zero element.  Float values outside the target integer's range
 * are undefined in the reference and saturate here. */
ttamd_status ttamd_cast(int device, ttamd_dtype from, ttamd_dtype to, int ndim, const int64_t *shape, const void *src,
                        int64_t offset, const int64_t *stride, void *out, void *stream);
/* BackendBase::assign (backend_base.h:78; CPU: cpu/kernel/assign.hpp:15-21): dst_view[i] = src_view[i] over one
 * shape; both operands are strided views of the same dtype (any dtype, bool included). */
ttamd_status ttamd_assign(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, void *dst, int64_t dst_offset,
                          const int64_t *dst_stride, const void *src, int64_t src_offset, const int64_t *src_stride,
                          void *stream);
/* BackendBase::where (backend_base.h:263): out = cond ? lhs : rhs; cond is a bool (one byte) view. */
ttamd_status ttamd_where(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, const void *cond,
                         int64_t cond_offset, const int64_t *cond_stride, const void *lhs, int64_t lhs_offset,
                         const int64_t *lhs_stride, const void *rhs, int64_t rhs_offset, const int64_t *rhs_stride,
                         void *out, void *stream);
/* BackendBase::sum(tensor) (dim = -1, one element out) and sum(tensor, dim) (that dimension removed).  The result has
 * the operand's dtype for f32 / f64; bool and every integer dtype are summed in 64 bits and the result is I64
 * (common/reduce.h:56-61, cpu/reduce.cpp:38-54), so `out` holds 8 bytes per element for them. */
ttamd_status ttamd_sum(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, const void *src, int64_t offset,
                       const int64_t *stride, int dim, void *out, void *stream);
/* BackendBase::full (backend_base.h:51): `value` points at one host scalar of `dtype`. */
ttamd_status ttamd_full(int device, ttamd_dtype dtype, const void *value, int64_t numel, void *out, void *stream);

/* nn::mse_loss(input, target, ReductionMode::mean) (nn/loss.cpp:69-72) and its backward in one pass over dense
 * [rows, cols] operands (f32 / f64).  What the reference computes op by op -- pow(input - target, 2), mean as
 * (x / numel).sum() (autograd/reduce_ops.cpp:195-205), and backward grad_input = (1 / numel) * 2 * (input - target)
 * (autograd/binary_ops.cpp:153-159) -- as one streaming kernel plus a one-workgroup finish: loss_out [1];
 * grad_input_out [rows, cols] or NULL; grad_colsum_out [cols] or NULL = grad_input summed over the rows (the bias
 * gradient of the Linear layer that produced `input`; cols <= 64 only, wider matrices sum with ttamd_sum).
 * Sums run in a fixed order (deterministic), not in the reference's element order. */
ttamd_status ttamd_mse_loss(int device, ttamd_dtype dtype, int64_t rows, int64_t cols, const void *input,
                            const void *target, void *loss_out, void *grad_input_out, void *grad_colsum_out,
                            void *stream);

/* The last Linear layer of a network together with the loss it feeds, forward and backward, for layers of at most 64
 * outputs (the 10 classes of the reference's MLP): what nn::Linear::forward (nn/linear.cpp:42-50), nn::mse_loss with
 * mean reduction (nn/loss.cpp:69-72) and their autograd nodes (autograd/reduce_ops.cpp:195-205,
 * binary_ops.cpp:153-159,173-179, unary_ops.cpp:568-573) compute op by op:
 *   output [rows, out]          = input [rows, in] . weight [in, out] + bias [out] (bias may be NULL)
 *   loss_out [1]                = mean((output - target)^2)
 *   grad_output_out [rows, out] = (1 / numel) * 2 * (output - target)
 *   grad_input_out [rows, in]   = (grad_output . weight^T) * where(relu_input < 0, 0, 1)  (relu_input [rows, in], the
 *                                 saved input of the ReLU that produced `input`, or NULL: no mask)
 *   grad_weight_out [in, out]   = input^T . grad_output;   grad_bias_out [out] (or NULL) = grad_output summed over rows.
 * All operands dense row-major, f32 / f64.  With f32, at most 16 outputs, in_features a multiple of 4 and 16-byte
 * aligned input / relu_input / grad_input_out these are two launches (every step but the sums over the rows is local
 * to a block of 16 rows); otherwise the call runs ttamd_batched_matmul and ttamd_mse_loss one after the other, with
 * the same results up to the order of the sums (all orders fixed: deterministic either way). */
ttamd_status ttamd_linear_mse_head(int device, ttamd_dtype dtype, int64_t rows, int64_t in_features, int64_t out_features,
                                   const void *input, const void *weight, const void *bias, const void *target,
                                   const void *relu_input, void *output, void *loss_out, void *grad_output_out,
                                   void *grad_input_out, void *grad_weight_out, void *grad_bias_out, void *stream);

/* BackendBase::uniform_real_ / normal_ (backend_base.h:96-103) for a dense float tensor with scalar parameters, as
 * nn::Linear's default initialisation calls them (nn/init.cpp:30-52,106-112).  dist 0 = uniform_real(low = p0,
 * high = p1), 1 = normal(mu = p0, std = p1).  *master_state is the caller's Generator state (tensor/random.cpp:46-63);
 * it advances by numel outputs.  Per-element states are produced on the host and uploaded, as the reference's GPU
 * backend does (cuda/distribution.cu:32-99), so uniform values are bit-identical to the CPU backend's. */
ttamd_status ttamd_random_fill(int device, ttamd_dtype dtype, int dist, double p0, double p1, uint64_t *master_state,
                               int64_t numel, void *out, void *stream);
/* The same draws written in place through a strided view (ndim <= 8, element strides >= 0), as the CPU backend's
 * in-place kernel does (cpu/distribution.cpp:96-139, cpu/kernel/distribution.hpp:28-32): element i of the view, i
 * its row-major rank over `shape`, takes the i-th master output as its state and lands at
 * data[offset + sum(index[d] * stride[d])] (common/util.h:18-34).  nn::Conv2d initialises its weight through
 * weight->permute({1,0,2,3}) (nn/conv2d.cpp:56), so the draw order runs over [C,O,k,k] while the storage is [O,C,k,k]. */
ttamd_status ttamd_random_fill_view(int device, ttamd_dtype dtype, int dist, double p0, double p1, uint64_t *master_state,
                                    int ndim, const int64_t *shape, const int64_t *stride, void *data, int64_t offset,
                                    void *stream);
/* The same with the per-element generator states supplied by the caller (host array, one per element of the view in
 * its row-major order): what an adapter inside the reference passes, whose Generator (include/tt/random.h:17-42)
 * hands out states only through operator() -- create_gen_states, cpu/distribution.cpp:31-38, draws them exactly so. */
ttamd_status ttamd_random_fill_states(int device, ttamd_dtype dtype, int dist, double p0, double p1, const uint64_t *states,
                                      int ndim, const int64_t *shape, const int64_t *stride, void *data, int64_t offset,
                                      void *stream);

/* The tensor forms of BackendBase::uniform_real / normal (backend_base.h:83-103; GPU peer cuda/distribution.cu:32-99):
 * a parameter pair per element.  p0 / p1 (low / high, or mu / std) are device views over the same `shape` as the result
 * -- storage pointer, element offset, element strides (0 for an expanded value) -- and element i of the result, i its
 * row-major rank, reads them at rank i, as the CPU backend reads params[i] of the parameters made contiguous
 * (cpu/distribution.cpp:42-47, cpu/kernel/distribution.hpp:28-32).  low < high per element is the caller's to keep
 * (the reference asserts it, common/kernel/distribution.hpp:95). */
ttamd_status ttamd_random_fill_states_params(int device, ttamd_dtype dtype, int dist, const void *p0, int64_t p0_offset,
                                             const int64_t *p0_stride, const void *p1, int64_t p1_offset,
                                             const int64_t *p1_stride, const uint64_t *states, int ndim, const int64_t *shape,
                                             const int64_t *stride, void *data, int64_t offset, void *stream);

/* ---- timing (no reference counterpart: the reference has no timers; used by the benchmark
 * to bracket kernels with HIP events on the stream they run on) ------------------------ */
ttamd_status ttamd_event_create(int device, void **event);
ttamd_status ttamd_event_destroy(void *event);
ttamd_status ttamd_event_record(void *event, void *stream);
ttamd_status ttamd_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronises on `stop` */

/* Name of the kernel variant the dispatcher would pick for a batched_matmul call with these
 * arguments (for profiles and tests; does not launch).  Returned pointer is static. */
const char *ttamd_batched_matmul_variant(ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs,
                                         const ttamd_view3 *rhs);

#ifdef __cplusplus
}
#endif
#endif /* TTAMD_H_ */
