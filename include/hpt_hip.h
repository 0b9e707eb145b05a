/*
 * hpt_hip.h — C ABI of libhpt_hip.so: the MI355X (gfx950) device side of Hpt's
 * reduction / softmax / layernorm path, as a `Hip` backend would bind it.
 *
 * Conventions
 *   - Every function returns an hpt_status (0 = ok). On failure a thread-local,
 *     human readable message is available from hpt_hip_last_error(). The text
 *     of parameter/shape errors follows Hpt's TensorError Display strings
 *     (hpt-common/src/error/shape.rs:62, hpt-common/src/error/param.rs:17).
 *   - Views describe memory the way Hpt's `_Tensor` does (hpt/src/tensor_base.rs:17-29):
 *     `data` is the already-offset element pointer (Hpt's Pointer<T>), `shape`
 *     and `strides` are i64 arrays of length `ndim`, strides in ELEMENTS.
 *   - Output tensors are allocated by the caller (through hpt_hip_alloc, i.e.
 *     the Hip allocator) and must be contiguous; the library never allocates or
 *     frees user-visible tensors. Scratch for multi-stage reductions is owned
 *     by the library: one buffer per (device, stream), taken from the same caching
 *     allocator, grown on demand, released by hpt_hip_cache_clear.
 *   - Kernels are enqueued on `stream` (a hipStream_t passed as void*; NULL =
 *     the device's default stream) and are NOT synchronised; the *_sync copy
 *     functions block until the copy is complete.
 *   - All functions may be called concurrently from several host threads.
 *     Calls that share one stream are ordered by that stream.
 */
#ifndef HPT_HIP_H
#define HPT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same dtype set (and order) as the DECLARE_KERNEL lists of the reference's
 * device kernels (hpt-cudakernels/src/reduce/sum.cu:4-16). */
typedef enum hpt_dtype {
    HPT_BOOL = 0,
    HPT_I8 = 1,
    HPT_I16 = 2,
    HPT_I32 = 3,
    HPT_I64 = 4,
    HPT_U8 = 5,
    HPT_U16 = 6,
    HPT_U32 = 7,
    HPT_U64 = 8,
    HPT_F16 = 9,
    HPT_BF16 = 10,
    HPT_F32 = 11,
    HPT_F64 = 12,
    HPT_DTYPE_COUNT = 13
} hpt_dtype;

/* One value per reduction method of NormalReduce / FloatReduce /
 * NormalEvalReduce / EvalReduce (hpt-traits/src/ops/reduce.rs:45-358). */
typedef enum hpt_reduce_op {
    HPT_SUM = 0,        /* NormalReduce::sum        reduce.rs:64  */
    HPT_PROD = 1,       /* NormalReduce::prod       reduce.rs:107 */
    HPT_MAX = 2,        /* NormalReduce::max        reduce.rs:137 */
    HPT_MIN = 3,        /* NormalReduce::min        reduce.rs:122 */
    HPT_MEAN = 4,       /* FloatReduce::mean        reduce.rs:300 */
    HPT_NANSUM = 5,     /* NormalEvalReduce::nansum reduce.rs:232 */
    HPT_NANPROD = 6,    /* NormalEvalReduce::nanprod reduce.rs:275 */
    HPT_REDUCEL1 = 7,   /* NormalReduce::reducel1   reduce.rs:152 */
    HPT_REDUCEL2 = 8,   /* FloatReduce::reducel2    reduce.rs:315 */
    HPT_REDUCEL3 = 9,   /* FloatReduce::reducel3    reduce.rs:334 */
    HPT_SUM_SQUARE = 10,/* NormalReduce::sum_square reduce.rs:171 */
    HPT_LOGSUMEXP = 11, /* FloatReduce::logsumexp   reduce.rs:353 */
    HPT_ALL = 12,       /* EvalReduce::all          reduce.rs:195 */
    HPT_ANY = 13,       /* EvalReduce::any          reduce.rs:211 */
    HPT_REDUCE_OP_COUNT = 14
} hpt_reduce_op;

/* Status codes; the Rust shim maps them onto TensorError variants
 * (hpt-common/src/error/base.rs:8-45). */
typedef enum hpt_status {
    HPT_OK = 0,
    HPT_ERR_PARAM = 1,   /* TensorError::Param  (duplicated axis, bad argument)         */
    HPT_ERR_SHAPE = 2,   /* TensorError::Shape  (axis out of range, size/shape mismatch) */
    HPT_ERR_DTYPE = 3,   /* unsupported dtype for this op                                */
    HPT_ERR_MEMORY = 4,  /* TensorError::Memory (allocation failed)                      */
    HPT_ERR_KERNEL = 5,  /* TensorError::Kernel (launch / execution failed)              */
    HPT_ERR_DEVICE = 6   /* TensorError::Device (no such device, runtime failure)        */
} hpt_status;

/* A strided view of device memory: what `_Tensor{data, layout}` holds
 * (hpt/src/tensor_base.rs:17-29; strides in elements, data already offset). */
typedef struct hpt_view {
    void* data;
    const int64_t* shape;
    const int64_t* strides;
    int32_t ndim;
    int32_t dtype; /* hpt_dtype */
} hpt_view;

/* ---- error / info ----------------------------------------------------- */

/* Thread-local message of the last failing call on this thread ("" if none). */
const char* hpt_hip_last_error(void);

/* Size in bytes of one element of `dtype` (0 for an invalid dtype). */
size_t hpt_hip_dtype_size(int32_t dtype);

/* Number of visible HIP devices. Replaces cudarc's device enumeration used by
 * hpt-allocator/src/allocators/cuda.rs:63-76. */
int32_t hpt_hip_device_count(int32_t* n);

/* ---- device allocator (hpt-allocator) ----------------------------------
 * An LRU caching allocator keyed by (bytes, align), one cache per device, with
 * the behaviour of CudaAllocator (hpt-allocator/src/allocators/cuda.rs:41-322):
 * a freed block goes back to the cache; a cache miss calls hipMalloc; when
 * hipMalloc fails, least-recently-used cache entries are released and the
 * allocation is retried (hpt-allocator/src/utils/allocate.rs:15-60). */

/* Allocator::allocate / allocate_zeroed (hpt-allocator/src/traits.rs:25-41). */
int32_t hpt_hip_alloc(int32_t dev, size_t bytes, size_t align, int32_t zeroed, void** out);
/* Allocator::deallocate (hpt-allocator/src/traits.rs:43-50): returns the block
 * to the cache. `p` must come from hpt_hip_alloc with the same (bytes, align).
 * The block may be handed out again at once: free it only after the stream that
 * last used it has finished with it. */
int32_t hpt_hip_free(int32_t dev, void* p, size_t bytes, size_t align);
/* Allocator::forget (hpt-allocator/src/allocators/cuda.rs:140-146; called by Tensor::forget,
 * hpt/src/backends/cuda/tensor_impls.rs:277-306): the allocator stops tracking `p`, which the
 * caller owns from now on (it came from hipMalloc: release it with hipFree). A pointer the
 * allocator does not know is ignored. The opposite direction, Tensor::from_raw
 * (hpt/src/backends/cpu/tensor_impls.rs:123-147), needs no call: every entry point takes any
 * device pointer, whoever allocated it, at any element-aligned address. */
int32_t hpt_hip_forget(int32_t dev, void* p);
/* resize_cuda_lru_cache (hpt/src/lib.rs:449-450). Evicted blocks are released. */
int32_t hpt_hip_cache_resize(int32_t dev, size_t entries);
/* Allocator::clear (hpt-allocator/src/traits.rs:55): release every cached block, and the
 * library's own scratch buffers of this device (after waiting for the device to go idle). */
int32_t hpt_hip_cache_clear(int32_t dev);
/* Counters for tests and leak checks: blocks handed out and not yet freed,
 * blocks sitting in the cache, and hipMalloc calls made so far. */
int32_t hpt_hip_alloc_stats(int32_t dev, uint64_t* live_blocks, uint64_t* cached_blocks,
                            uint64_t* device_mallocs);

/* ---- transfers (to_cuda / to_cpu) --------------------------------------
 * Synchronous copies, as `to_cuda` (hpt/src/backends/cpu/tensor_impls.rs:295-313)
 * and `to_cpu` (hpt/src/backends/cuda/tensor_impls.rs:142-169) perform. */
int32_t hpt_hip_memcpy_h2d_sync(int32_t dev, void* dst, const void* src, size_t bytes);
int32_t hpt_hip_memcpy_d2h_sync(int32_t dev, void* dst, const void* src, size_t bytes);
int32_t hpt_hip_memcpy_d2d_sync(int32_t dev, void* dst, const void* src, size_t bytes);
/* Block until everything queued on `stream` has finished. */
int32_t hpt_hip_stream_synchronize(int32_t dev, void* stream);
/* Block until everything queued on the device, on any stream, has finished. The reference's device
 * backend has one stream per device and synchronous copies (hpt/src/backends/cuda/tensor_impls.rs:142-169),
 * so it never needs this; here streams belong to the caller, and an owner of memory that was used on
 * a stream which no longer exists has only the whole device to wait for before the block is freed. */
int32_t hpt_hip_device_synchronize(int32_t dev);

/* ---- host-side shape logic ---------------------------------------------- */

/* process_axes (hpt-common/src/axis/axis.rs:38-73): negative axes wrap, an
 * axis outside 0..ndim is HPT_ERR_SHAPE, a repeated axis is HPT_ERR_PARAM.
 * Writes `naxes` normalised axes to `out`. */
int32_t hpt_hip_process_axes(const int64_t* axes, int32_t naxes, int32_t ndim, int64_t* out);

/* Layout::reduce (hpt-common/src/layout/layout_utils.rs:310-344): shape of the
 * result of reducing `axes` of `shape`; a full reduction without keep_dims
 * yields shape [1]. `out_shape` must hold max(ndim, 1) entries. */
int32_t hpt_hip_reduce_shape(const int64_t* shape, int32_t ndim, const int64_t* axes,
                             int32_t naxes, int32_t keep_dims, int64_t* out_shape,
                             int32_t* out_ndim);

/* Output dtype of a reduction: the input dtype for NormalReduce ops, bool for
 * all/any, FloatBinaryType<T> for FloatReduce ops
 * (hpt-types/src/promotion/normal_promote/_*.rs, impl_float_out_binary_promote). */
int32_t hpt_hip_reduce_out_dtype(int32_t op, int32_t in_dtype, int32_t* out_dtype);

/* Describe, without touching a device, which kernel family and launch shape
 * hpt_hip_reduce would use for this view and these axes. `buf` receives a short
 * text such as "row vec=4 tpr=256 rows=8192 cols=3136 split=1". */
int32_t hpt_hip_reduce_plan(int32_t op, const hpt_view* in, const int64_t* axes, int32_t naxes,
                            char* buf, size_t buflen);
/* Same for softmax/log_softmax (n_norm_dims = 0, axis given) and layernorm
 * (axis ignored, n_norm_dims trailing dims). */
int32_t hpt_hip_normalize_plan(const hpt_view* in, int64_t axis, int32_t n_norm_dims, char* buf,
                               size_t buflen);

/* ---- the hot path --------------------------------------------------------- */

/* Axis reduction. Replaces, for a Hip tensor, the device path behind
 * NormalReduce / FloatReduce / NormalEvalReduce / EvalReduce:
 * `reduce`, `reduce2`, `reduce3` (hpt/src/backends/cuda/tensor_internal/common_reduce.rs:30-47)
 * → `contiguous_reduce` / `uncontiguous_reduce`
 * (hpt/src/backends/cuda/utils/reduce/reduce.rs:641-838), CPU twin
 * hpt/src/backends/cpu/utils/reduce/reduce.rs:224-346.
 *   in      : any strided view (contiguous, permuted, sliced, stepped).
 *   axes    : axes to reduce (negative allowed); naxes == 0 reduces nothing.
 *   init_out: non-zero = overwrite `out`; zero = combine the reduction with the
 *             value already in `out` (the `sum_`/`nansum_` accumulate form,
 *             hpt-traits/src/ops/reduce.rs:84-92).
 *   out     : contiguous, dtype = hpt_hip_reduce_out_dtype(op, in->dtype), element
 *             count = product of the kept dims (keep_dims is a host-side reshape,
 *             hpt/src/backends/cpu/utils/reduce/reduce_template.rs:252). */
int32_t hpt_hip_reduce(int32_t dev, void* stream, int32_t op, const hpt_view* in,
                       const int64_t* axes, int32_t naxes, int32_t init_out, hpt_view* out);

/* hpt_hip_reduce for callers that cannot allocate device memory. It has no counterpart in
 * the reference: it is for code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc. Same arguments and results as hpt_hip_reduce (the
 * same kernels run), but the partial accumulators of a reduction that is split over
 * workgroups go to a static device array of HPT_HIP_STATIC_SCRATCH_BYTES that is part
 * of the library's image on every device, and the call makes no allocation of any kind.
 * A reduction whose partials need more than that is refused with HPT_ERR_MEMORY before
 * anything is launched (hpt_hip_reduce_plan shows the split: outputs x split x
 * accumulator size). Every call on one device shares that device's array, and nothing in
 * it has to start from a known value (each call writes what it reads): calls on
 * different streams of one device that overlap in time race; calls ordered by a
 * stream or by the host do not. The array's address is looked up on the first call on a
 * device: make that call outside any graph capture. */
#define HPT_HIP_STATIC_SCRATCH_BYTES (4u << 20)
int32_t hpt_hip_reduce_static(int32_t dev, void* stream, int32_t op, const hpt_view* in,
                              const int64_t* axes, int32_t naxes, int32_t init_out, hpt_view* out);

/* IndexReduce::argmax / argmin (hpt-traits/src/ops/reduce.rs:26,41; CPU
 * hpt/src/backends/cpu/utils/reduce/reduce.rs:45-170, 348-364 and
 * hpt/src/backends/cpu/kernels/argreduce_kernels.rs:2-71; device
 * hpt/src/backends/cuda/tensor_internal/arg_reduce.rs:18-63). One axis; the
 * result is the i64 position along that axis of the first maximum/minimum
 * (ties resolve to the lowest index, NaN never wins). `out` is contiguous i64. */
int32_t hpt_hip_argreduce(int32_t dev, void* stream, int32_t is_max, const hpt_view* in,
                          int64_t axis, hpt_view* out);

/* NormalizationOps::softmax / log_softmax (hpt-traits/src/ops/normalization.rs:51,64;
 * CPU hpt/src/backends/cpu/tensor_internal/normalization.rs:205-221 →
 * hpt/src/backends/cpu/kernels/normalization/softmax.rs:32-295, log_softmax.rs:33-298;
 * device hpt/src/backends/cuda/tensor_internal/softmax.rs:85-481). `in` may be
 * any strided view of a float dtype; `out` is contiguous with in's shape and
 * dtype. Half types are accumulated in f32 and rounded once. */
int32_t hpt_hip_softmax(int32_t dev, void* stream, int32_t log, const hpt_view* in, int64_t axis,
                        hpt_view* out);

/* NormalizationOps::layernorm (hpt-traits/src/ops/normalization.rs:30-37; CPU
 * hpt/src/backends/cpu/tensor_internal/normalization.rs:49-203; device
 * hpt/src/backends/cuda/tensor_internal/layernorm.rs:47-211 + layernorm_post).
 * Normalises over the trailing `n_norm_dims` dims with biased variance and
 * `eps` inside the square root, then applies gamma / beta (either may be NULL;
 * each is a contiguous tensor whose shape equals the normalised dims, same
 * dtype as `out`). `in` may be any strided view; `out` is contiguous. */
int32_t hpt_hip_layernorm(int32_t dev, void* stream, const hpt_view* in, int32_t n_norm_dims,
                          const hpt_view* gamma, const hpt_view* beta, double eps, hpt_view* out);

/* ---- fused forms of what the callers do around softmax / layernorm ---------
 * No trait of the reference has these signatures; they fuse the exact sequences its
 * transformer example runs (hpt-examples/examples/transformer/main.rs) and give the
 * results those sequences give. */

/* scores.mul_(scaling) -> fill -inf where key > query -> softmax(-1)
 * (hpt-examples/examples/transformer/main.rs:233-246, with the mask of :79 `tri`): the
 * causal mask is a PARAMETER, not data: row q of every (Q x K) matrix (Q = in.shape[ndim-2],
 * K = the last dim) keeps keys 0 .. q + causal_offset; the masked part of the input is never
 * read (its outputs are 0, or -inf for log). `scale` is rounded to in's dtype (the scalar
 * operand of `mul_` has it) and scale * x is rounded to in's dtype before the softmax, as
 * the separate `mul_` would have stored it. A row with no key left is NaN, like
 * softmax of a row of -inf. `in` any strided view of a float dtype with ndim >= 2, `out`
 * contiguous. */
int32_t hpt_hip_softmax_causal(int32_t dev, void* stream, int32_t log, const hpt_view* in, double scale,
                               int64_t causal_offset, hpt_view* out);

/* layernorm(x + residual) (hpt-examples/examples/transformer/main.rs:87-91): the sum is
 * rounded to the tensors' dtype, as the separate `+` would have stored it, then
 * normalised as hpt_hip_layernorm does. `residual`: contiguous, in's shape and dtype. */
int32_t hpt_hip_add_layernorm(int32_t dev, void* stream, const hpt_view* in, const hpt_view* residual,
                              int32_t n_norm_dims, const hpt_view* gamma, const hpt_view* beta, double eps,
                              hpt_view* out);

/* ---- the steps either side of the path ------------------------------------
 * What the callers of reductions and normalisations do to their operands just
 * before and after, kept on the device. */

/* Contiguous::contiguous (hpt-traits/src/ops/unary.rs:882; device
 * hpt/src/backends/cuda/tensor_internal/normal_out_unary.rs:286-310 launching
 * hpt-cudakernels/src/strided_copy.cu:6-14): copy any strided view into the
 * contiguous `out` of the same shape and dtype. This is also the first step of
 * `to_cpu` on a view (hpt/src/backends/cuda/tensor_impls.rs:154-160). */
int32_t hpt_hip_contiguous(int32_t dev, void* stream, const hpt_view* in, hpt_view* out);
/* Describes the kernel hpt_hip_contiguous would pick (tests, tuning). */
int32_t hpt_hip_contiguous_plan(const hpt_view* in, const hpt_view* out, char* buf, size_t buflen);

/* astype (hpt/src/backends/cuda/tensor_impls.rs:129-140; the cast every FloatReduce /
 * NormalizationOps entry applies to a non-float input, whose output dtype is
 * FloatBinaryType<T>: hpt-types/src/type_promote.rs): `in` any strided view, `out`
 * contiguous, same shape, a FLOAT dtype (or in's own dtype: a plain strided copy).
 * Integers convert as Rust's `as` does (nearest even; to f16 / bf16 through f32), floats
 * with one rounding. */
int32_t hpt_hip_cast(int32_t dev, void* stream, const hpt_view* in, hpt_view* out);

/* set_val (hpt-cudakernels/src/set_val.cu:4-12; used by `full` / `zeros` / `ones`,
 * hpt/src/backends/cuda/tensor_internal/normal_creation.rs): every element of the
 * contiguous `out` becomes `*value`, one element of out's dtype in HOST memory. */
int32_t hpt_hip_fill(int32_t dev, void* stream, hpt_view* out, const void* value);

typedef enum hpt_binary_op { HPT_BIN_ADD = 0, HPT_BIN_SUB = 1, HPT_BIN_MUL = 2, HPT_BIN_DIV = 3 } hpt_binary_op;

/* NormalBinOps::add_ / sub_ / mul_ / div_ (hpt-traits/src/ops/binary.rs:34,52,70,149;
 * device hpt/src/backends/cuda/utils/binary/binary_normal.rs:29-) for operands of ONE
 * dtype: out = lhs (op) rhs. `lhs` and `rhs` are strided views of out's shape; a
 * broadcast dim is passed with stride 0, as Hpt's `expand` produces it
 * (hpt-common/src/layout/layout_utils.rs `broadcast`). `out` is contiguous and may be
 * the very tensor `lhs` or `rhs` views (same data, shape and strides): the in-place
 * `add_` / `mul_` that layernorm's single-affine branches call
 * (hpt/src/backends/cpu/tensor_internal/normalization.rs:187-192). Integers wrap; bool
 * add is OR and mul is AND (sub / div undefined); div is for float dtypes (Hpt's
 * integer division changes the dtype). f16 / bf16 compute in f32 and round once.
 * An operand whose contiguous dim is not the innermost one (`b.t()`) is transposed
 * tile by tile inside the kernel; no operand is copied first. */
int32_t hpt_hip_binary(int32_t dev, void* stream, int32_t op, const hpt_view* lhs, const hpt_view* rhs,
                       hpt_view* out);
/* Describes the kernel hpt_hip_binary would pick (tests, tuning). */
int32_t hpt_hip_binary_plan(const hpt_view* lhs, const hpt_view* rhs, const hpt_view* out, char* buf, size_t buflen);

#ifdef __cplusplus
}
#endif
#endif /* HPT_HIP_H */
