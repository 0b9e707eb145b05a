/*
 * hpt_oracle.h — TEST INFRASTRUCTURE, not part of the product.
 *
 * A plain-C restatement, on the CPU, of the algorithms of Hpt's CPU backend for
 * the reduction / softmax / layernorm path, used as the checker in tests/, in
 * __graft_entry__.smoke() and as the "cpu_baseline" leg of bench.py. Nothing in
 * the shipped library (hpt_amd/, include/) may call into it.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the Hpt repository). What pins each function is listed in hpt_oracle.c.
 */
#ifndef HPT_ORACLE_H
#define HPT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype and op numbering: identical to hpt_dtype / hpt_reduce_op of the C ABI */
enum {
    ORC_BOOL = 0, ORC_I8, ORC_I16, ORC_I32, ORC_I64, ORC_U8, ORC_U16, ORC_U32, ORC_U64,
    ORC_F16, ORC_BF16, ORC_F32, ORC_F64
};
enum {
    ORC_SUM = 0, ORC_PROD, ORC_MAX, ORC_MIN, ORC_MEAN, ORC_NANSUM, ORC_NANPROD, ORC_REDUCEL1,
    ORC_REDUCEL2, ORC_REDUCEL3, ORC_SUM_SQUARE, ORC_LOGSUMEXP, ORC_ALL, ORC_ANY
};

/* How intermediate results are rounded.
 *   NATIVE: every operation is rounded to the type Hpt's CPU backend computes
 *           in (T for NormalReduce ops, FloatBinaryType<T> for the others):
 *           the literal CPU semantics, including f16/bf16 accumulators.
 *   F32   : f16/bf16 are widened to f32, every operation is rounded to f32 and
 *           the result is rounded to the output type once (what the north star
 *           calls "accumulated in f32"); other types as NATIVE.
 *   F64   : floating types accumulate in f64 and round once at the end
 *           (the "truth" the f32 tolerance is measured against).
 *   EXACT : as F64, and the additive reductions (sum, mean, nansum, reducel1/2/3,
 *           sum_square, logsumexp) add their terms without error (expansion
 *           arithmetic, as Python's math.fsum) and round the exact sum once: the
 *           truth for sums of millions of f64 terms, where a running f64 sum
 *           itself drifts. Reductions only.                                  */
enum { ORC_ACC_NATIVE = 0, ORC_ACC_F32 = 1, ORC_ACC_F64 = 2, ORC_ACC_EXACT = 3 };

typedef struct orc_view {
    const void* data;        /* already-offset element pointer */
    const int64_t* shape;
    const int64_t* strides;  /* in elements */
    int32_t ndim;
    int32_t dtype;
} orc_view;

/* ---- shape logic --------------------------------------------------------- */
int orc_process_axes(const int64_t* axes, int naxes, int ndim, int64_t* out, char* err, size_t errlen);
int orc_reduce_shape(const int64_t* shape, int ndim, const int64_t* axes, int naxes, int keep_dims,
                     int64_t* out_shape, int* out_ndim, char* err, size_t errlen);
void orc_shape_to_strides(const int64_t* shape, int ndim, int64_t* strides);
int orc_is_contiguous(const int64_t* shape, const int64_t* strides, int ndim);
int orc_coalesce_dims(const int64_t* shape, const int64_t* strides, int ndim, int* group_of_dim);
void orc_mt_intervals(int64_t size, int64_t nthreads, int64_t* out_pairs);
void orc_mt_intervals_simd(int64_t size, int64_t nthreads, int64_t vec, int64_t* out_pairs);
int orc_slice_process(const int64_t* shape, const int64_t* strides, int ndim, const int64_t* index,
                      int nindex, int64_t alpha, int64_t* out_shape, int64_t* out_strides,
                      int* out_ndim, int64_t* out_offset);
int orc_reduce_out_dtype(int op, int in_dtype);

/* ---- the hot path, restated ------------------------------------------------ */
/* `out` is contiguous in the kept dims' order. `lanes` > 1 restates the SIMD
 * accumulator structure of the contiguous row kernel. Returns 0 on success. */
int orc_reduce(int op, const orc_view* in, const int64_t* axes, int naxes, void* out, int acc_mode,
               int lanes);
int orc_argreduce(int is_max, const orc_view* in, int64_t axis, int64_t* out);
int orc_softmax(int log, const orc_view* in, int64_t axis, void* out, int acc_mode, int lanes);
int orc_layernorm(const orc_view* in, int n_norm_dims, const void* gamma, const void* beta,
                  double eps, void* out, int acc_mode);

/* ---- the timed "restated Hpt CPU path" (f32, contiguous rows, threads) ---- */
void orc_mt_layernorm_f32(const float* x, int64_t rows, int64_t cols, const float* gamma,
                          const float* beta, float eps, float* out, int nthreads);
void orc_mt_softmax_f32(const float* x, int64_t rows, int64_t cols, float* out, int log,
                        int nthreads);
void orc_mt_reduce_rows_f32(const float* x, int64_t rows, int64_t cols, float* out, int op,
                            int nthreads);
float orc_vexpf(float x); /* the polynomial exp used by the timed softmax */
int orc_physical_cores(void);

/* scalar conversions, exported for tests */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);

#ifdef __cplusplus
}
#endif
#endif
