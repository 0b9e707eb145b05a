/*
 * hpt_oracle.c — TEST INFRASTRUCTURE, not part of the product.
 *
 * CPU restatement of Hpt's CPU algorithms for axis reductions, arg-reductions,
 * softmax / log_softmax and layernorm. Hpt itself (Rust) cannot be built in
 * this pipeline, so each function below restates the reference source it
 * names and is pinned by the checks listed with it (tests/test_oracle_*.py):
 *
 *   function                 follows (Hpt repo)                                   pinned by
 *   orc_process_axes         hpt-common/src/axis/axis.rs:38-73                    KATs of hpt-tests/src/hpt_common/axis.rs:6-50
 *   orc_reduce_shape         hpt-common/src/layout/layout_utils.rs:310-344        brute force vs numpy shapes; full reduce -> [1]
 *   orc_is_contiguous        hpt-common/src/layout/layout_utils.rs:363-375        numpy flags on random views
 *   orc_coalesce_dims        hpt-common/src/layout/layout_utils.rs:384-410        hand-worked cases + offset-enumeration invariant
 *   orc_mt_intervals[_simd]  hpt-common/src/shape/shape_utils.rs:775-786,892-949  KATs of shape_utils.rs:718-760 docs and
 *                                                                                 hpt-tests/src/hpt_common/shape_utils.rs:12-52
 *   orc_slice_process        hpt-common/src/slice.rs:41-120                       doc KAT slice.rs:30-38; numpy slicing brute force
 *   orc_reduce (ints)        cpu/tensor_internal/common_reduce.rs:24-330,         bit-exact vs numpy wrap-around sums / min / max
 *                            hpt-types/src/scalars/impls.rs:28-75
 *   orc_reduce (floats)      cpu/kernels/reduce.rs:608-791,                       doc KATs hpt-traits/src/ops/reduce.rs:58-350; vs
 *                            hpt-types/src/vectors/utils.rs:83-105                numpy float64 sums; lane-structure invariants
 *   orc_reduce, ACC_EXACT    (no counterpart: the exactly summed f64 truth)        math.fsum: ill-conditioned sums (1e100 + 1 - 1e100), 1.3 M terms
 *   orc_argreduce            cpu/kernels/argreduce_kernels.rs:2-71                numpy argmax/argmin (first extremum), tie cases
 *   orc_softmax              cpu/kernels/softmax.rs:81-362,                       torch.softmax/log_softmax (float64) as the
 *                            cpu/kernels/normalization/logsoftmax.rs:81-364       reference's tests do; rows sum to 1; shift invariance
 *   orc_layernorm            cpu/tensor_internal/normalization.rs:49-203          torch layer_norm; constant rows -> beta; 2-element rows
 *   orc_mt_*_f32             same kernels, threaded with mt_intervals over        equality with orc_softmax / orc_layernorm /
 *                            physical cores (hpt/src/lib.rs:519-535)              orc_reduce on the same input
 *
 * Not pinnable without running Hpt (and therefore tolerance-only): the exact
 * f32 bit pattern of float sums, which in Hpt depends on the SIMD width chosen
 * at build time and, for full reductions, on rayon's split points.
 */
#define _GNU_SOURCE
#include "hpt_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#define ORC_MAX_RANK 32

/* ---- scalar conversions --------------------------------------------------- */

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, as the `half` crate's f16::from_f32 */
uint16_t orc_f32_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t exp = (u >> 23) & 0xff;
    uint32_t man = u & 0x7fffffu;
    if (exp == 255) return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e;
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) ++half_man;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1fffu;
    uint16_t r = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1))) ++r; /* may carry into exp: correct */
    return r;
}

float orc_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even with NaN quieting (hpt-types .../avx2/bf16x16.rs:60-85) */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static int dt_is_float(int dt) { return dt >= ORC_F16; }
static int dt_is_signed_int(int dt) { return dt >= ORC_I8 && dt <= ORC_I64; }

/* integer element as a sign/zero-extended 64-bit word */
static uint64_t load_u(const void* p, int dt, int64_t off) {
    switch (dt) {
        case ORC_BOOL: return ((const uint8_t*)p)[off] != 0;
        case ORC_I8: return (uint64_t)(int64_t)((const int8_t*)p)[off];
        case ORC_I16: return (uint64_t)(int64_t)((const int16_t*)p)[off];
        case ORC_I32: return (uint64_t)(int64_t)((const int32_t*)p)[off];
        case ORC_I64: return (uint64_t)((const int64_t*)p)[off];
        case ORC_U8: return ((const uint8_t*)p)[off];
        case ORC_U16: return ((const uint16_t*)p)[off];
        case ORC_U32: return ((const uint32_t*)p)[off];
        case ORC_U64: return ((const uint64_t*)p)[off];
        default: return 0;
    }
}
static void store_u(void* p, int dt, int64_t off, uint64_t v) {
    switch (dt) {
        case ORC_BOOL: ((uint8_t*)p)[off] = v != 0; break;
        case ORC_I8: case ORC_U8: ((uint8_t*)p)[off] = (uint8_t)v; break;
        case ORC_I16: case ORC_U16: ((uint16_t*)p)[off] = (uint16_t)v; break;
        case ORC_I32: case ORC_U32: ((uint32_t*)p)[off] = (uint32_t)v; break;
        default: ((uint64_t*)p)[off] = v; break;
    }
}
/* truncate a 64-bit word to the width of dt and re-extend (two's-complement wrap) */
static uint64_t wrap_u(int dt, uint64_t v) {
    switch (dt) {
        case ORC_BOOL: return v != 0;
        case ORC_I8: return (uint64_t)(int64_t)(int8_t)v;
        case ORC_I16: return (uint64_t)(int64_t)(int16_t)v;
        case ORC_I32: return (uint64_t)(int64_t)(int32_t)v;
        case ORC_U8: return (uint8_t)v;
        case ORC_U16: return (uint16_t)v;
        case ORC_U32: return (uint32_t)v;
        default: return v;
    }
}
/* any element as a double (`as f64` for 64-bit integers) */
static double load_f(const void* p, int dt, int64_t off) {
    switch (dt) {
        case ORC_F16: return orc_f16_to_f32(((const uint16_t*)p)[off]);
        case ORC_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[off]);
        case ORC_F32: return ((const float*)p)[off];
        case ORC_F64: return ((const double*)p)[off];
        case ORC_U64: return (double)((const uint64_t*)p)[off];
        default: return (double)(int64_t)load_u(p, dt, off);
    }
}
/* round a double to the precision of float dtype dt (identity for others) */
static double round_to(int dt, double v) {
    switch (dt) {
        case ORC_F16: return orc_f16_to_f32(orc_f32_to_f16((float)v));
        case ORC_BF16: return orc_bf16_to_f32(orc_f32_to_bf16((float)v));
        case ORC_F32: return (double)(float)v;
        default: return v;
    }
}
static void store_f(void* p, int dt, int64_t off, double v) {
    switch (dt) {
        case ORC_F16: ((uint16_t*)p)[off] = orc_f32_to_f16((float)v); break;
        case ORC_BF16: ((uint16_t*)p)[off] = orc_f32_to_bf16((float)v); break;
        case ORC_F32: ((float*)p)[off] = (float)v; break;
        case ORC_F64: ((double*)p)[off] = v; break;
        default: break;
    }
}
/* Note on double rounding: f16/bf16 values are produced as float(v) then
 * rounded to half. For sums, products, quotients and square roots of values
 * that are exact in the narrower type, rounding the double result first to f32
 * and then to half equals a single rounding (53 >= 2*24+2 and 24 >= 2*11+2),
 * which is also how the `half` crate computes (f32 op, then round). */

/* ---- shape logic --------------------------------------------------------- */

/* hpt-common/src/axis/axis.rs:38-73 */
int orc_process_axes(const int64_t* axes, int naxes, int ndim, int64_t* out, char* err,
                     size_t errlen) {
    for (int i = 0; i < naxes; ++i) {
        int64_t a = axes[i];
        for (int j = 0; j < i; ++j) {
            if (axes[j] == a) {
                if (err) snprintf(err, errlen, "Axis %lld is duplicated", (long long)a);
                return 1;
            }
        }
        int64_t v = a < 0 ? a + ndim : a;
        if (ndim > 0 && (v < 0 || v >= ndim)) {
            if (err)
                snprintf(err, errlen, "Dimension out of range: expected in 0..%d, got %lld", ndim,
                         (long long)v);
            return 2;
        }
        out[i] = v;
    }
    return 0;
}

/* hpt-common/src/layout/layout_utils.rs:310-344 */
int orc_reduce_shape(const int64_t* shape, int ndim, const int64_t* axes, int naxes, int keep_dims,
                     int64_t* out_shape, int* out_ndim, char* err, size_t errlen) {
    int64_t norm[ORC_MAX_RANK];
    int rc = orc_process_axes(axes, naxes, ndim, norm, err, errlen);
    if (rc) return rc;
    int n = 0;
    for (int i = 0; i < ndim; ++i) {
        int is_red = 0;
        for (int j = 0; j < naxes; ++j) is_red |= norm[j] == i;
        if (is_red) {
            if (keep_dims) out_shape[n++] = 1;
        } else {
            out_shape[n++] = shape[i];
        }
    }
    if (n == 0) out_shape[n++] = 1;
    *out_ndim = n;
    return 0;
}

void orc_shape_to_strides(const int64_t* shape, int ndim, int64_t* strides) {
    int64_t s = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        strides[i] = s;
        s *= shape[i];
    }
}

/* hpt-common/src/layout/layout_utils.rs:363-375 */
int orc_is_contiguous(const int64_t* shape, const int64_t* strides, int ndim) {
    int64_t expected = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        if (shape[i] == 0) continue;
        if (strides[i] != expected) return 0;
        expected *= shape[i];
    }
    return 1;
}

/* hpt-common/src/layout/layout_utils.rs:384-410: walk from the last dim; dim i
 * joins the current group when strides[i] == stride*size of the dim after it.
 * Writes the group id (0 = outermost group) of every dim; returns the number of groups. */
int orc_coalesce_dims(const int64_t* shape, const int64_t* strides, int ndim, int* group_of_dim) {
    if (ndim == 0) return 0;
    int rev[ORC_MAX_RANK];
    int g = 0;
    rev[ndim - 1] = 0;
    int64_t cur_stride = strides[ndim - 1], cur_size = shape[ndim - 1];
    for (int i = ndim - 2; i >= 0; --i) {
        if (strides[i] != cur_stride * cur_size) ++g;
        rev[i] = g;
        cur_stride = strides[i];
        cur_size = shape[i];
    }
    for (int i = 0; i < ndim; ++i) group_of_dim[i] = g - rev[i];
    return g + 1;
}

/* hpt-common/src/shape/shape_utils.rs:775-786 */
void orc_mt_intervals(int64_t size, int64_t nthreads, int64_t* out) {
    for (int64_t i = 0; i < nthreads; ++i) {
        int64_t q = size / nthreads, r = size % nthreads;
        int64_t start = i * q + (i < r ? i : r);
        int64_t end = start + q + (i < r ? 1 : 0);
        out[2 * i] = start;
        out[2 * i + 1] = end;
    }
}

/* hpt-common/src/shape/shape_utils.rs:892-949 */
void orc_mt_intervals_simd(int64_t size, int64_t nthreads, int64_t vec, int64_t* out) {
    int64_t aligned = (size / vec) * vec;
    int64_t rem = size - aligned;
    int64_t n = 0;
    if (aligned > 0) {
        int64_t blocks = aligned / vec;
        int64_t base = blocks / nthreads, extra = blocks % nthreads;
        int64_t start = 0;
        for (int64_t i = 0; i < nthreads; ++i) {
            int64_t b = base + (i < extra ? 1 : 0);
            int64_t end = start + b * vec;
            out[2 * n] = start;
            out[2 * n + 1] = end;
            ++n;
            start = end;
        }
        if (rem > 0) out[2 * (n - 1) + 1] += rem;
    }
    if (aligned == 0 && rem > 0) {
        out[0] = 0;
        out[1] = rem;
        for (int64_t i = 1; i < nthreads; ++i) out[2 * i] = out[2 * i + 1] = 0;
    } else if (aligned > 0) {
        for (; n < nthreads; ++n) out[2 * n] = out[2 * n + 1] = aligned;
    } else {
        for (; n < nthreads; ++n) out[2 * n] = out[2 * n + 1] = 0;
    }
}

/* hpt-common/src/slice.rs:41-120. `index` holds nindex (start, end, step)
 * triples; end == INT64_MAX means "to the end"; (0, 0, INT64_MAX) is an ellipsis. */
int orc_slice_process(const int64_t* shape, const int64_t* strides, int ndim, const int64_t* index,
                      int nindex, int64_t alpha, int64_t* out_shape, int64_t* out_strides,
                      int* out_ndim, int64_t* out_offset) {
    const int64_t BIG = 0x7FFFFFFFFFFFFFFFll;
    int64_t rshape[ORC_MAX_RANK], rstrides[ORC_MAX_RANK], idx[3 * ORC_MAX_RANK];
    if (nindex > ndim) return 1;
    for (int i = 0; i < ndim; ++i) {
        rshape[i] = shape[i] * alpha;
        rstrides[i] = strides[i] * alpha;
    }
    int ell = -1;
    for (int i = 0; i < nindex; ++i)
        if (index[3 * i] == 0 && index[3 * i + 1] == 0 && index[3 * i + 2] == BIG) {
            ell = i;
            break;
        }
    int n = 0;
    if (ell >= 0) {
        int missing = ndim - (nindex - 1);
        for (int i = 0; i < ell; ++i, ++n) memcpy(idx + 3 * n, index + 3 * i, 24);
        for (int i = 0; i < missing; ++i, ++n) {
            idx[3 * n] = 0;
            idx[3 * n + 1] = BIG;
            idx[3 * n + 2] = 1;
        }
        for (int i = ell + 1; i < nindex; ++i, ++n) memcpy(idx + 3 * n, index + 3 * i, 24);
    } else {
        memcpy(idx, index, (size_t)nindex * 24);
        n = nindex;
    }
    int64_t ptr = 0;
    for (int d = 0; d < n; ++d) {
        int64_t start = idx[3 * d], end = idx[3 * d + 1], step = idx[3 * d + 2];
        if (end == BIG) end = shape[d];
        if (start < 0) start += shape[d];
        if (end < 0) end += shape[d];
        if (start >= shape[d]) start = shape[d] - 1;
        if (end > shape[d]) end = shape[d];
        int64_t length = 0;
        if (step > 0) length = (end - start + step - 1) / step;
        else if (step < 0) length = (end - start + step + 1) / step;
        if (length > 0) {
            rshape[d] = length * alpha;
            ptr += start * rstrides[d];
            rstrides[d] *= step;
        } else {
            rshape[d] = 0;
        }
    }
    int m = 0;
    for (int i = 0; i < ndim; ++i) {
        if (rshape[i] == 0) continue;
        out_shape[m] = rshape[i];
        out_strides[m] = rstrides[i];
        ++m;
    }
    *out_ndim = m;
    *out_offset = ptr;
    return 0;
}

/* FloatBinaryType<T>: hpt-types/src/promotion/normal_promote/_*.rs (impl_float_out_binary_promote!(T, T, ..)) */
static int float_out_dtype(int dt) {
    switch (dt) {
        case ORC_BOOL: case ORC_I8: case ORC_I16: case ORC_U8: case ORC_U16: case ORC_F16: return ORC_F16;
        case ORC_I32: case ORC_U32: case ORC_F32: return ORC_F32;
        case ORC_BF16: return ORC_BF16;
        default: return ORC_F64;
    }
}

int orc_reduce_out_dtype(int op, int dt) {
    switch (op) {
        case ORC_MEAN: case ORC_REDUCEL2: case ORC_REDUCEL3: case ORC_LOGSUMEXP: return float_out_dtype(dt);
        case ORC_ALL: case ORC_ANY: return ORC_BOOL;
        default: return dt;
    }
}

/* the type arithmetic is rounded to, for a value type `vt` under an accumulate mode */
static int acc_dtype(int vt, int mode) {
    if (!dt_is_float(vt)) return vt;
    if (mode == ORC_ACC_F64 || mode == ORC_ACC_EXACT) return ORC_F64;
    if (mode == ORC_ACC_F32) return vt == ORC_F64 ? ORC_F64 : ORC_F32;
    return vt;
}

/* ---- iteration helpers ------------------------------------------------------ */

typedef struct {
    int n;
    int64_t size[ORC_MAX_RANK], stride[ORC_MAX_RANK], idx[ORC_MAX_RANK];
} odo;

static void odo_reset(odo* o) {
    for (int i = 0; i < o->n; ++i) o->idx[i] = 0;
}
/* advance; returns the change of offset, sets *done when wrapping to all-zero */
static int64_t odo_next(odo* o, int* done) {
    int64_t d = 0;
    for (int i = o->n - 1; i >= 0; --i) {
        if (o->idx[i] + 1 < o->size[i]) {
            ++o->idx[i];
            *done = 0;
            return d + o->stride[i];
        }
        d -= o->idx[i] * o->stride[i];
        o->idx[i] = 0;
    }
    *done = 1;
    return d;
}
static int64_t odo_count(const odo* o) {
    int64_t c = 1;
    for (int i = 0; i < o->n; ++i) c *= o->size[i];
    return c;
}

/* ---- reductions ------------------------------------------------------------- */

typedef struct {
    int op, in_dt, out_dt, acc_dt, is_int;
    double count_r; /* reduce size rounded to the accumulate type (mean) */
} rctx;

/* float path: identity, pre-op, combine, post-op (cpu/tensor_internal/common_reduce.rs:24-483) */
static double f_identity(const rctx* c) {
    switch (c->op) {
        case ORC_PROD: case ORC_NANPROD: return 1.0;
        case ORC_MAX: return -INFINITY;
        case ORC_MIN: return INFINITY;
        default: return 0.0;
    }
}
static double f_pre(const rctx* c, double x) {
    const int a = c->acc_dt;
    switch (c->op) {
        case ORC_NANSUM: return isnan(x) ? 0.0 : x;
        case ORC_NANPROD: return isnan(x) ? 1.0 : x;
        case ORC_REDUCEL1: return fabs(x);
        case ORC_SUM_SQUARE: return round_to(a, x * x);
        case ORC_MEAN: return round_to(a, x);
        case ORC_REDUCEL2: { double v = round_to(a, x); return round_to(a, v * v); }
        case ORC_REDUCEL3: { double v = round_to(a, fabs(x)); return round_to(a, pow(v, 3.0)); }
        case ORC_LOGSUMEXP: return round_to(a, exp(round_to(a, x)));
        default: return x;
    }
}
static double f_comb(const rctx* c, double a, double b) {
    switch (c->op) {
        case ORC_PROD: case ORC_NANPROD: return round_to(c->acc_dt, a * b);
        case ORC_MAX: return fmax(a, b); /* Rust f32::max ignores NaN: hpt-types/src/scalars/_f32.rs:55-57 */
        case ORC_MIN: return fmin(a, b);
        default: return round_to(c->acc_dt, a + b);
    }
}
static double f_post(const rctx* c, double a) {
    const int t = c->acc_dt;
    switch (c->op) {
        case ORC_MEAN: return round_to(t, a / c->count_r);
        case ORC_REDUCEL2: return round_to(t, sqrt(a));
        case ORC_REDUCEL3: return round_to(t, pow(a, round_to(t, 1.0 / 3.0)));
        case ORC_LOGSUMEXP: return round_to(t, log(a));
        default: return a;
    }
}

/* integer path: wrapping arithmetic (hpt-types/src/scalars/impls.rs:28-75), bool add = or, mul = and */
static uint64_t i_identity(const rctx* c) {
    const int dt = c->in_dt;
    switch (c->op) {
        case ORC_PROD: case ORC_NANPROD: return 1;
        case ORC_MAX:
            switch (dt) {
                case ORC_I8: return (uint64_t)(int64_t)INT8_MIN;
                case ORC_I16: return (uint64_t)(int64_t)INT16_MIN;
                case ORC_I32: return (uint64_t)(int64_t)INT32_MIN;
                case ORC_I64: return (uint64_t)INT64_MIN;
                default: return 0;
            }
        case ORC_MIN:
            switch (dt) {
                case ORC_BOOL: return 1;
                case ORC_I8: return INT8_MAX;
                case ORC_I16: return INT16_MAX;
                case ORC_I32: return INT32_MAX;
                case ORC_I64: return INT64_MAX;
                case ORC_U8: return UINT8_MAX;
                case ORC_U16: return UINT16_MAX;
                case ORC_U32: return UINT32_MAX;
                default: return UINT64_MAX;
            }
        case ORC_ALL: return 1;
        default: return 0;
    }
}
static uint64_t i_pre(const rctx* c, uint64_t x) {
    switch (c->op) {
        case ORC_REDUCEL1:
            if (dt_is_signed_int(c->in_dt) && (int64_t)x < 0) return wrap_u(c->in_dt, 0 - x);
            return x;
        case ORC_SUM_SQUARE: return c->in_dt == ORC_BOOL ? x : wrap_u(c->in_dt, x * x);
        case ORC_ALL: case ORC_ANY: return x != 0;
        default: return x;
    }
}
static uint64_t i_comb(const rctx* c, uint64_t a, uint64_t b) {
    const int dt = c->in_dt;
    const int sgn = dt_is_signed_int(dt);
    switch (c->op) {
        case ORC_PROD: case ORC_NANPROD: return dt == ORC_BOOL ? (a & b) : wrap_u(dt, a * b);
        case ORC_MAX:
            if (dt == ORC_BOOL) return a | b;
            return sgn ? ((int64_t)a > (int64_t)b ? a : b) : (a > b ? a : b);
        case ORC_MIN:
            if (dt == ORC_BOOL) return a & b;
            return sgn ? ((int64_t)a < (int64_t)b ? a : b) : (a < b ? a : b);
        case ORC_ALL: return a & b;
        case ORC_ANY: return a | b;
        default: return dt == ORC_BOOL ? (a | b) : wrap_u(dt, a + b);
    }
}

/* Exact summation of doubles (Shewchuk's expansions, the algorithm of Python's math.fsum): `p` holds
 * non-overlapping partials in increasing magnitude whose exact sum is the exact sum of everything added;
 * two-sum (hi = x + y, lo = y - (hi - x) with |x| >= |y|) moves each new term through them without error.
 * Non-finite terms are added apart, as IEEE would (inf + -inf = NaN). */
typedef struct {
    int n;
    double p[80];
    double special;
    int has_special;
} exact_sum;

static void exact_reset(exact_sum* e) {
    e->n = 0;
    e->special = 0.0;
    e->has_special = 0;
}
static void exact_add(exact_sum* e, double x) {
    if (!isfinite(x)) {
        e->special += x;
        e->has_special = 1;
        return;
    }
    int i = 0;
    for (int j = 0; j < e->n; ++j) {
        double y = e->p[j];
        if (fabs(x) < fabs(y)) {
            const double t = x;
            x = y;
            y = t;
        }
        const double hi = x + y;
        const double lo = y - (hi - x);
        if (lo != 0.0) e->p[i++] = lo;
        x = hi;
    }
    e->p[i++] = x;
    e->n = i;
}
static double exact_result(const exact_sum* e) {
    if (e->has_special) return e->special;
    int n = e->n;
    double hi = 0.0, lo = 0.0;
    if (n > 0) {
        hi = e->p[--n];
        while (n > 0) { /* add the partials from the largest down until one does not fit exactly */
            const double x = hi, y = e->p[--n];
            hi = x + y;
            lo = y - (hi - x);
            if (lo != 0.0) break;
        }
        /* half-way case: the rest of the partials decides the rounding direction */
        if (n > 0 && ((lo < 0.0 && e->p[n - 1] < 0.0) || (lo > 0.0 && e->p[n - 1] > 0.0))) {
            const double y = lo * 2.0, x = hi + y;
            if (y == x - hi) hi = x;
        }
    }
    return hi;
}

static int split_axes(const orc_view* in, const int64_t* axes, int naxes, odo* kept, odo* red) {
    int64_t norm[ORC_MAX_RANK];
    if (orc_process_axes(axes, naxes, in->ndim, norm, NULL, 0)) return 1;
    kept->n = red->n = 0;
    for (int i = 0; i < in->ndim; ++i) {
        int is_red = 0;
        for (int j = 0; j < naxes; ++j) is_red |= norm[j] == i;
        odo* o = is_red ? red : kept;
        o->size[o->n] = in->shape[i];
        o->stride[o->n] = in->strides[i];
        ++o->n;
    }
    odo_reset(kept);
    odo_reset(red);
    return 0;
}

int orc_reduce(int op, const orc_view* in, const int64_t* axes, int naxes, void* out, int acc_mode,
               int lanes) {
    odo kept, red;
    if (split_axes(in, axes, naxes, &kept, &red)) return 1;
    const int64_t K = odo_count(&kept), R = odo_count(&red);
    rctx c;
    c.op = op;
    c.in_dt = in->dtype;
    c.out_dt = orc_reduce_out_dtype(op, in->dtype);
    const int float_op = op == ORC_MEAN || op == ORC_REDUCEL2 || op == ORC_REDUCEL3 || op == ORC_LOGSUMEXP;
    const int bool_op = op == ORC_ALL || op == ORC_ANY;
    c.is_int = !float_op && (!dt_is_float(in->dtype) || bool_op);
    c.acc_dt = acc_dtype(float_op ? c.out_dt : in->dtype, acc_mode);
    c.count_r = round_to(c.acc_dt, (double)R);
    if (K == 0) return 0;

    /* the innermost reduced axis, when dense, is walked with `lanes` accumulators
     * folded in lane order (hpt-types/src/vectors/utils.rs:83-105) */
    const int lane_mode = lanes > 1 && red.n > 0 && red.stride[red.n - 1] == 1 && !c.is_int &&
                          !float_op && acc_mode != ORC_ACC_F64 && acc_mode != ORC_ACC_EXACT;
    /* ORC_ACC_EXACT: the additive ops keep the running sum as a list of non-overlapping f64 partials
     * (exact_sum below), so the result is the f64 nearest the exact sum of the terms whatever their
     * number or order: the truth does not drift the way a running f64 sum does */
    const int additive = op == ORC_SUM || op == ORC_MEAN || op == ORC_NANSUM || op == ORC_REDUCEL1 ||
                         op == ORC_REDUCEL2 || op == ORC_REDUCEL3 || op == ORC_SUM_SQUARE || op == ORC_LOGSUMEXP;
    const int exact = acc_mode == ORC_ACC_EXACT && additive && !c.is_int;
    const int64_t inner = red.n ? red.size[red.n - 1] : 1;

    int64_t koff = 0;
    for (int64_t o = 0; o < K; ++o) {
        if (c.is_int) {
            uint64_t acc = i_identity(&c);
            if (R > 0) {
                int64_t roff = 0;
                int done = 0;
                odo_reset(&red);
                while (!done) {
                    uint64_t x;
                    if (dt_is_float(in->dtype)) x = load_f(in->data, in->dtype, koff + roff) != 0.0; /* all/any of floats */
                    else x = load_u(in->data, in->dtype, koff + roff);
                    acc = i_comb(&c, acc, i_pre(&c, x));
                    roff += odo_next(&red, &done);
                }
            }
            store_u(out, c.out_dt, o, acc);
        } else {
            double acc = f_identity(&c);
            if (R > 0 && lane_mode) {
                odo outer = red;
                outer.n = red.n - 1;
                odo_reset(&outer);
                int64_t roff = 0;
                int done = 0;
                double lane[64];
                while (!done) {
                    const int64_t base = koff + roff;
                    const int64_t nvec = inner / lanes;
                    for (int l = 0; l < lanes; ++l) lane[l] = f_identity(&c);
                    for (int64_t v = 0; v < nvec; ++v)
                        for (int l = 0; l < lanes; ++l)
                            lane[l] = f_comb(&c, lane[l], f_pre(&c, load_f(in->data, in->dtype, base + v * lanes + l)));
                    double r = f_identity(&c);
                    for (int64_t i = nvec * lanes; i < inner; ++i)
                        r = f_comb(&c, r, f_pre(&c, load_f(in->data, in->dtype, base + i)));
                    for (int l = 0; l < lanes; ++l) r = f_comb(&c, r, lane[l]);
                    acc = f_comb(&c, acc, r);
                    if (outer.n == 0) break;
                    roff += odo_next(&outer, &done);
                }
            } else if (R > 0 && exact) {
                int64_t roff = 0;
                int done = 0;
                exact_sum es;
                exact_reset(&es);
                odo_reset(&red);
                while (!done) {
                    exact_add(&es, f_pre(&c, load_f(in->data, in->dtype, koff + roff)));
                    roff += odo_next(&red, &done);
                }
                acc = exact_result(&es);
            } else if (R > 0) {
                int64_t roff = 0;
                int done = 0;
                odo_reset(&red);
                while (!done) {
                    acc = f_comb(&c, acc, f_pre(&c, load_f(in->data, in->dtype, koff + roff)));
                    roff += odo_next(&red, &done);
                }
            }
            store_f(out, c.out_dt, o, f_post(&c, acc));
        }
        int kd;
        koff += odo_next(&kept, &kd);
    }
    return 0;
}

/* cpu/kernels/argreduce_kernels.rs:2-71: strict compare from NEG_INF/INF, index 0 */
int orc_argreduce(int is_max, const orc_view* in, int64_t axis, int64_t* out) {
    odo kept, red;
    if (split_axes(in, &axis, 1, &kept, &red)) return 1;
    const int64_t K = odo_count(&kept);
    const int64_t n = red.size[0], st = red.stride[0];
    const int is_f = dt_is_float(in->dtype);
    const int sgn = dt_is_signed_int(in->dtype);
    int64_t koff = 0;
    for (int64_t o = 0; o < K; ++o) {
        int64_t best = 0;
        if (is_f) {
            double bv = is_max ? -INFINITY : INFINITY;
            for (int64_t i = 0; i < n; ++i) {
                double v = load_f(in->data, in->dtype, koff + i * st);
                if (is_max ? v > bv : v < bv) {
                    bv = v;
                    best = i;
                }
            }
        } else {
            rctx c;
            c.op = is_max ? ORC_MAX : ORC_MIN;
            c.in_dt = in->dtype;
            uint64_t bv = i_identity(&c);
            for (int64_t i = 0; i < n; ++i) {
                uint64_t v = load_u(in->data, in->dtype, koff + i * st);
                int better = sgn ? (is_max ? (int64_t)v > (int64_t)bv : (int64_t)v < (int64_t)bv)
                                 : (is_max ? v > bv : v < bv);
                if (better) {
                    bv = v;
                    best = i;
                }
            }
        }
        out[o] = best;
        int kd;
        koff += odo_next(&kept, &kd);
    }
    return 0;
}

/* ---- softmax / log_softmax ---------------------------------------------------
 * Row kernel cpu/kernels/softmax.rs:204-319 (max; exp(x - max) stored and summed
 * in lanes; divide) and its strided / column variants :81-201, :322-489; the
 * log form cpu/kernels/normalization/logsoftmax.rs:203-320 (x - max stored, exp
 * summed, ln(sum) subtracted). Output is contiguous with the input's shape. */
int orc_softmax(int log_form, const orc_view* in, int64_t axis, void* out, int acc_mode, int lanes) {
    odo kept, red;
    if (!dt_is_float(in->dtype)) return 3;
    if (split_axes(in, &axis, 1, &kept, &red)) return 1;
    int64_t ax;
    orc_process_axes(&axis, 1, in->ndim, &ax, NULL, 0);
    int64_t ostr[ORC_MAX_RANK];
    orc_shape_to_strides(in->shape, in->ndim, ostr);
    odo okept;
    okept.n = 0;
    for (int i = 0; i < in->ndim; ++i)
        if (i != ax) {
            okept.size[okept.n] = in->shape[i];
            okept.stride[okept.n] = ostr[i];
            ++okept.n;
        }
    odo_reset(&okept);
    const int64_t K = odo_count(&kept), n = red.size[0], st = red.stride[0], ost = ostr[ax];
    const int dt = in->dtype;
    const int a = acc_dtype(dt, acc_mode);
    /* values parked in the output between passes are rounded to the output type
     * only in the literal mode; the other modes keep them in the compute type */
    const int park = acc_mode == ORC_ACC_NATIVE ? dt : a;
    if (K == 0 || n == 0) return 0;
    double* tmp = (double*)malloc(sizeof(double) * (size_t)n);
    if (!tmp) return 4;
    const int lane_mode = lanes > 1 && st == 1 && acc_mode != ORC_ACC_F64;
    int64_t koff = 0, ooff = 0;
    for (int64_t o = 0; o < K; ++o) {
        double mx = -INFINITY;
        for (int64_t i = 0; i < n; ++i) mx = fmax(mx, load_f(in->data, dt, koff + i * st));
        double lane[64];
        for (int l = 0; l < 64; ++l) lane[l] = 0.0;
        double tail = 0.0, seq = 0.0;
        const int64_t nvec = lane_mode ? n / lanes : 0;
        for (int64_t i = 0; i < n; ++i) {
            const double d = round_to(a, load_f(in->data, dt, koff + i * st) - mx);
            const double e = round_to(a, exp(d));
            const double parked = round_to(park, log_form ? d : e);
            tmp[i] = parked;
            const double addend = log_form ? e : parked;
            if (lane_mode) {
                if (i < nvec * lanes) lane[i % lanes] = round_to(a, lane[i % lanes] + addend);
                else tail = round_to(a, tail + addend);
            } else {
                seq = round_to(a, seq + addend);
            }
        }
        double sum = seq;
        if (lane_mode) {
            double vs = 0.0; /* vec_sum: hpt-types/src/vectors/utils.rs:70-79 */
            for (int l = 0; l < lanes; ++l) vs = round_to(a, vs + lane[l]);
            sum = round_to(a, tail + vs);
        }
        if (log_form) {
            const double ls = round_to(a, log(sum));
            for (int64_t i = 0; i < n; ++i) store_f(out, dt, ooff + i * ost, round_to(a, tmp[i] - ls));
        } else {
            for (int64_t i = 0; i < n; ++i) store_f(out, dt, ooff + i * ost, round_to(a, tmp[i] / sum));
        }
        int kd;
        koff += odo_next(&kept, &kd);
        ooff += odo_next(&okept, &kd);
    }
    free(tmp);
    return 0;
}

/* ---- layernorm -------------------------------------------------------------------
 * cpu/tensor_internal/normalization.rs:49-203: per row, sum -> mean; sum of
 * (x - mean)^2 -> biased variance; (x - mean) / sqrt(var + eps); then
 * gamma * y + beta (:185-202). All in FloatBinaryType<T> (= T for floats).
 * Only the mathematics is restated; the reference's pointer odometer is not. */
int orc_layernorm(const orc_view* in, int n_norm, const void* gamma, const void* beta, double eps,
                  void* out, int acc_mode) {
    if (!dt_is_float(in->dtype)) return 3;
    if (n_norm <= 0 || n_norm > in->ndim) return 1;
    odo kept, red;
    kept.n = red.n = 0;
    for (int i = 0; i < in->ndim; ++i) {
        odo* o = i >= in->ndim - n_norm ? &red : &kept;
        o->size[o->n] = in->shape[i];
        o->stride[o->n] = in->strides[i];
        ++o->n;
    }
    odo_reset(&kept);
    const int64_t K = odo_count(&kept), n = odo_count(&red);
    const int dt = in->dtype;
    const int a = acc_dtype(dt, acc_mode);
    const int park = acc_mode == ORC_ACC_NATIVE ? dt : a;
    if (K == 0 || n == 0) return 0;
    double* tmp = (double*)malloc(sizeof(double) * (size_t)n);
    if (!tmp) return 4;
    const double nr = round_to(a, (double)n);
    const double epsr = round_to(a, eps);
    int64_t koff = 0;
    for (int64_t o = 0; o < K; ++o) {
        int64_t roff = 0;
        int done = 0;
        odo_reset(&red);
        int64_t i = 0;
        double sum = 0.0;
        while (!done) {
            tmp[i] = round_to(a, load_f(in->data, dt, koff + roff));
            sum = round_to(a, sum + tmp[i]);
            ++i;
            roff += odo_next(&red, &done);
        }
        const double mean = round_to(a, sum / nr);
        double var = 0.0;
        for (i = 0; i < n; ++i) {
            const double d = round_to(a, tmp[i] - mean);
            var = round_to(a, var + round_to(a, d * d));
        }
        var = round_to(a, var / nr);
        const double den = round_to(a, sqrt(round_to(a, var + epsr)));
        for (i = 0; i < n; ++i) {
            double y = round_to(park, round_to(a, round_to(a, tmp[i] - mean) / den));
            if (gamma && beta) {
                y = round_to(a, round_to(a, load_f(gamma, dt, i) * y) + load_f(beta, dt, i));
            } else if (gamma) {
                y = round_to(a, y * load_f(gamma, dt, i));
            } else if (beta) {
                y = round_to(a, y + load_f(beta, dt, i));
            }
            store_f(out, dt, o * n + i, y);
        }
        int kd;
        koff += odo_next(&kept, &kd);
    }
    free(tmp);
    return 0;
}

/* ==== the timed "restated Hpt CPU path" =====================================
 * f32, contiguous [rows, cols]; rows are split over threads with mt_intervals
 * (hpt-common/src/shape/shape_utils.rs:775-786); Hpt sizes its pools with the
 * number of physical cores (hpt/src/lib.rs:519-535). Row kernels keep 8 lane
 * accumulators (an AVX2 f32x8, hpt-types/src/vectors/arch_simd/_256bit) and
 * fold them in lane order. */

#define LANES 8

int orc_physical_cores(void) {
    /* distinct (physical id, core id) pairs of /proc/cpuinfo; falls back to the online CPU count */
    FILE* f = fopen("/proc/cpuinfo", "r");
    long online = sysconf(_SC_NPROCESSORS_ONLN);
    if (online < 1) online = 1;
    if (!f) return (int)online;
    enum { MAXP = 4096 };
    static int seen[MAXP][2];
    int nseen = 0, phys = -1, core = -1;
    char line[512];
    while (fgets(line, sizeof line, f)) {
        int v;
        if (sscanf(line, "physical id : %d", &v) == 1) phys = v;
        else if (sscanf(line, "core id : %d", &v) == 1) core = v;
        else if (line[0] == '\n') {
            if (phys >= 0 && core >= 0) {
                int dup = 0;
                for (int i = 0; i < nseen; ++i) dup |= seen[i][0] == phys && seen[i][1] == core;
                if (!dup && nseen < MAXP) {
                    seen[nseen][0] = phys;
                    seen[nseen][1] = core;
                    ++nseen;
                }
            }
            phys = core = -1;
        }
    }
    fclose(f);
    if (nseen == 0 || nseen > online) return (int)online;
    return nseen;
}

/* A branch-free polynomial exp the compiler can vectorise (the role SLEEF's
 * xexpf plays for Hpt's vector path, hpt-types/.../sleef/libm/sleefsimdsp.rs:1061):
 * x = n*ln2 + r, |r| <= ln2/2, degree-6 polynomial, scale by 2^n. */
static inline float vexpf(float x) {
    const float log2e = 1.442695040888963f;
    const float ln2_hi = 0.693145751953125f, ln2_lo = 1.428606765330187e-06f;
    float xc = x < -103.0f ? -103.0f : (x > 88.7f ? 88.7f : x);
    float n = __builtin_roundf(xc * log2e);
    float r = (xc - n * ln2_hi) - n * ln2_lo;
    float p = 1.0f / 720.0f;
    p = p * r + 1.0f / 120.0f;
    p = p * r + 1.0f / 24.0f;
    p = p * r + 1.0f / 6.0f;
    p = p * r + 0.5f;
    p = p * r + 1.0f;
    p = p * r + 1.0f;
    /* 2^n in two steps so that n down to -149 stays representable */
    int ni = (int)n;
    int n1 = ni / 2, n2 = ni - n1;
    union { int32_t i; float f; } s1, s2;
    s1.i = (n1 + 127) << 23;
    s2.i = (n2 + 127) << 23;
    float res = p * s1.f * s2.f;
    return x < -104.0f ? 0.0f : res;
}
float orc_vexpf(float x) { return vexpf(x); }

typedef struct {
    const float *x, *gamma, *beta;
    float* out;
    int64_t r0, r1, cols;
    float eps;
    int flag;
} job_t;

static void* ln_worker(void* arg) {
    job_t* j = (job_t*)arg;
    const int64_t n = j->cols;
    for (int64_t r = j->r0; r < j->r1; ++r) {
        const float* x = j->x + r * n;
        float* y = j->out + r * n;
        /* three scalar passes, cpu/tensor_internal/normalization.rs:126-171 */
        float sum = 0.0f;
        for (int64_t i = 0; i < n; ++i) sum += x[i];
        const float mean = sum / (float)n;
        float var = 0.0f;
        for (int64_t i = 0; i < n; ++i) {
            float d = x[i] - mean;
            var += d * d;
        }
        var = var / (float)n;
        const float den = sqrtf(var + j->eps);
        for (int64_t i = 0; i < n; ++i) y[i] = (x[i] - mean) / den;
    }
    return NULL;
}
static void* affine_worker(void* arg) {
    job_t* j = (job_t*)arg;
    const int64_t n = j->cols;
    /* the separate affine pass over the whole result, normalization.rs:185-202 */
    for (int64_t r = j->r0; r < j->r1; ++r) {
        float* y = j->out + r * n;
        if (j->gamma && j->beta)
            for (int64_t i = 0; i < n; ++i) y[i] = j->gamma[i] * y[i] + j->beta[i];
        else if (j->gamma)
            for (int64_t i = 0; i < n; ++i) y[i] = y[i] * j->gamma[i];
        else if (j->beta)
            for (int64_t i = 0; i < n; ++i) y[i] = y[i] + j->beta[i];
    }
    return NULL;
}

static void run_rows(void* (*fn)(void*), job_t proto, int64_t rows, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    if (nthreads > rows) nthreads = rows > 0 ? (int)rows : 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
    job_t* jobs = (job_t*)malloc(sizeof(job_t) * (size_t)nthreads);
    int64_t* iv = (int64_t*)malloc(sizeof(int64_t) * 2 * (size_t)nthreads);
    orc_mt_intervals(rows, nthreads, iv);
    for (int t = 0; t < nthreads; ++t) {
        jobs[t] = proto;
        jobs[t].r0 = iv[2 * t];
        jobs[t].r1 = iv[2 * t + 1];
        if (t > 0) pthread_create(&th[t], NULL, fn, &jobs[t]);
    }
    fn(&jobs[0]);
    for (int t = 1; t < nthreads; ++t) pthread_join(th[t], NULL);
    free(th);
    free(jobs);
    free(iv);
}

void orc_mt_layernorm_f32(const float* x, int64_t rows, int64_t cols, const float* gamma,
                          const float* beta, float eps, float* out, int nthreads) {
    job_t j;
    memset(&j, 0, sizeof j);
    j.x = x;
    j.gamma = gamma;
    j.beta = beta;
    j.out = out;
    j.cols = cols;
    j.eps = eps;
    run_rows(ln_worker, j, rows, nthreads);
    if (gamma || beta) run_rows(affine_worker, j, rows, nthreads);
}

static inline float lanes_max(const float* x, int64_t n) {
    /* array_vec_reduce with max, hpt-types/src/vectors/utils.rs:83-105 */
    float lane[LANES];
    for (int l = 0; l < LANES; ++l) lane[l] = -INFINITY;
    const int64_t nv = n / LANES;
    for (int64_t v = 0; v < nv; ++v)
        for (int l = 0; l < LANES; ++l) {
            float t = x[v * LANES + l];
            lane[l] = lane[l] > t ? lane[l] : t;
        }
    float r = -INFINITY;
    for (int64_t i = nv * LANES; i < n; ++i) r = fmaxf(r, x[i]);
    for (int l = 0; l < LANES; ++l) r = fmaxf(r, lane[l]);
    return r;
}

static void* softmax_worker(void* arg) {
    job_t* j = (job_t*)arg;
    const int64_t n = j->cols, nv = n / LANES;
    const int log_form = j->flag;
    for (int64_t r = j->r0; r < j->r1; ++r) {
        const float* x = j->x + r * n;
        float* y = j->out + r * n;
        const float mx = lanes_max(x, n);
        float lane[LANES];
        for (int l = 0; l < LANES; ++l) lane[l] = 0.0f;
        for (int64_t v = 0; v < nv; ++v)
            for (int l = 0; l < LANES; ++l) {
                float d = x[v * LANES + l] - mx;
                float e = vexpf(d);
                y[v * LANES + l] = log_form ? d : e;
                lane[l] += e;
            }
        float sum = 0.0f;
        for (int64_t i = nv * LANES; i < n; ++i) { /* scalar tail uses libm, softmax.rs:247-252 */
            float d = x[i] - mx;
            float e = expf(d);
            y[i] = log_form ? d : e;
            sum += e;
        }
        float vs = 0.0f;
        for (int l = 0; l < LANES; ++l) vs += lane[l];
        sum += vs;
        if (log_form) {
            const float ls = logf(sum);
            for (int64_t i = 0; i < n; ++i) y[i] = y[i] - ls;
        } else {
            for (int64_t i = 0; i < n; ++i) y[i] = y[i] / sum;
        }
    }
    return NULL;
}

void orc_mt_softmax_f32(const float* x, int64_t rows, int64_t cols, float* out, int log_form,
                        int nthreads) {
    job_t j;
    memset(&j, 0, sizeof j);
    j.x = x;
    j.out = out;
    j.cols = cols;
    j.flag = log_form;
    run_rows(softmax_worker, j, rows, nthreads);
}

static void* reduce_rows_worker(void* arg) {
    job_t* j = (job_t*)arg;
    const int64_t n = j->cols, nv = n / LANES;
    const int op = j->flag;
    for (int64_t r = j->r0; r < j->r1; ++r) {
        const float* x = j->x + r * n;
        if (op == ORC_MAX) {
            j->out[r] = lanes_max(x, n);
            continue;
        }
        float lane[LANES];
        for (int l = 0; l < LANES; ++l) lane[l] = 0.0f;
        for (int64_t v = 0; v < nv; ++v)
            for (int l = 0; l < LANES; ++l) lane[l] += x[v * LANES + l];
        float s = 0.0f;
        for (int64_t i = nv * LANES; i < n; ++i) s += x[i];
        for (int l = 0; l < LANES; ++l) s += lane[l];
        j->out[r] = op == ORC_MEAN ? s / (float)n : s;
    }
    return NULL;
}

/* row sums / means / maxima: cpu/kernels/reduce.rs:608-658 */
void orc_mt_reduce_rows_f32(const float* x, int64_t rows, int64_t cols, float* out, int op,
                            int nthreads) {
    job_t j;
    memset(&j, 0, sizeof j);
    j.x = x;
    j.out = out;
    j.cols = cols;
    j.flag = op;
    run_rows(reduce_rows_worker, j, rows, nthreads);
}
