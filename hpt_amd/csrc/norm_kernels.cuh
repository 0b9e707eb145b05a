// Softmax, log_softmax and layernorm kernels of libhpt_hip.
//
//   row_reg_kernel     a row of the output is contiguous and the input row has
//                      a small stride: `tpr` threads load the row ONCE into
//                      registers (128-bit loads when the stride is 1), compute
//                      the row statistics with cross-lane shuffles (and LDS
//                      above one wavefront) and write the result: one HBM read
//                      and one HBM write per element.
//   row_stream_kernel  any layout and any row length: a first sweep computes
//                      the statistics online (running max + rescaled sum for
//                      softmax, Welford mean/M2 with Chan's merge for
//                      layernorm), a second sweep re-reads the row and writes.
//                      With tpr == 1 every lane owns a row, which is the
//                      coalesced mapping when the normalised axis is not the
//                      innermost one.
//
// Semantics follow the CPU reference: softmax = exp(x - max) / sum
// (hpt/src/backends/cpu/kernels/softmax.rs:204-319), log_softmax = x - max -
// ln(sum) (hpt/src/backends/cpu/kernels/normalization/logsoftmax.rs:203-320),
// layernorm = (x - mean) / sqrt(biased_var + eps) * gamma + beta
// (hpt/src/backends/cpu/tensor_internal/normalization.rs:126-201). f16/bf16
// are computed in f32 and rounded once on the store; f64 in f64. One
// reciprocal per row replaces the per-element division.
#pragma once

#include "device_utils.cuh"
#include "norm_entry.hpp"

namespace hpt {

template <class CT> struct MaxC {
    __device__ static __forceinline__ CT comb(CT a, CT b) {
        if constexpr (sizeof(CT) == 8) return fmax(a, b);
        else return fmaxf(a, b);
    }
};
template <class CT> struct SumC {
    __device__ static __forceinline__ CT comb(CT a, CT b) { return a + b; }
};

// exp / log in the compute type. f32 tensors use the accurate library
// routines (tolerance 1e-5 against the CPU path); half tensors, whose results
// are rounded to 8 or 11 significant bits anyway, use the hardware exp2/log2.
template <class T> __device__ __forceinline__ float exp_ct(float x) {
    if constexpr (sizeof(T) == 2) return __expf(x);
    else return expf(x);
}
template <class T> __device__ __forceinline__ double exp_ct(double x) { return exp(x); }
template <class T> __device__ __forceinline__ float log_ct(float x) {
    if constexpr (sizeof(T) == 2) return __logf(x);
    else return logf(x);
}
template <class T> __device__ __forceinline__ double log_ct(double x) { return log(x); }
__device__ __forceinline__ float rsqrt_ct(float x) { return 1.0f / sqrtf(x); }
__device__ __forceinline__ double rsqrt_ct(double x) { return 1.0 / sqrt(x); }

template <class CT> __device__ __forceinline__ CT neg_inf() {
    if constexpr (sizeof(CT) == 8) return -__builtin_huge_val();
    else return -__builtin_huge_valf();
}

// type the layernorm row statistics are accumulated in
template <class T> struct StatType { using type = float; };
template <> struct StatType<float> { using type = double; };
template <> struct StatType<double> { using type = double; };

template <class Op, class CT>
__device__ __forceinline__ CT row_all_reduce(CT v, int tpr, CT* smem) {
    if (tpr <= 64) return group_reduce<Op>(v, tpr);
    return block_reduce<Op>(v, smem);
}

// ---- rows held in registers ---------------------------------------------------
template <int KIND, class T, int VEC, int NCHUNK>
__global__ void __launch_bounds__(1024) row_reg_kernel(const NormArgs a) {
    using CT = typename Elem<T>::Wide;
    __shared__ __align__(8) unsigned char smem_stat[16 * sizeof(double)];
    CT* smem = reinterpret_cast<CT*>(smem_stat);
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int64_t row = (int64_t)blockIdx.x * a.rpb + ty;
    const bool valid = row < a.rows;
    const int64_t nv = a.cols / VEC;
    const T* in_row = (const T*)a.in + (valid ? offset_of(a.kept_in, row) : 0);
    T* out_row = (T*)a.out + (valid ? row * a.cols : 0);

    CT x[NCHUNK][VEC];
    constexpr bool kSoft = KIND != NORM_LAYERNORM;
    const CT fill = kSoft ? neg_inf<CT>() : (CT)0;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int64_t iv = (int64_t)c * tpr + tx;
        if (valid && iv < nv) {
            if constexpr (VEC > 1) {
                Pack<T, VEC> v = load_pack<T, VEC>(in_row + iv * VEC);
#pragma unroll
                for (int j = 0; j < VEC; ++j) x[c][j] = Elem<T>::widen(v.v[j]);
            } else {
                x[c][0] = Elem<T>::widen(in_row[iv * a.sa]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[c][j] = fill;
        }
    }

    if constexpr (kSoft) {
        CT m = neg_inf<CT>();
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int j = 0; j < VEC; ++j) m = MaxC<CT>::comb(m, x[c][j]);
        m = row_all_reduce<MaxC<CT>>(m, tpr, smem);
        CT s = 0;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                CT d = x[c][j] - m;
                CT e = exp_ct<T>(d);
                s += e;
                x[c][j] = KIND == NORM_SOFTMAX ? e : d;
            }
        s = row_all_reduce<SumC<CT>>(s, tpr, smem);
        const CT k = KIND == NORM_SOFTMAX ? (CT)1 / s : log_ct<T>(s);
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[c][j] = KIND == NORM_SOFTMAX ? x[c][j] * k : x[c][j] - k;
    } else {
        // Row statistics of f32 (and f64) rows are taken in f64: x - mean is then
        // exact before it is rounded, so rows whose spread is small against
        // their offset keep full f32 accuracy. Half types use f32.
        using ST = typename StatType<T>::type;
        ST* ssmem = reinterpret_cast<ST*>(smem_stat);
        ST s = 0;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += (ST)x[c][j];
        s = row_all_reduce<SumC<ST>>(s, tpr, ssmem);
        const ST mean = s / (ST)a.cols;
        ST q = 0;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const bool in_row_c = ((int64_t)c * tpr + tx) < nv;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const ST d = in_row_c ? (ST)x[c][j] - mean : (ST)0;
                x[c][j] = (CT)d;
                q += d * d;
            }
        }
        q = row_all_reduce<SumC<ST>>(q, tpr, ssmem);
        const CT rstd = (CT)rsqrt_ct(q / (ST)a.cols + (ST)a.eps);
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int64_t iv = (int64_t)c * tpr + tx;
            if (iv < nv) {
                if constexpr (VEC > 1) {
                    if (a.gamma) {
                        Pack<T, VEC> g = load_pack<T, VEC>((const T*)a.gamma + iv * VEC);
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[c][j] = x[c][j] * rstd * Elem<T>::widen(g.v[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[c][j] *= rstd;
                    }
                    if (a.beta) {
                        Pack<T, VEC> b = load_pack<T, VEC>((const T*)a.beta + iv * VEC);
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[c][j] += Elem<T>::widen(b.v[j]);
                    }
                } else {
                    CT y = x[c][0] * rstd;
                    if (a.gamma) y *= Elem<T>::widen(((const T*)a.gamma)[iv]);
                    if (a.beta) y += Elem<T>::widen(((const T*)a.beta)[iv]);
                    x[c][0] = y;
                }
            }
        }
    }

    if (!valid) return;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int64_t iv = (int64_t)c * tpr + tx;
        if (iv < nv) {
            if constexpr (VEC > 1) {
                Pack<T, VEC> o;
#pragma unroll
                for (int j = 0; j < VEC; ++j) o.v[j] = Elem<T>::narrow(x[c][j]);
                store_pack<T, VEC>(out_row + iv * VEC, o);
            } else {
                out_row[iv] = Elem<T>::narrow(x[c][0]);
            }
        }
    }
}

// ---- streaming rows: online statistics, then a second sweep ------------------

// running (max, sum of exp(x - max))
template <class CT> struct SoftStat {
    CT m, s;
};
template <class T, class CT> struct SoftStatOp {
    __device__ static __forceinline__ SoftStat<CT> comb(SoftStat<CT> a, SoftStat<CT> b) {
        SoftStat<CT> r;
        r.m = MaxC<CT>::comb(a.m, b.m);
        // a side that has seen nothing (m = -inf, s = 0) must not produce inf - inf
        CT sa = a.s == (CT)0 ? (CT)0 : a.s * exp_ct<T>(a.m - r.m);
        CT sb = b.s == (CT)0 ? (CT)0 : b.s * exp_ct<T>(b.m - r.m);
        r.s = sa + sb;
        return r;
    }
};
// running (count, mean, sum of squared deviations)
template <class CT> struct MomentStat {
    CT n, mean, m2;
};
template <class CT> struct MomentStatOp {
    __device__ static __forceinline__ MomentStat<CT> comb(MomentStat<CT> a, MomentStat<CT> b) {
        MomentStat<CT> r;
        r.n = a.n + b.n;
        if (r.n == (CT)0) {
            r.mean = 0;
            r.m2 = 0;
            return r;
        }
        const CT d = b.mean - a.mean;
        const CT f = b.n / r.n;
        r.mean = a.mean + d * f;
        r.m2 = a.m2 + b.m2 + d * d * a.n * f;
        return r;
    }
};

template <class Op, class S> __device__ __forceinline__ S stat_all_reduce(S v, int tpr, S* smem) {
    if (tpr == 1) return v;
    if (tpr <= 64) return group_reduce<Op>(v, tpr);
    return block_reduce<Op>(v, smem);
}

template <int KIND, class T, int VEC>
__global__ void __launch_bounds__(1024) row_stream_kernel(const NormArgs a) {
    using CT = typename Elem<T>::Wide;
    __shared__ __align__(16) unsigned char smem_raw[16 * 3 * sizeof(double)];
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int64_t row = (int64_t)blockIdx.x * a.rpb + ty;
    const bool valid = row < a.rows;
    const int64_t nv = a.cols / VEC;
    const T* in_row = (const T*)a.in + (valid ? offset_of(a.kept_in, row) : 0);
    T* out_row = (T*)a.out + (valid ? offset_of(a.kept_out, row) : 0);
    const bool one_dim = a.norm_in.n <= 1;

    auto load = [&](int64_t iv, CT* x) {
        if constexpr (VEC > 1) {
            Pack<T, VEC> v = load_pack<T, VEC>(in_row + iv * VEC);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[j] = Elem<T>::widen(v.v[j]);
        } else {
            const int64_t off = one_dim ? iv * a.sa : offset_of(a.norm_in, iv);
            x[0] = Elem<T>::widen(in_row[off]);
        }
    };
    auto store = [&](int64_t iv, const CT* y) {
        if constexpr (VEC > 1) {
            Pack<T, VEC> o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o.v[j] = Elem<T>::narrow(y[j]);
            store_pack<T, VEC>(out_row + iv * VEC, o);
        } else {
            out_row[iv * a.out_axis_stride] = Elem<T>::narrow(y[0]);
        }
    };

    if constexpr (KIND != NORM_LAYERNORM) {
        SoftStat<CT> st{neg_inf<CT>(), (CT)0};
        if (valid) {
            for (int64_t iv = tx; iv < nv; iv += tpr) {
                CT x[VEC];
                load(iv, x);
                CT cm = x[0];
#pragma unroll
                for (int j = 1; j < VEC; ++j) cm = MaxC<CT>::comb(cm, x[j]);
                if (cm > st.m) {
                    st.s = st.s == (CT)0 ? (CT)0 : st.s * exp_ct<T>(st.m - cm);
                    st.m = cm;
                }
                if (st.m > neg_inf<CT>()) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) st.s += exp_ct<T>(x[j] - st.m);
                }
            }
        }
        st = stat_all_reduce<SoftStatOp<T, CT>>(st, tpr, (SoftStat<CT>*)smem_raw);
        if (!valid) return;
        const CT k = KIND == NORM_SOFTMAX ? (CT)1 / st.s : log_ct<T>(st.s);
        for (int64_t iv = tx; iv < nv; iv += tpr) {
            CT x[VEC];
            load(iv, x);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                CT d = x[j] - st.m;
                x[j] = KIND == NORM_SOFTMAX ? exp_ct<T>(d) * k : d - k;
            }
            store(iv, x);
        }
    } else {
        using ST = typename StatType<T>::type;
        MomentStat<ST> st{(ST)0, (ST)0, (ST)0};
        if (valid) {
            // Per thread: sums of (x - k) and (x - k)^2 around the first element k
            // it sees (no division per element, no cancellation against a far
            // origin), turned into (count, mean, M2) once at the end.
            ST k = 0, s1 = 0, s2 = 0, n = 0;
            bool first = true;
            for (int64_t iv = tx; iv < nv; iv += tpr) {
                CT x[VEC];
                load(iv, x);
                if (first) {
                    k = (ST)x[0];
                    first = false;
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const ST d = (ST)x[j] - k;
                    s1 += d;
                    s2 += d * d;
                }
                n += (ST)VEC;
            }
            if (n > (ST)0) {
                st.n = n;
                st.mean = k + s1 / n;
                st.m2 = s2 - s1 * s1 / n;
                if (st.m2 < (ST)0) st.m2 = 0;
            }
        }
        st = stat_all_reduce<MomentStatOp<ST>>(st, tpr, (MomentStat<ST>*)smem_raw);
        if (!valid) return;
        const ST mean = st.mean;
        const CT rstd = (CT)rsqrt_ct(st.m2 / (ST)a.cols + (ST)a.eps);
        for (int64_t iv = tx; iv < nv; iv += tpr) {
            CT x[VEC];
            load(iv, x);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                CT y = (CT)((ST)x[j] - mean) * rstd;
                const int64_t col = iv * VEC + j;
                if (a.gamma) y *= Elem<T>::widen(((const T*)a.gamma)[col]);
                if (a.beta) y += Elem<T>::widen(((const T*)a.beta)[col]);
                x[j] = y;
            }
            store(iv, x);
        }
    }
}

}  // namespace hpt
