// The reduction operators: for each op of the reference's reduce traits, the
// accumulator type, identity, per-element pre-op, combine and post-op.
//
// Op tables follow hpt/src/backends/cpu/tensor_internal/common_reduce.rs:24-483
// (sum: init 0, a+b; prod: init 1, a*b; max: init NEG_INF; min: init INF;
// reducel1: |a|; sum_square: a*a; nansum/nanprod: NaN -> identity; all/any:
// is_true with &/|; mean/reducel2/reducel3/logsumexp: cast to FloatBinaryType,
// then /count, sqrt, pow(1/3), ln). Half types accumulate in f32 and are
// rounded once when the result is stored.
#pragma once

#include "device_utils.hpp"

namespace hpt {

template <class T> struct Limits;
#define HPT_LIMITS(T, LO, HI)                                                \
    template <> struct Limits<T> {                                           \
        __device__ static __forceinline__ T lowest() { return LO; }          \
        __device__ static __forceinline__ T highest() { return HI; }         \
    };
// NEG_INF / INF of integer types are MIN / MAX (hpt-types/src/dtype.rs:235-238, 396-409)
HPT_LIMITS(int32_t, INT32_MIN, INT32_MAX)
HPT_LIMITS(uint32_t, 0u, UINT32_MAX)
HPT_LIMITS(int64_t, INT64_MIN, INT64_MAX)
HPT_LIMITS(uint64_t, 0ull, UINT64_MAX)
HPT_LIMITS(float, -__builtin_huge_valf(), __builtin_huge_valf())
HPT_LIMITS(double, -__builtin_huge_val(), __builtin_huge_val())
#undef HPT_LIMITS

// lowest/highest value of element type T, expressed in its compare type
template <class T> struct ElemRange {
    using C = typename Elem<T>::Cmp;
    __device__ static __forceinline__ C lowest() { return Limits<C>::lowest(); }
    __device__ static __forceinline__ C highest() { return Limits<C>::highest(); }
};
#define HPT_RANGE(T, LO, HI)                                                 \
    template <> struct ElemRange<T> {                                        \
        using C = typename Elem<T>::Cmp;                                     \
        __device__ static __forceinline__ C lowest() { return LO; }          \
        __device__ static __forceinline__ C highest() { return HI; }         \
    };
HPT_RANGE(int8_t, INT8_MIN, INT8_MAX)
HPT_RANGE(int16_t, INT16_MIN, INT16_MAX)
HPT_RANGE(uint8_t, 0u, UINT8_MAX)
HPT_RANGE(uint16_t, 0u, UINT16_MAX)
HPT_RANGE(bool8, 0u, 1u)
#undef HPT_RANGE

// FloatBinaryType<T> (hpt-types/src/promotion/normal_promote/_*.rs)
// Accumulator of the additive ops. f32 (and the integer types whose float
// type is f32) accumulate in f64: the kernels are HBM-bound, f64 adds run at
// full rate, and the stored f32 is then the correctly rounded sum whatever the
// summation order, so multi-stage results do not depend on the launch shape.
// f16/bf16 accumulate in f32 and are rounded once.
template <class T> struct SumAcc { using type = typename Elem<T>::Wide; };
template <> struct SumAcc<float> { using type = double; };

template <class T> struct FloatOut { using type = T; using acc = typename SumAcc<T>::type; };
template <> struct FloatOut<bool8> { using type = f16_t; using acc = float; };
template <> struct FloatOut<int8_t> { using type = f16_t; using acc = float; };
template <> struct FloatOut<int16_t> { using type = f16_t; using acc = float; };
template <> struct FloatOut<uint8_t> { using type = f16_t; using acc = float; };
template <> struct FloatOut<uint16_t> { using type = f16_t; using acc = float; };
template <> struct FloatOut<int32_t> { using type = float; using acc = double; };
template <> struct FloatOut<uint32_t> { using type = float; using acc = double; };
template <> struct FloatOut<int64_t> { using type = double; using acc = double; };
template <> struct FloatOut<uint64_t> { using type = double; using acc = double; };

template <class T, class F> __device__ __forceinline__ F to_float_acc(T x) {
    if constexpr (Elem<T>::is_float) return (F)Elem<T>::widen(x);
    else return (F)Elem<T>::cmp(x);
}

// NaN-ignoring max/min for floats (Rust f32::max/min, hpt-types/src/scalars/_f32.rs:55-57)
template <class C> __device__ __forceinline__ C cmax(C a, C b) {
    if constexpr (__is_floating_point(C)) return __builtin_fmax(a, b);
    else return a > b ? a : b;
}
template <class C> __device__ __forceinline__ C cmin(C a, C b) {
    if constexpr (__is_floating_point(C)) return __builtin_fmin(a, b);
    else return a < b ? a : b;
}
template <> __device__ __forceinline__ float cmax<float>(float a, float b) { return fmaxf(a, b); }
template <> __device__ __forceinline__ float cmin<float>(float a, float b) { return fminf(a, b); }
template <> __device__ __forceinline__ double cmax<double>(double a, double b) { return fmax(a, b); }
template <> __device__ __forceinline__ double cmin<double>(double a, double b) { return fmin(a, b); }

// ---- same-dtype ops: sum, prod, nansum, nanprod, reducel1, sum_square --------
template <int OP, class T> struct ArithOp {
    using In = T;
    using Out = T;
    using Wide = typename Elem<T>::Wide;
    using Acc = typename SumAcc<T>::type;
    static constexpr bool is_mul = (OP == HPT_PROD || OP == HPT_NANPROD);
    __device__ static __forceinline__ Acc identity() {
        if constexpr (Elem<T>::is_bool) return is_mul ? 1u : 0u;
        else return is_mul ? (Acc)1 : (Acc)0;
    }
    __device__ static __forceinline__ Acc pre(T x, int64_t) {
        Acc w = (Acc)Elem<T>::widen(x);
        if constexpr (OP == HPT_NANSUM || OP == HPT_NANPROD) {
            if (Elem<T>::is_nan(x)) return identity();
            return w;
        } else if constexpr (OP == HPT_REDUCEL1) {
            if constexpr (Elem<T>::is_float) return w < 0 ? -w : w;
            else if constexpr (Elem<T>::is_signed) {
                auto c = Elem<T>::cmp(x);
                return (Acc)(c < 0 ? (Acc)0 - (Acc)c : (Acc)c);
            } else return w;
        } else if constexpr (OP == HPT_SUM_SQUARE) {
            if constexpr (Elem<T>::is_bool) return w;
            else return w * w;
        } else {
            return w;
        }
    }
    __device__ static __forceinline__ Acc comb(Acc a, Acc b) {
        if constexpr (Elem<T>::is_bool) return is_mul ? (a & b) : (a | b);
        else return is_mul ? a * b : a + b;
    }
    __device__ static __forceinline__ Out post(Acc a, double) { return Elem<T>::narrow((Wide)a); }
    __device__ static __forceinline__ Acc from_out(Out o) { return (Acc)Elem<T>::widen(o); }
};

// ---- max / min ----------------------------------------------------------------
template <int OP, class T> struct MinMaxOp {
    using In = T;
    using Out = T;
    using Acc = typename Elem<T>::Cmp;
    __device__ static __forceinline__ Acc identity() {
        return OP == HPT_MAX ? ElemRange<T>::lowest() : ElemRange<T>::highest();
    }
    __device__ static __forceinline__ Acc pre(T x, int64_t) { return Elem<T>::cmp(x); }
    __device__ static __forceinline__ Acc comb(Acc a, Acc b) {
        return OP == HPT_MAX ? cmax<Acc>(a, b) : cmin<Acc>(a, b);
    }
    __device__ static __forceinline__ Out post(Acc a, double) { return Elem<T>::from_cmp(a); }
    __device__ static __forceinline__ Acc from_out(Out o) { return Elem<T>::cmp(o); }
};

// ---- float-output ops: mean, reducel2, reducel3, logsumexp -----------------------
template <int OP, class T> struct FloatOp {
    using In = T;
    using Out = typename FloatOut<T>::type;
    using Acc = typename FloatOut<T>::acc;
    using OutWide = typename Elem<Out>::Wide;  // the precision the reference computes pre/post ops in
    __device__ static __forceinline__ Acc identity() { return (Acc)0; }
    __device__ static __forceinline__ Acc pre(T x, int64_t) {
        // `a.cast()` to FloatBinaryType<T> first (common_reduce.rs:352-482), then widen
        OutWide f = to_float_acc<T, OutWide>(x);
        if constexpr (OP == HPT_REDUCEL2) return (Acc)f * (Acc)f;
        else if constexpr (OP == HPT_REDUCEL3) {
            Acc a = (Acc)(f < 0 ? -f : f);
            return a * a * a;
        } else if constexpr (OP == HPT_LOGSUMEXP) {
            // Two-byte results are rounded to 8 or 11 significant bits: the hardware exp2 on the scaled
            // argument (|x| * 6e-8 relative error) is exact enough there at a quarter of the instructions,
            // and two-byte rows carry twice the elements per byte (f16 [2048, 151936] logsumexp(1) 4.0 TB/s
            // with the reduced form, where sum runs at 6.8).
            if constexpr (sizeof(OutWide) == 8) return (Acc)exp(f);
            else if constexpr (sizeof(Out) == 2) return (Acc)__expf(f);
            else return (Acc)exp_reduced(f);
        } else return (Acc)f;
    }
    __device__ static __forceinline__ Acc comb(Acc a, Acc b) { return a + b; }
    __device__ static __forceinline__ Out post(Acc a, double count) {
        Acc r;
        if constexpr (OP == HPT_MEAN) r = a / (Acc)count;
        else if constexpr (OP == HPT_REDUCEL2) {
            if constexpr (sizeof(Acc) == 8) r = sqrt(a); else r = sqrtf(a);
        } else if constexpr (OP == HPT_REDUCEL3) {
            if constexpr (sizeof(Acc) == 8) r = cbrt(a); else r = cbrtf(a);
        } else {
            if constexpr (sizeof(Acc) == 8) r = log(a); else r = logf(a);
        }
        return Elem<Out>::narrow((OutWide)r);
    }
    __device__ static __forceinline__ Acc from_out(Out o) { return (Acc)Elem<Out>::widen(o); }
};

// ---- all / any ----------------------------------------------------------------
template <int OP, class T> struct BoolOp {
    using In = T;
    using Out = bool8;
    using Acc = uint32_t;
    __device__ static __forceinline__ Acc identity() { return OP == HPT_ALL ? 1u : 0u; }
    __device__ static __forceinline__ Acc pre(T x, int64_t) { return Elem<T>::truthy(x) ? 1u : 0u; }
    __device__ static __forceinline__ Acc comb(Acc a, Acc b) { return OP == HPT_ALL ? (a & b) : (a | b); }
    __device__ static __forceinline__ Out post(Acc a, double) { return bool8{(uint8_t)(a != 0)}; }
    __device__ static __forceinline__ Acc from_out(Out o) { return o.v != 0; }
};

// ---- argmax / argmin ----------------------------------------------------------
// First extremum wins: strict compare from NEG_INF / INF with index 0
// (hpt/src/backends/cpu/kernels/argreduce_kernels.rs:13-21, 49-57); when two
// partial results hold equal values the lower index is kept, and a NaN never
// replaces anything because both comparisons are false for it.
template <class C> struct alignas(sizeof(C) == 8 ? 16 : 8) ArgPair {
    C val;
    typename std::conditional<sizeof(C) == 8, int64_t, int32_t>::type idx;
};

template <bool IS_MAX, class T> struct ArgOp {
    using In = T;
    using Out = int64_t;
    using C = typename Elem<T>::Cmp;
    using Acc = ArgPair<C>;
    __device__ static __forceinline__ Acc identity() {
        Acc a;
        a.val = IS_MAX ? ElemRange<T>::lowest() : ElemRange<T>::highest();
        a.idx = 0;
        return a;
    }
    __device__ static __forceinline__ Acc pre(T x, int64_t r) {
        if (Elem<T>::is_nan(x)) return identity();
        Acc a;
        a.val = Elem<T>::cmp(x);
        a.idx = (decltype(a.idx))r;
        return a;
    }
    __device__ static __forceinline__ Acc comb(Acc a, Acc b) {
        bool better = IS_MAX ? (b.val > a.val) : (b.val < a.val);
        bool tie = (b.val == a.val) && (b.idx < a.idx);
        return (better || tie) ? b : a;
    }
    __device__ static __forceinline__ Out post(Acc a, double) { return (int64_t)a.idx; }
    __device__ static __forceinline__ Acc from_out(Out) { return identity(); }
    // Fold element x at index r into acc when r only grows within the lane: the
    // strict compare alone keeps the first extremum, exactly the CPU scan.
    __device__ static __forceinline__ void accumulate(Acc& acc, T x, int64_t r) {
        const C v = Elem<T>::cmp(x);
        const bool better = IS_MAX ? (v > acc.val) : (v < acc.val);
        if (better) {
            acc.val = v;
            acc.idx = (decltype(acc.idx))r;
        }
    }
};

// acc = comb(acc, pre(x, r)), or the op's own cheaper in-order form when it has one.
template <class Op, class = void> struct HasAccumulate { static constexpr bool value = false; };
template <class Op>
struct HasAccumulate<Op, decltype(Op::accumulate(*(typename Op::Acc*)nullptr, typename Op::In{}, (int64_t)0))> {
    static constexpr bool value = true;
};
template <class Op>
__device__ __forceinline__ void fold_in(typename Op::Acc& acc, typename Op::In x, int64_t r) {
    if constexpr (HasAccumulate<Op>::value) Op::accumulate(acc, x, r);
    else acc = Op::comb(acc, Op::pre(x, r));
}

}  // namespace hpt
