// Device-side building blocks shared by every kernel of libhpt_hip (gfx950):
// element types, 128-bit vector access, index arithmetic over coalesced
// dimension lists, and wavefront-64 / workgroup combines.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "common.hpp"

namespace hpt {

// ---- element types --------------------------------------------------------

struct bool8 { uint8_t v; };
struct bf16_t { uint16_t bits; };
using f16_t = _Float16;

template <int DT> struct DType;
template <> struct DType<HPT_BOOL> { using type = bool8; };
template <> struct DType<HPT_I8> { using type = int8_t; };
template <> struct DType<HPT_I16> { using type = int16_t; };
template <> struct DType<HPT_I32> { using type = int32_t; };
template <> struct DType<HPT_I64> { using type = int64_t; };
template <> struct DType<HPT_U8> { using type = uint8_t; };
template <> struct DType<HPT_U16> { using type = uint16_t; };
template <> struct DType<HPT_U32> { using type = uint32_t; };
template <> struct DType<HPT_U64> { using type = uint64_t; };
template <> struct DType<HPT_F16> { using type = f16_t; };
template <> struct DType<HPT_BF16> { using type = bf16_t; };
template <> struct DType<HPT_F32> { using type = float; };
template <> struct DType<HPT_F64> { using type = double; };

__device__ __forceinline__ float bf16_to_float(bf16_t h) {
    return __uint_as_float((uint32_t)h.bits << 16);
}
// round-to-nearest-even, NaN stays a quiet NaN: gfx950 converts in hardware
// (v_cvt_pk_bf16_f32, two values per instruction when neighbours are converted together)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
    return r;
}

// Per element type: the type arithmetic is carried out in (`Wide`), the type
// order comparisons are carried out in (`Cmp`), and conversions.
//   floats  : f16/bf16/f32 compute in float, f64 in double
//   integers: two's-complement wrapping arithmetic, done on unsigned words
//             (hpt-types/src/scalars/impls.rs:31-48 uses wrapping_add/mul)
template <class T> struct Elem;

#define HPT_INT_ELEM(T, W, C, SIGNED)                                                    \
    template <> struct Elem<T> {                                                         \
        using Wide = W;                                                                  \
        using Cmp = C;                                                                   \
        static constexpr bool is_float = false;                                          \
        static constexpr bool is_signed = SIGNED;                                        \
        static constexpr bool is_bool = false;                                           \
        __device__ static __forceinline__ W widen(T x) { return (W)(C)x; }               \
        __device__ static __forceinline__ T narrow(W x) { return (T)x; }                 \
        __device__ static __forceinline__ C cmp(T x) { return (C)x; }                    \
        __device__ static __forceinline__ T from_cmp(C x) { return (T)x; }               \
        __device__ static __forceinline__ bool is_nan(T) { return false; }               \
        __device__ static __forceinline__ bool truthy(T x) { return x != 0; }            \
    };
HPT_INT_ELEM(int8_t, uint32_t, int32_t, true)
HPT_INT_ELEM(int16_t, uint32_t, int32_t, true)
HPT_INT_ELEM(int32_t, uint32_t, int32_t, true)
HPT_INT_ELEM(int64_t, uint64_t, int64_t, true)
HPT_INT_ELEM(uint8_t, uint32_t, uint32_t, false)
HPT_INT_ELEM(uint16_t, uint32_t, uint32_t, false)
HPT_INT_ELEM(uint32_t, uint32_t, uint32_t, false)
HPT_INT_ELEM(uint64_t, uint64_t, uint64_t, false)
#undef HPT_INT_ELEM

template <> struct Elem<bool8> {
    using Wide = uint32_t;
    using Cmp = uint32_t;
    static constexpr bool is_float = false;
    static constexpr bool is_signed = false;
    static constexpr bool is_bool = true;
    __device__ static __forceinline__ uint32_t widen(bool8 x) { return x.v != 0; }
    __device__ static __forceinline__ bool8 narrow(uint32_t x) { return bool8{(uint8_t)(x != 0)}; }
    __device__ static __forceinline__ uint32_t cmp(bool8 x) { return x.v != 0; }
    __device__ static __forceinline__ bool8 from_cmp(uint32_t x) { return bool8{(uint8_t)(x != 0)}; }
    __device__ static __forceinline__ bool is_nan(bool8) { return false; }
    __device__ static __forceinline__ bool truthy(bool8 x) { return x.v != 0; }
};

#define HPT_FLOAT_ELEM(T, W, TOW, FROMW)                                                 \
    template <> struct Elem<T> {                                                         \
        using Wide = W;                                                                  \
        using Cmp = W;                                                                   \
        static constexpr bool is_float = true;                                           \
        static constexpr bool is_signed = true;                                          \
        static constexpr bool is_bool = false;                                           \
        __device__ static __forceinline__ W widen(T x) { return TOW; }                   \
        __device__ static __forceinline__ T narrow(W x) { return FROMW; }                \
        __device__ static __forceinline__ W cmp(T x) { return widen(x); }                \
        __device__ static __forceinline__ T from_cmp(W x) { return narrow(x); }          \
        __device__ static __forceinline__ bool is_nan(T x) { W w = widen(x); return w != w; } \
        __device__ static __forceinline__ bool truthy(T x) { return widen(x) != (W)0; }  \
    };
HPT_FLOAT_ELEM(f16_t, float, (float)x, (f16_t)x)
HPT_FLOAT_ELEM(bf16_t, float, bf16_to_float(x), float_to_bf16(x))
HPT_FLOAT_ELEM(float, float, x, x)
HPT_FLOAT_ELEM(double, double, x, x)
#undef HPT_FLOAT_ELEM

// ---- vector access -----------------------------------------------------------

template <class T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

template <class T, int N>
__device__ __forceinline__ Pack<T, N> load_pack(const T* p) {
    return *reinterpret_cast<const Pack<T, N>*>(p);
}
template <class T, int N>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, N>& v) {
    *reinterpret_cast<Pack<T, N>*>(p) = v;
}
// N consecutive elements from an address that is only element-aligned: one wide load all the
// same (global memory takes unaligned vector accesses), at the cost of touching two lines now and
// then. For small operands that sit in cache: gamma / beta of a row that starts off a boundary.
template <class T, int N>
__device__ __forceinline__ Pack<T, N> load_pack_unaligned(const T* p) {
    Pack<T, N> v;
    __builtin_memcpy(&v, p, sizeof(T) * N);
    return v;
}

// Streaming (non-temporal) forms for data that is touched exactly once: the
// access is marked so that it does not displace reusable lines from the caches.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#ifndef HPT_STREAMING_ACCESS
#define HPT_STREAMING_ACCESS 1
#endif
template <class T, int N>
__device__ __forceinline__ Pack<T, N> load_pack_stream(const T* p) {
#if HPT_STREAMING_ACCESS
    if constexpr (sizeof(T) * N == 16) {
        union { u32x4 u; Pack<T, N> v; } c;
        c.u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        return c.v;
    } else if constexpr (sizeof(T) * N == 8) {
        union { u32x2 u; Pack<T, N> v; } c;
        c.u = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
        return c.v;
    } else
#endif
        return load_pack<T, N>(p);
}
template <class T, int N>
__device__ __forceinline__ void store_pack_stream(T* p, const Pack<T, N>& v) {
#if HPT_STREAMING_ACCESS
    if constexpr (sizeof(T) * N == 16) {
        union { u32x4 u; Pack<T, N> v; } c;
        c.v = v;
        __builtin_nontemporal_store(c.u, reinterpret_cast<u32x4*>(p));
    } else if constexpr (sizeof(T) * N == 8) {
        union { u32x2 u; Pack<T, N> v; } c;
        c.v = v;
        __builtin_nontemporal_store(c.u, reinterpret_cast<u32x2*>(p));
    } else
#endif
        store_pack<T, N>(p, v);
}

// ---- f16 data used straight from its packed registers ---------------------------
// v_fma_mix_f32 reads a half out of either side of a 32-bit register and widens it
// inside the multiply-add: (float)x * b + c costs one instruction instead of a
// conversion plus the arithmetic, with the same single rounding. The compiler picks it
// for fma(widened half, b, c) as long as it cannot fold the multiplication away, so
// where b is 1 the caller passes a 1.0 the compiler cannot see through (opaque_one).
__device__ __forceinline__ float opaque_one() {
    float one = 1.0f;
    asm volatile("" : "+v"(one));
    return one;
}

// widen(x) * b + c for any element type; one instruction for f16.
template <class T>
__device__ __forceinline__ typename Elem<T>::Wide widen_fma(T x, typename Elem<T>::Wide b, typename Elem<T>::Wide c) {
    if constexpr (std::is_same<T, f16_t>::value) return __builtin_fmaf((float)x, b, c);
    else return Elem<T>::widen(x) * b + c;
}

template <class T, int N>
__device__ __forceinline__ void store_pack_unaligned(T* p, const Pack<T, N>& v) {
    __builtin_memcpy(p, &v, sizeof(T) * N);
}

// ---- exponential ---------------------------------------------------------------
// e^x for f32 data. The error of the hardware route exp2(x * log2 e) grows with |x| (the product
// is rounded before the exponential sees it: |x| * 6e-8 relative). Here x = n ln 2 + r is split
// exactly first (Cody-Waite, two fused multiply-adds), the hardware exp2 gets an argument of at
// most 1/2 in magnitude, and the result is scaled by 2^n: within about 2 ulp over the whole range
// (1.2 ulp from the reduction and the final rounding, the rest the hardware's) at a third of the
// library routine's cost - which is what bounded read-only passes that take an exponential per
// element (39 -> 34 us for the statistics pass of an f32 [32768, 1024] softmax(axis=0); the
// hardware route alone, too inaccurate here, runs it in 27).
// NONPOS: the caller's arguments never exceed 0 (softmax: x - max), so the upper end needs no care.
template <bool NONPOS = false> __device__ __forceinline__ float exp_reduced(float x) {
    // n is kept above -150: e^x is 0 below 2^-150 anyway, and x = -inf then gives r = -inf and
    // exp2(-inf) = 0 instead of the inf - inf an unbounded n would make. (A NaN x is dropped by the
    // max and comes back through r.)
    const float n = __builtin_rintf(__builtin_fmaxf(x * 1.44269504f, -150.0f));
    float r = __builtin_fmaf(n, -0.693145752f, x);  // ln 2, high part (the product is exact for |n| < 2^10)
    r = __builtin_fmaf(n, -1.42860682e-6f, r);      // ln 2, low part
    const float e = __builtin_amdgcn_exp2f(r * 1.44269504f);
    float v = __builtin_ldexpf(e, (int)n);
    // above e^89 the result is +inf (+inf itself would make the reduction inf - inf)
    if constexpr (!NONPOS) v = x > 89.0f ? __builtin_huge_valf() : v;
    return v;
}

// ---- index arithmetic -----------------------------------------------------

// Offset (in elements) of linear index `idx` over dims `d`, outermost first.
__device__ __forceinline__ int64_t offset_of(const Dims& d, int64_t idx) {
    int64_t off = 0;
    if (((uint64_t)idx >> 32) == 0) {
        uint32_t i32 = (uint32_t)idx;
        for (int i = d.n - 1; i > 0; --i) {
            uint32_t s = (uint32_t)d.size[i];
            uint32_t q = i32 / s;
            off += (int64_t)(i32 - q * s) * d.stride[i];
            i32 = q;
        }
        if (d.n > 0) off += (int64_t)i32 * d.stride[0];
    } else {
        for (int i = d.n - 1; i > 0; --i) {
            int64_t s = d.size[i];
            int64_t q = idx / s;
            off += (idx - q * s) * d.stride[i];
            idx = q;
        }
        if (d.n > 0) off += idx * d.stride[0];
    }
    return off;
}

// ---- wavefront / workgroup combines ---------------------------------------

template <class A> __device__ __forceinline__ A shfl_xor_any(A v, int mask) {
    static_assert(sizeof(A) % 4 == 0, "shuffle works on 32-bit words");
    constexpr int W = sizeof(A) / 4;
    union { A a; int w[W]; } in, out;
    in.a = v;
#pragma unroll
    for (int i = 0; i < W; ++i) out.w[i] = __shfl_xor(in.w[i], mask, 64);
    return out.a;
}

// Move every 32-bit word of v along a DPP lane pattern (a VALU modifier, a few
// cycles) instead of through the LDS crossbar that __shfl uses.
template <int CTRL, class A> __device__ __forceinline__ A dpp_move(A v) {
    static_assert(sizeof(A) % 4 == 0, "DPP moves 32-bit words");
    constexpr int W = sizeof(A) / 4;
    union { A a; int w[W]; } in, out;
    in.a = v;
#pragma unroll
    for (int i = 0; i < W; ++i) out.w[i] = __builtin_amdgcn_update_dpp(0, in.w[i], CTRL, 0xF, 0xF, true);
    return out.a;
}

// All-reduce over aligned groups of `width` consecutive lanes (power of two, <= 64).
// Inside a row of 16 lanes the butterfly runs on DPP patterns: swap within pairs
// (quad_perm [1,0,3,2]), swap pairs (quad_perm [2,3,0,1]), mirror within 8
// (row_half_mirror), mirror within 16 (row_mirror); rows are then combined with
// two cross-lane shuffles. Every lane of a group ends with the same value.
template <class Op, class A> __device__ __forceinline__ A group_reduce(A v, int width) {
    if (width >= 2) v = Op::comb(v, dpp_move<0xB1>(v));
    if (width >= 4) v = Op::comb(v, dpp_move<0x4E>(v));
    if (width >= 8) v = Op::comb(v, dpp_move<0x141>(v));
    if (width >= 16) v = Op::comb(v, dpp_move<0x140>(v));
    if (width >= 32) v = Op::comb(v, shfl_xor_any(v, 16));
    if (width >= 64) v = Op::comb(v, shfl_xor_any(v, 32));
    return v;
}

// All-reduce over the whole workgroup (blockDim.x * blockDim.y threads, a
// multiple of 64). `smem` must hold one A per wavefront (<= 16).
template <class Op, class A> __device__ __forceinline__ A block_reduce(A v, A* smem) {
    const int tid = threadIdx.y * blockDim.x + threadIdx.x;
    const int nwaves = (blockDim.x * blockDim.y) >> 6;
    v = group_reduce<Op>(v, 64);
    __syncthreads();  // protect smem from a previous use
    if ((tid & 63) == 0) smem[tid >> 6] = v;
    __syncthreads();
    A r = smem[0];
    for (int w = 1; w < nwaves; ++w) r = Op::comb(r, smem[w]);
    return r;
}

}  // namespace hpt
