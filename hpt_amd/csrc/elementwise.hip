// The steps either side of the reduction / normalisation path, on device:
//   strided copy   `contiguous()` of any view (hpt-cudakernels/src/strided_copy.cu:6-14,
//                  hpt/src/backends/cuda/tensor_internal/normal_out_unary.rs:286-310)
//   fill           `set_val` (hpt-cudakernels/src/set_val.cu:4-12)
//   add/sub/mul/div with broadcasting, also in place: the `add_` / `mul_` that layernorm's
//                  single-affine branches use (hpt/src/backends/cpu/tensor_internal/
//                  normalization.rs:187-192; trait hpt-traits/src/ops/binary.rs:9-152)
// All are HBM-bound: the work is in keeping both sides of the copy on whole cache lines.
#include <cstring>

#include "device_utils.hpp"
#include "elementwise_entry.hpp"

namespace hpt {

namespace {

#ifndef EW_UNR2
#define EW_UNR2 2
#endif
// vectors per thread: a copy keeps four loads in flight per thread; with two operands two
// vectors each are better (more workgroups resident, the same bytes in flight)
template <int NIN> constexpr int ew_unroll() { return NIN == 2 ? EW_UNR2 : 4; }

struct EwArgs {
    void* out;
    const void* in[2];
    int64_t stride[2][kMaxDims];
    int64_t size[kMaxDims];
    int n;
    int64_t total_v;  // vectors (of VEC output elements) in all
    int64_t inner_v;  // vectors along the innermost dim
};

// ---- operators ---------------------------------------------------------------------
// Integers wrap (hpt-types/src/scalars/impls.rs:31-48); bool add is OR and mul is AND;
// f16 / bf16 widen to f32, operate, round once (what the `half` crate does per operation).
template <int OP, class T> struct BinOp {
    __device__ static __forceinline__ T apply(T x, T y) {
        if constexpr (Elem<T>::is_bool) {
            const bool a = x.v != 0, b = y.v != 0;
            return bool8{(uint8_t)(OP == EW_ADD ? (a || b) : (a && b))};
        } else {
            using W = typename Elem<T>::Wide;
            const W a = Elem<T>::widen(x), b = Elem<T>::widen(y);
            W r;
            if constexpr (OP == EW_ADD) r = a + b;
            else if constexpr (OP == EW_SUB) r = a - b;
            else if constexpr (OP == EW_MUL) r = a * b;
            else r = a / b;
            return Elem<T>::narrow(r);
        }
    }
};

// Innermost position (in vectors) of output vector `v` and the operands' element offsets of
// its outer position.
template <int NIN>
__device__ __forceinline__ void ew_locate(const EwArgs& a, int64_t v, int64_t& iv, int64_t (&off)[2]) {
    const int last = a.n - 1;
    off[0] = off[1] = 0;
    if (((uint64_t)a.total_v >> 31) == 0) {
        uint32_t r = (uint32_t)v;
        uint32_t q = r / (uint32_t)a.inner_v;
        iv = r - q * (uint32_t)a.inner_v;
        for (int i = last - 1; i >= 0; --i) {
            const uint32_t s = (uint32_t)a.size[i];
            const uint32_t q2 = q / s;
            const uint32_t idx = q - q2 * s;
            q = q2;
#pragma unroll
            for (int k = 0; k < NIN; ++k) off[k] += (int64_t)idx * a.stride[k][i];
        }
    } else {
        int64_t q = v / a.inner_v;
        iv = v - q * a.inner_v;
        for (int i = last - 1; i >= 0; --i) {
            const int64_t q2 = q / a.size[i];
            const int64_t idx = q - q2 * a.size[i];
            q = q2;
#pragma unroll
            for (int k = 0; k < NIN; ++k) off[k] += idx * a.stride[k][i];
        }
    }
}

// ---- lanes along the innermost dim ---------------------------------------------------
// Thread t of a workgroup takes vectors t, t + 256, ... of the workgroup's 256 * UNR: UNR loads
// per operand are in flight before the first result is stored.
// SS = 2 (copy only): the innermost dim has input stride 2 (a [:, ::2] view): two full
// vectors are loaded per output vector and the odd positions dropped, which moves the same
// cache lines as a gather of single elements with a fraction of the instructions. (A
// 16-byte aligned vector that holds one valid element never leaves that element's page, so
// the unused last element of the last vector is safe to touch.)
template <int OP, class T, int VEC, int NIN, int SS = 1>
__global__ void __launch_bounds__(256) ew_inner_kernel(const EwArgs a) {
    constexpr int UNR = ew_unroll<NIN>();
    Pack<T, VEC> x[UNR], y[UNR];
    int64_t vi[UNR];
    const int last = a.n - 1;
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const int64_t v = ((int64_t)blockIdx.x * UNR + u) * 256 + threadIdx.x;
        vi[u] = v;
        if (v >= a.total_v) continue;
        int64_t off[2], iv;
        ew_locate<NIN>(a, v, iv, off);
        auto fetch = [&](int k, Pack<T, VEC>& dst) {
            const T* p = (const T*)a.in[k] + off[k];
            const int64_t s = a.stride[k][last];
            if constexpr (SS == 2) {
                const Pack<T, VEC> lo = load_pack_stream<T, VEC>(p + iv * (2 * VEC));
                const Pack<T, VEC> hi = load_pack_stream<T, VEC>(p + iv * (2 * VEC) + VEC);
#pragma unroll
                for (int j = 0; j < VEC / 2; ++j) {
                    dst.v[j] = lo.v[2 * j];
                    dst.v[VEC / 2 + j] = hi.v[2 * j];
                }
            } else if constexpr (VEC > 1) {
                if (s == 1) {
                    dst = load_pack_stream<T, VEC>(p + iv * VEC);
                } else {  // broadcast along the innermost dim
                    const T e = *p;
#pragma unroll
                    for (int j = 0; j < VEC; ++j) dst.v[j] = e;
                }
            } else {
                dst.v[0] = p[iv * s];
            }
        };
        fetch(0, x[u]);
        if constexpr (NIN == 2) fetch(1, y[u]);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        if (vi[u] >= a.total_v) continue;
        Pack<T, VEC> r;
        if constexpr (NIN == 2) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[j] = BinOp<OP, T>::apply(x[u].v[j], y[u].v[j]);
        } else {
            r = x[u];
        }
        T* o = (T*)a.out + vi[u] * VEC;
        if constexpr (VEC > 1) store_pack_stream<T, VEC>(o, r);
        else *o = r.v[0];
    }
}

// ---- copy of a view whose contiguous dim is not the innermost one ------------------------
// Dim B (size nB) is contiguous in the input, dim A (the innermost of the output, size nA)
// has input stride sA. A wavefront moves (8 VEC along B) x (8 VEC along A) tiles: lane
// (rg, cl) loads VEC vectors of VEC consecutive B positions (one per A position) and stores
// VEC vectors of VEC consecutive A positions. Both sides move whole 128-byte lines; the
// transpose itself is a renaming of registers. The other dims ride on blockIdx.z.
struct TransposeArgs {
    const void* in;
    void* out;
    int64_t sA;         // input stride of A (elements)
    int64_t oB;         // output stride of B
    int nA, nB;
    int nother;
    int osize[kMaxDims];
    int64_t oin[kMaxDims], oout[kMaxDims];  // strides of the other dims in input / output
    int ntA;            // (LDS form) tiles along A
};

template <class U>
__global__ void __launch_bounds__(256) ew_transpose_kernel(const TransposeArgs a) {
    constexpr int VEC = 16 / sizeof(U);
    constexpr int TB = 8 * VEC, TA = 8 * VEC, NA = 2;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int rg = lane & 7, cl = lane >> 3;
    // The four wavefronts of a workgroup take neighbouring B tiles (512 contiguous bytes of the
    // input per A position) and each wavefront takes two neighbouring A tiles (256 contiguous
    // bytes of the output per B position): measured 15 % faster than one tile per wavefront
    // with the wavefronts spread along A.
    const int b0 = (blockIdx.x * 4 + w) * TB + rg * VEC;
    const int a_base = blockIdx.y * (NA * TA) + cl * VEC;
    if (b0 >= a.nB || a_base >= a.nA) return;
    int64_t ioff = 0, ooff = 0;
    {
        uint32_t q = blockIdx.z;
        for (int i = a.nother - 1; i >= 0; --i) {
            const uint32_t s = (uint32_t)a.osize[i];
            const uint32_t q2 = q / s;
            const uint32_t idx = q - q2 * s;
            q = q2;
            ioff += (int64_t)idx * a.oin[i];
            ooff += (int64_t)idx * a.oout[i];
        }
    }
    const U* in = (const U*)a.in + ioff + b0;
    Pack<U, VEC> v[NA][VEC];
    bool have[NA];
#pragma unroll
    for (int s = 0; s < NA; ++s) {
        const int a0 = a_base + s * TA;
        have[s] = a0 < a.nA;
        if (have[s]) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[s][i] = load_pack_stream<U, VEC>(in + (int64_t)(a0 + i) * a.sA);
        }
    }
    U* out = (U*)a.out + ooff + (int64_t)b0 * a.oB + a_base;
#pragma unroll
    for (int k = 0; k < VEC; ++k)
#pragma unroll
        for (int s = 0; s < NA; ++s) {
            if (!have[s]) continue;
            Pack<U, VEC> o;
#pragma unroll
            for (int i = 0; i < VEC; ++i) o.v[i] = v[s][i].v[k];
            store_pack_stream<U, VEC>(out + (int64_t)k * a.oB + s * TA, o);
        }
}

// The same copy for views with at least a whole tile in both dims, through LDS: a workgroup moves a
// (16 VEC along B) x (16 VEC along A) tile. Loading, 16 lanes run along B (256 contiguous bytes of
// the input per A position, four A positions per instruction); a lane transposes its VEC x VEC block
// in registers and parks the VEC result vectors in LDS, one per B position; storing, 16 lanes run
// along A (256 contiguous bytes of the output per B position, four B positions per instruction).
// With the register transpose alone a lane's share of B and of A is fixed, 128 bytes each way, and
// eight 128-byte pieces per instruction is the slowest of the store patterns.
// LDS holds [16 VEC rows (B)][16 chunks of 16 bytes (A)]; chunk c of row b sits at c ^ (b / VEC): the
// 16 lanes of a quarter wavefront then hit 16 different 16-byte bank groups both when they write
// (same chunk, rows VEC apart) and when they read (same row, chunks 0..15).
template <class U>
__global__ void __launch_bounds__(256) ew_transpose_lds_kernel(const TransposeArgs a) {
    constexpr int VEC = 16 / sizeof(U);
    constexpr int TB = 16 * VEC, TA = 16 * VEC;
    __shared__ __align__(16) unsigned char tile[TB * 256];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int64_t ioff = 0, ooff = 0;
    {
        uint32_t q = blockIdx.z;
        for (int i = a.nother - 1; i >= 0; --i) {
            const uint32_t s = (uint32_t)a.osize[i];
            const uint32_t q2 = q / s;
            const uint32_t idx = q - q2 * s;
            q = q2;
            ioff += (int64_t)idx * a.oin[i];
            ooff += (int64_t)idx * a.oout[i];
        }
    }
    // Tiles are numbered along A first: workgroups that run at the same time then write neighbouring
    // 256-byte pieces of the same output rows (f16 [4096, 8192].permute(1, 0): 26.7 us; numbered along B
    // first, which gives the READS that locality instead, 28.7 us).
    const int tb = blockIdx.x / a.ntA, ta = blockIdx.x - tb * a.ntA;
    const int B0 = tb * TB, A0 = ta * TA;
    {
        const int jb = lane & 15, ac = w * 4 + (lane >> 4);
        const int b = B0 + jb * VEC, a0 = A0 + ac * VEC;
        if (b < a.nB && a0 < a.nA) {  // (both sizes are multiples of VEC: a chunk is inside or outside as a whole)
            const U* in = (const U*)a.in + ioff + (int64_t)a0 * a.sA + b;
            Pack<U, VEC> v[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[i] = load_pack_stream<U, VEC>(in + (int64_t)i * a.sA);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                Pack<U, VEC> o;
#pragma unroll
                for (int i = 0; i < VEC; ++i) o.v[i] = v[i].v[k];
                *(Pack<U, VEC>*)(tile + (jb * VEC + k) * 256 + ((ac ^ jb) << 4)) = o;
            }
        }
    }
    __syncthreads();
    {
        const int ca = lane & 15, rl = w * 4 + (lane >> 4);
        const int a0 = A0 + ca * VEC;
        U* out = (U*)a.out + ooff + a0;
#pragma unroll
        for (int it = 0; it < VEC; ++it) {
            const int row = it * 16 + rl;
            const int b = B0 + row;
            if (b < a.nB && a0 < a.nA) {
                const Pack<U, VEC> o = *(const Pack<U, VEC>*)(tile + row * 256 + (((ca ^ (row / VEC)) & 15) << 4));
                store_pack_stream<U, VEC>(out + (int64_t)b * a.oB, o);
            }
        }
    }
}

// ---- binary op with operands whose contiguous dim is not the innermost one -------------------
// a + b.t(), a.t() * b.t() into a contiguous result: the same tiles as ew_transpose_lds_kernel. The
// operands of MASK (bit k = operand k) are contiguous along B and come through LDS, transposed; an
// operand outside MASK lies like the result (contiguous along A, or broadcast along it) and is read
// by the lane that writes the result, at the very position when the result overwrites it in place.
// (The lanes-along-the-innermost-dim kernel gathers such an operand element by element: f32
// [8192, 4096] x.t() + y.t() 283 us.)
struct TransposeBinArgs {
    const void* in[2];
    void* out;
    int64_t sA[2];  // operand strides along A, the result's innermost dim (outside MASK: 1 or 0)
    int64_t sB[2];  // operand strides along B (in MASK: 1)
    int64_t oB;     // result stride along B
    int nA, nB, ntA;
    int nother;
    int osize[kMaxDims];
    int64_t oin[2][kMaxDims], oout[kMaxDims];  // strides of the other dims
};

template <int OP, class T, int MASK>
__global__ void __launch_bounds__(256) ew_binary_transpose_kernel(const TransposeBinArgs a) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TB = 16 * VEC, TA = 16 * VEC;
    constexpr int NTILE = (MASK & 1) + (MASK >> 1 & 1);
    static_assert(NTILE >= 1 && NTILE * TB * 256 <= 64 * 1024, "LDS");
    __shared__ __align__(16) unsigned char tile[NTILE][TB * 256];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int64_t ioff[2] = {0, 0}, ooff = 0;
    {
        uint32_t q = blockIdx.z;
        for (int i = a.nother - 1; i >= 0; --i) {
            const uint32_t s = (uint32_t)a.osize[i];
            const uint32_t q2 = q / s;
            const uint32_t idx = q - q2 * s;
            q = q2;
            ioff[0] += (int64_t)idx * a.oin[0][i];
            ioff[1] += (int64_t)idx * a.oin[1][i];
            ooff += (int64_t)idx * a.oout[i];
        }
    }
    const int tb = blockIdx.x / a.ntA, ta = blockIdx.x - tb * a.ntA;
    const int B0 = tb * TB, A0 = ta * TA;
    {
        const int jb = lane & 15, ac = w * 4 + (lane >> 4);
        const int b = B0 + jb * VEC, a0 = A0 + ac * VEC;
        if (b < a.nB && a0 < a.nA) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (!(MASK >> k & 1)) continue;
                constexpr int kFirst = MASK & 1 ? 0 : 1;
                unsigned char* tl = tile[k == kFirst ? 0 : NTILE - 1];
                const T* in = (const T*)a.in[k] + ioff[k] + (int64_t)a0 * a.sA[k] + b;
                Pack<T, VEC> v[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) v[i] = load_pack_stream<T, VEC>(in + (int64_t)i * a.sA[k]);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    Pack<T, VEC> o;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) o.v[i] = v[i].v[j];
                    *(Pack<T, VEC>*)(tl + (jb * VEC + j) * 256 + ((ac ^ jb) << 4)) = o;
                }
            }
        }
    }
    __syncthreads();
    {
        const int ca = lane & 15, rl = w * 4 + (lane >> 4);
        const int a0 = A0 + ca * VEC;
        T* out = (T*)a.out + ooff + a0;
#pragma unroll
        for (int it = 0; it < VEC; ++it) {
            const int row = it * 16 + rl;
            const int b = B0 + row;
            if (b < a.nB && a0 < a.nA) {
                Pack<T, VEC> x[2];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    if (MASK >> k & 1) {
                        constexpr int kFirst = MASK & 1 ? 0 : 1;
                        const unsigned char* tl = tile[k == kFirst ? 0 : NTILE - 1];
                        x[k] = *(const Pack<T, VEC>*)(tl + row * 256 + (((ca ^ (row / VEC)) & 15) << 4));
                    } else {
                        const T* in = (const T*)a.in[k] + ioff[k] + (int64_t)b * a.sB[k];
                        if (a.sA[k] == 1) {
                            x[k] = load_pack_stream<T, VEC>(in + a0);
                        } else {  // broadcast along A
                            const T e = *in;
#pragma unroll
                            for (int j = 0; j < VEC; ++j) x[k].v[j] = e;
                        }
                    }
                }
                Pack<T, VEC> o;
#pragma unroll
                for (int j = 0; j < VEC; ++j) o.v[j] = BinOp<OP, T>::apply(x[0].v[j], x[1].v[j]);
                store_pack_stream<T, VEC>(out + (int64_t)b * a.oB, o);
            }
        }
    }
}

// ---- dtype casts ----------------------------------------------------------------------
// Scalar<T>::cast as astype uses it (hpt/src/backends/cuda/tensor_impls.rs:129-140): integers go
// to a float type through Rust's `as` (round to nearest even; f16 / bf16 through f32, as the
// generated conversions do), floats to floats with ONE rounding. f64 -> f16 / bf16 has no
// hardware instruction: the value is first rounded to f32 "to odd" (truncate, then set the
// last bit if anything was lost), which makes the second, nearest-even rounding exact.
__device__ __forceinline__ float double_to_float_round_to_odd(double d) {
    float f = (float)d;
    if ((double)f != d && d == d && fabsf(f) != __builtin_huge_valf()) {
        uint32_t u = __float_as_uint(f);
        if (fabs((double)f) > fabs(d)) u -= 1;  // step back towards zero
        u |= 1u;
        f = __uint_as_float(u);
    }
    return f;
}

template <class TI, class TO> __device__ __forceinline__ TO cast_elem(TI x) {
    if constexpr (std::is_same<TI, TO>::value) {
        return x;
    } else if constexpr (Elem<TO>::is_float) {
        using WO = typename Elem<TO>::Wide;
        if constexpr (Elem<TI>::is_bool) {
            return Elem<TO>::narrow((WO)(x.v != 0));
        } else if constexpr (Elem<TI>::is_float) {
            if constexpr (std::is_same<TI, double>::value && sizeof(TO) == 2)
                return Elem<TO>::narrow(double_to_float_round_to_odd(x));
            else
                return Elem<TO>::narrow((WO)Elem<TI>::widen(x));
        } else {
            return Elem<TO>::narrow((WO)x);
        }
    } else {
        static_assert(sizeof(TI) == 0, "cast to a non-float dtype is not provided");
    }
}

template <class TI, class TO, int VEC>
__global__ void __launch_bounds__(256) ew_cast_kernel(const EwArgs a) {
    constexpr int UNR = 4;
    Pack<TI, VEC> x[UNR];
    int64_t vi[UNR];
    const int last = a.n - 1;
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const int64_t v = ((int64_t)blockIdx.x * UNR + u) * 256 + threadIdx.x;
        vi[u] = v;
        if (v >= a.total_v) continue;
        int64_t off[2], iv;
        ew_locate<1>(a, v, iv, off);
        const TI* p = (const TI*)a.in[0] + off[0];
        if constexpr (VEC > 1) x[u] = load_pack<TI, VEC>(p + iv * VEC);
        else x[u].v[0] = p[iv * a.stride[0][last]];
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        if (vi[u] >= a.total_v) continue;
        Pack<TO, VEC> r;
#pragma unroll
        for (int j = 0; j < VEC; ++j) r.v[j] = cast_elem<TI, TO>(x[u].v[j]);
        store_pack<TO, VEC>((TO*)a.out + vi[u] * VEC, r);
    }
}

// ---- fill -----------------------------------------------------------------------------
// `pattern` holds the element replicated over 16 bytes.
__global__ void __launch_bounds__(256) fill_vec_kernel(u32x4* out, u32x4 pattern, int64_t nvec) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nvec) __builtin_nontemporal_store(pattern, out + i);
}
template <class U> __global__ void __launch_bounds__(256) fill_scalar_kernel(U* out, U value, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = value;
}

EwArgs make_args(const EwPlan& p, void* out, const void* in0, const void* in1) {
    EwArgs a{};
    a.out = out;
    a.in[0] = in0;
    a.in[1] = in1;
    a.n = p.n;
    for (int i = 0; i < p.n; ++i) {
        a.size[i] = p.size[i];
        for (int k = 0; k < p.nin; ++k) a.stride[k][i] = p.stride[k][i];
    }
    a.inner_v = p.size[p.n - 1] / p.vec;
    a.total_v = p.total / p.vec;
    return a;
}

template <int OP, class T, int NIN>
void launch_inner(const EwPlan& p, void* out, const void* in0, const void* in1, hipStream_t st) {
    constexpr int FULL = 16 / sizeof(T);
    const EwArgs a = make_args(p, out, in0, in1);
    const int64_t blocks = (a.total_v + 256 * ew_unroll<NIN>() - 1) / (256 * ew_unroll<NIN>());
    if (blocks > 0x7fffffff) fail(HPT_ERR_SHAPE, "elementwise: tensor too large for one launch");
    if constexpr (NIN == 1 && FULL > 1) {
        if (p.vec == FULL && p.sstride == 2) {
            ew_inner_kernel<OP, T, FULL, NIN, 2><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
            return;
        }
    }
    if (p.vec == FULL && FULL > 1) ew_inner_kernel<OP, T, FULL, NIN><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
    else ew_inner_kernel<OP, T, 1, NIN><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
}

template <class U> void launch_transpose(const EwPlan& p, void* out, const void* in, hipStream_t st) {
    constexpr int VEC = 16 / sizeof(U);
    TransposeArgs t{};
    const int last = p.n - 1;
    t.in = in;
    t.out = out;
    t.nA = (int)p.size[last];
    t.sA = p.stride[0][last];
    t.nB = (int)p.size[p.tdim];
    int64_t ostride[kMaxDims];
    int64_t acc = 1;
    for (int i = last; i >= 0; --i) {
        ostride[i] = acc;
        acc *= p.size[i];
    }
    t.oB = ostride[p.tdim];
    int64_t others = 1;
    for (int i = 0; i < p.n; ++i) {
        if (i == p.tdim || i == last) continue;
        t.osize[t.nother] = (int)p.size[i];
        t.oin[t.nother] = p.stride[0][i];
        t.oout[t.nother] = ostride[i];
        ++t.nother;
        others *= p.size[i];
    }
    if (p.tile_lds) {
        constexpr int T = 16 * VEC;
        t.ntA = (t.nA + T - 1) / T;
        const int64_t tiles = (int64_t)t.ntA * ((t.nB + T - 1) / T);
        if (tiles > 0x7fffffff) fail(HPT_ERR_SHAPE, "strided copy: too many tiles for the transposing kernel");
        dim3 grid((unsigned)tiles, 1, (unsigned)others);
        ew_transpose_lds_kernel<U><<<grid, dim3(256), 0, st>>>(t);
        return;
    }
    constexpr int TILE = 8 * VEC;
    dim3 grid((unsigned)((t.nB + 4 * TILE - 1) / (4 * TILE)), (unsigned)((t.nA + 2 * TILE - 1) / (2 * TILE)), (unsigned)others);
    if (grid.y > 65535) fail(HPT_ERR_SHAPE, "strided copy: innermost dim too long for the transposing kernel");
    ew_transpose_kernel<U><<<grid, dim3(256), 0, st>>>(t);
}

template <class U> void launch_copy_sized(const EwPlan& p, void* out, const void* in, hipStream_t st) {
    if (p.kind == EwKind::Transpose) launch_transpose<U>(p, out, in, st);
    else launch_inner<EW_COPY, U, 1>(p, out, in, nullptr, st);
}

template <int OP, class T>
void launch_binary_transpose(const EwPlan& p, void* out, const void* a, const void* b, hipStream_t st) {
    if constexpr (sizeof(T) >= 2) {
        constexpr int VEC = 16 / sizeof(T);
        TransposeBinArgs t{};
        const int last = p.n - 1;
        t.in[0] = a;
        t.in[1] = b;
        t.out = out;
        t.nA = (int)p.size[last];
        t.nB = (int)p.size[p.tdim];
        int64_t ostride[kMaxDims];
        int64_t acc = 1;
        for (int i = last; i >= 0; --i) {
            ostride[i] = acc;
            acc *= p.size[i];
        }
        t.oB = ostride[p.tdim];
        for (int k = 0; k < 2; ++k) {
            t.sA[k] = p.stride[k][last];
            t.sB[k] = p.stride[k][p.tdim];
        }
        int64_t others = 1;
        for (int i = 0; i < p.n; ++i) {
            if (i == p.tdim || i == last) continue;
            t.osize[t.nother] = (int)p.size[i];
            t.oin[0][t.nother] = p.stride[0][i];
            t.oin[1][t.nother] = p.stride[1][i];
            t.oout[t.nother] = ostride[i];
            ++t.nother;
            others *= p.size[i];
        }
        constexpr int TILE = 16 * VEC;
        t.ntA = (t.nA + TILE - 1) / TILE;
        const int64_t tiles = (int64_t)t.ntA * ((t.nB + TILE - 1) / TILE);
        if (tiles > 0x7fffffff) fail(HPT_ERR_SHAPE, "binary: too many tiles for the transposing kernel");
        const dim3 grid((unsigned)tiles, 1, (unsigned)others);
        switch (p.tmask) {
            case 1: ew_binary_transpose_kernel<OP, T, 1><<<grid, dim3(256), 0, st>>>(t); return;
            case 2: ew_binary_transpose_kernel<OP, T, 2><<<grid, dim3(256), 0, st>>>(t); return;
            case 3: ew_binary_transpose_kernel<OP, T, 3><<<grid, dim3(256), 0, st>>>(t); return;
            default: break;
        }
    }
    fail(HPT_ERR_KERNEL, "binary: no transposing kernel for this plan");
}

template <int OP> void launch_binary_op(int dtype, const EwPlan& p, void* out, const void* a, const void* b, hipStream_t st) {
    switch (dtype) {
#define HPT_CASE(DT)                                                                 \
    case DT:                                                                         \
        if (p.kind == EwKind::Transpose)                                             \
            launch_binary_transpose<OP, typename DType<DT>::type>(p, out, a, b, st); \
        else                                                                         \
            launch_inner<OP, typename DType<DT>::type, 2>(p, out, a, b, st);         \
        return;
        HPT_CASE(HPT_I8) HPT_CASE(HPT_I16) HPT_CASE(HPT_I32) HPT_CASE(HPT_I64) HPT_CASE(HPT_U8) HPT_CASE(HPT_U16)
        HPT_CASE(HPT_U32) HPT_CASE(HPT_U64) HPT_CASE(HPT_F16) HPT_CASE(HPT_BF16) HPT_CASE(HPT_F32) HPT_CASE(HPT_F64)
#undef HPT_CASE
        case HPT_BOOL:
            if constexpr (OP == EW_ADD || OP == EW_MUL) {
                launch_inner<OP, bool8, 2>(p, out, a, b, st);
                return;
            }
            break;
        default: break;
    }
    fail(HPT_ERR_DTYPE, "binary: unsupported dtype %s for this operator", dtype_name(dtype));
}

}  // namespace

void launch_strided_copy(int dtype, const EwPlan& p, void* out, const void* in, hipStream_t st) {
    if (p.kind == EwKind::Empty) return;
    switch (dtype_size(dtype)) {
        case 1: launch_copy_sized<uint8_t>(p, out, in, st); break;
        case 2: launch_copy_sized<uint16_t>(p, out, in, st); break;
        case 4: launch_copy_sized<uint32_t>(p, out, in, st); break;
        case 8: launch_copy_sized<uint64_t>(p, out, in, st); break;
        default: fail(HPT_ERR_DTYPE, "strided copy: invalid dtype %d", dtype);
    }
}

void launch_binary(int op, int dtype, const EwPlan& p, void* out, const void* a, const void* b, hipStream_t st) {
    if (p.kind == EwKind::Empty) return;
    const bool is_float = dtype == HPT_F16 || dtype == HPT_BF16 || dtype == HPT_F32 || dtype == HPT_F64;
    switch (op) {
        case EW_ADD: launch_binary_op<EW_ADD>(dtype, p, out, a, b, st); break;
        case EW_SUB: launch_binary_op<EW_SUB>(dtype, p, out, a, b, st); break;
        case EW_MUL: launch_binary_op<EW_MUL>(dtype, p, out, a, b, st); break;
        case EW_DIV:
            // integer division promotes to a float type in Hpt (a different output dtype): not provided
            if (!is_float) fail(HPT_ERR_DTYPE, "binary: div is provided for float dtypes only, got %s", dtype_name(dtype));
            launch_binary_op<EW_DIV>(dtype, p, out, a, b, st);
            break;
        default: fail(HPT_ERR_PARAM, "binary: unknown operator %d", op);
    }
}

void launch_fill(int dtype, void* out, int64_t n, const void* value, hipStream_t st) {
    if (n == 0) return;
    const size_t es = dtype_size(dtype);
    unsigned char pat[16];
    for (size_t i = 0; i < 16; ++i) pat[i] = ((const unsigned char*)value)[i % es];
    unsigned char* p = (unsigned char*)out;
    int64_t done = 0;
    if (((uintptr_t)p % 16) == 0 && n * (int64_t)es >= 16) {
        const int64_t nvec = n * (int64_t)es / 16;
        u32x4 pattern;
        memcpy(&pattern, pat, 16);
        fill_vec_kernel<<<dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, st>>>((u32x4*)p, pattern, nvec);
        done = nvec * 16 / (int64_t)es;
    }
    const int64_t rest = n - done;
    if (rest > 0) {
        const unsigned blocks = (unsigned)((rest + 255) / 256);
        unsigned char* q = p + done * es;
        switch (es) {
            case 1: { uint8_t v; memcpy(&v, value, 1); fill_scalar_kernel<uint8_t><<<blocks, 256, 0, st>>>((uint8_t*)q, v, rest); break; }
            case 2: { uint16_t v; memcpy(&v, value, 2); fill_scalar_kernel<uint16_t><<<blocks, 256, 0, st>>>((uint16_t*)q, v, rest); break; }
            case 4: { uint32_t v; memcpy(&v, value, 4); fill_scalar_kernel<uint32_t><<<blocks, 256, 0, st>>>((uint32_t*)q, v, rest); break; }
            default: { uint64_t v; memcpy(&v, value, 8); fill_scalar_kernel<uint64_t><<<blocks, 256, 0, st>>>((uint64_t*)q, v, rest); break; }
        }
    }
}

namespace {

template <class TI, class TO> void launch_cast_t(const EwPlan& p, void* out, const void* in, hipStream_t st) {
    // vector width of the wider of the two types (the plan was made for it)
    constexpr int FULL = 16 / (sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO));
    const EwArgs a = make_args(p, out, in, nullptr);
    const int64_t blocks = (a.total_v + 1023) / 1024;
    if (blocks > 0x7fffffff) fail(HPT_ERR_SHAPE, "cast: tensor too large for one launch");
    if (p.vec == FULL && FULL > 1) ew_cast_kernel<TI, TO, FULL><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
    else ew_cast_kernel<TI, TO, 1><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
}

template <class TO> bool launch_cast_to(int in_dtype, const EwPlan& p, void* out, const void* in, hipStream_t st) {
    switch (in_dtype) {
#define HPT_CASE(DT)                                                      \
    case DT:                                                              \
        launch_cast_t<typename DType<DT>::type, TO>(p, out, in, st);      \
        return true;
        HPT_CASE(HPT_BOOL) HPT_CASE(HPT_I8) HPT_CASE(HPT_I16) HPT_CASE(HPT_I32) HPT_CASE(HPT_I64) HPT_CASE(HPT_U8)
        HPT_CASE(HPT_U16) HPT_CASE(HPT_U32) HPT_CASE(HPT_U64) HPT_CASE(HPT_F16) HPT_CASE(HPT_BF16) HPT_CASE(HPT_F32)
        HPT_CASE(HPT_F64)
#undef HPT_CASE
        default: return false;
    }
}

}  // namespace

void launch_cast(int in_dtype, int out_dtype, const EwPlan& p, void* out, const void* in, hipStream_t st) {
    if (p.kind == EwKind::Empty) return;
    bool ok = false;
    switch (out_dtype) {
        case HPT_F16: ok = launch_cast_to<f16_t>(in_dtype, p, out, in, st); break;
        case HPT_BF16: ok = launch_cast_to<bf16_t>(in_dtype, p, out, in, st); break;
        case HPT_F32: ok = launch_cast_to<float>(in_dtype, p, out, in, st); break;
        case HPT_F64: ok = launch_cast_to<double>(in_dtype, p, out, in, st); break;
        default: break;
    }
    if (!ok) fail(HPT_ERR_DTYPE, "cast: %s -> %s is not provided (the output must be a float dtype)", dtype_name(in_dtype),
                  dtype_name(out_dtype));
}

}  // namespace hpt
