// The two reduction kernels of libhpt_hip and their launcher.
//
//   row_reduce_kernel  lanes walk the reduced index space of one output
//                      (a reduced dim owns the smallest stride): 128-bit loads
//                      along the row, combine over the lanes of a wavefront by
//                      cross-lane shuffles, over wavefronts through LDS.
//   col_reduce_kernel  lanes walk neighbouring outputs (a kept dim owns the
//                      smallest stride): every lane accumulates its own
//                      outputs while thread rows stride over the reduced range;
//                      the thread rows are combined through LDS.
//
// When there are too few outputs to fill 256 CUs, several workgroups share one
// output: each writes a partial accumulator, and the workgroup that arrives
// last (a device-scope counter per output) folds the partials in a fixed order,
// so results are bit-identical from run to run. The counter is reset by that
// last workgroup, so the scratch needs no clearing between launches.
//
// These replace the eight kernel variants per op of the reference's device
// path (hpt-cudakernels/src/reduce/reduce_template.cuh:8-198) and the CPU
// kernels hpt/src/backends/cpu/kernels/reduce.rs:153-791.
#pragma once

#include "reduce_entry.hpp"
#include "reduce_ops.cuh"

namespace hpt {

struct RowArgs {
    const void* in;
    void* out;
    void* partial;
    unsigned* counters;
    Dims kept;   // output index -> input offset
    Dims redo;   // outer reduced dims (all reduced dims but the innermost)
    int64_t K;       // outputs
    int64_t rout;    // product of redo sizes
    int64_t rin_v;   // innermost reduced length, in vectors
    int64_t sr;      // innermost reduced stride in elements (1 when VEC > 1)
    int64_t qchunk;  // outer reduced indices per split
    int64_t ichunk;  // inner vectors per split
    double count;    // elements reduced per output (mean)
    int tpr, tpr_log2, rpb, split_q, split_i, init_out;
};

struct ColArgs {
    const void* in;
    void* out;
    void* partial;
    unsigned* counters;
    Dims kept_outer;  // kept dims except the innermost
    Dims red;         // reduced dims
    int64_t K;        // outputs
    int64_t kin;      // innermost kept size
    int64_t sk;       // its stride (1 when VEC > 1)
    int64_t R;        // reduced elements per output
    int64_t chunk;    // reduced indices per split
    double count;
    int split, init_out;
};

template <class Op>
__device__ __forceinline__ void write_out(void* out, int64_t o, typename Op::Acc acc, int init_out,
                                          double count) {
    typename Op::Out* p = (typename Op::Out*)out + o;
    if (!init_out) acc = Op::comb(Op::from_out(*p), acc);
    *p = Op::post(acc, count);
}

template <class Op, int VEC>
__global__ void __launch_bounds__(1024) row_reduce_kernel(const RowArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    __shared__ Acc smem[16];
    __shared__ int s_last;

    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int64_t row = (int64_t)blockIdx.x * a.rpb + ty;
    const bool valid = row < a.K;
    Acc acc = Op::identity();

    if (valid) {
        const T* base = (const T*)a.in + offset_of(a.kept, row);
        const int sq = blockIdx.y / a.split_i;
        const int si = blockIdx.y - sq * a.split_i;
        const int64_t q0 = sq * a.qchunk;
        const int64_t q1 = min(a.rout, q0 + a.qchunk);
        const int64_t i0 = si * a.ichunk;
        const int64_t i1 = min(a.rin_v, i0 + a.ichunk);
        const int64_t ni = i1 - i0;
        if (ni >= tpr || q1 - q0 <= 1) {
            for (int64_t q = q0; q < q1; ++q) {
                const T* p = base + offset_of(a.redo, q);
#pragma unroll 4
                for (int64_t iv = i0 + tx; iv < i1; iv += tpr) {
                    if constexpr (VEC > 1) {
                        Pack<T, VEC> v = load_pack<T, VEC>(p + iv * VEC);
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            acc = Op::comb(acc, Op::pre(v.v[j], iv * VEC + j));
                    } else {
                        acc = Op::comb(acc, Op::pre(p[iv * a.sr], iv));
                    }
                }
            }
        } else if (ni > 0) {
            // short inner runs: spread the lanes over (outer, inner) pairs
            const int64_t total = (q1 - q0) * ni;
            for (int64_t t = tx; t < total; t += tpr) {
                int64_t dq, di;
                if (((uint64_t)total >> 32) == 0) {
                    uint32_t d = (uint32_t)t / (uint32_t)ni;
                    dq = d;
                    di = (uint32_t)t - d * (uint32_t)ni;
                } else {
                    dq = t / ni;
                    di = t - dq * ni;
                }
                const T* p = base + offset_of(a.redo, q0 + dq);
                const int64_t iv = i0 + di;
                if constexpr (VEC > 1) {
                    Pack<T, VEC> v = load_pack<T, VEC>(p + iv * VEC);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc = Op::comb(acc, Op::pre(v.v[j], iv * VEC + j));
                } else {
                    acc = Op::comb(acc, Op::pre(p[iv * a.sr], iv));
                }
            }
        }
    }

    if (tpr <= 64) acc = group_reduce<Op>(acc, tpr);
    else acc = block_reduce<Op>(acc, smem);

    const int split = a.split_q * a.split_i;
    if (split == 1) {
        if (tx == 0 && valid) write_out<Op>(a.out, row, acc, a.init_out, a.count);
        return;
    }

    // several workgroups per output: one output per workgroup here (rpb == 1)
    Acc* part = (Acc*)a.partial + row * split;
    // Only the thread that wrote the partial releases it: a device-scope fence
    // writes back the L2 of this XCD, so it must not run once per wavefront.
    if (threadIdx.x == 0) {
        part[blockIdx.y] = acc;
        __threadfence();
        unsigned prev = atomicAdd(&a.counters[row], 1u);
        s_last = (prev == (unsigned)(split - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    acc = Op::identity();
    for (int s = threadIdx.x; s < split; s += blockDim.x) acc = Op::comb(acc, part[s]);
    acc = block_reduce<Op>(acc, smem);
    if (threadIdx.x == 0) {
        write_out<Op>(a.out, row, acc, a.init_out, a.count);
        a.counters[row] = 0;
    }
}

template <class Op, int VEC>
__global__ void __launch_bounds__(1024) col_reduce_kernel(const ColArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Acc* smem = (Acc*)smem_raw;
    __shared__ int s_last;

    const int bx = blockDim.x, by = blockDim.y;
    const int tx = threadIdx.x, ty = threadIdx.y;
    const int64_t o0 = ((int64_t)blockIdx.x * bx + tx) * VEC;
    const bool valid = o0 < a.K;
    Acc acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::identity();

    if (valid) {
        int64_t outer, inner;
        if (((uint64_t)o0 >> 32) == 0 && ((uint64_t)a.kin >> 32) == 0) {
            uint32_t q = (uint32_t)o0 / (uint32_t)a.kin;
            outer = q;
            inner = (uint32_t)o0 - q * (uint32_t)a.kin;
        } else {
            outer = o0 / a.kin;
            inner = o0 - outer * a.kin;
        }
        const T* base = (const T*)a.in + offset_of(a.kept_outer, outer) + inner * a.sk;
        const int64_t r0 = (int64_t)blockIdx.y * a.chunk;
        const int64_t r1 = min(a.R, r0 + a.chunk);
        if (a.red.n <= 1) {
            const int64_t rs = a.red.n ? a.red.stride[0] : 0;
#pragma unroll 4
            for (int64_t r = r0 + ty; r < r1; r += by) {
                const T* p = base + r * rs;
                if constexpr (VEC > 1) {
                    Pack<T, VEC> v = load_pack<T, VEC>(p);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = Op::comb(acc[j], Op::pre(v.v[j], r));
                } else {
                    acc[0] = Op::comb(acc[0], Op::pre(*p, r));
                }
            }
        } else {
#pragma unroll 2
            for (int64_t r = r0 + ty; r < r1; r += by) {
                const T* p = base + offset_of(a.red, r);
                if constexpr (VEC > 1) {
                    Pack<T, VEC> v = load_pack<T, VEC>(p);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = Op::comb(acc[j], Op::pre(v.v[j], r));
                } else {
                    acc[0] = Op::comb(acc[0], Op::pre(*p, r));
                }
            }
        }
    }

    // fold the thread rows: row 0 collects, in row order
    auto fold_rows = [&]() {
        if (by == 1) return;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < VEC; ++j) smem[((size_t)ty * bx + tx) * VEC + j] = acc[j];
        __syncthreads();
        if (ty == 0) {
            for (int y = 1; y < by; ++y) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    acc[j] = Op::comb(acc[j], smem[((size_t)y * bx + tx) * VEC + j]);
            }
        }
    };
    fold_rows();

    if (a.split == 1) {
        if (ty == 0 && valid) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) write_out<Op>(a.out, o0 + j, acc[j], a.init_out, a.count);
        }
        return;
    }

    Acc* part = (Acc*)a.partial;
    if (ty == 0 && valid) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) part[(int64_t)blockIdx.y * a.K + o0 + j] = acc[j];
    }
    if (ty == 0) __threadfence();  // the writers release their partials
    __syncthreads();
    if (tx == 0 && ty == 0) {
        unsigned prev = atomicAdd(&a.counters[blockIdx.x], 1u);
        s_last = (prev == (unsigned)(a.split - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::identity();
    if (valid) {
        for (int s = ty; s < a.split; s += by) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = Op::comb(acc[j], part[(int64_t)s * a.K + o0 + j]);
        }
    }
    fold_rows();
    if (ty == 0 && valid) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) write_out<Op>(a.out, o0 + j, acc[j], a.init_out, a.count);
    }
    if (tx == 0 && ty == 0) a.counters[blockIdx.x] = 0;
}

// Fill `n` outputs with the op's identity (a reduced dim of size 0).
template <class Op>
__global__ void identity_fill_kernel(void* out, int64_t n, int init_out, double count) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) write_out<Op>(out, i, Op::identity(), init_out, count);
}

inline int ilog2(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

template <class Op>
void launch_reduce_t(const ReducePlan& p, const void* in, void* out, const ReduceScratch& sc,
                     hipStream_t st, int init_out) {
    using T = typename Op::In;
    constexpr int FULL = 16 / sizeof(T);
    const double count = (double)p.R;
    if (p.kind == ReduceKind::Empty) return;
    if (p.kind == ReduceKind::Identity) {
        int64_t blocks = (p.K + 255) / 256;
        identity_fill_kernel<Op><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(out, p.K, init_out, count);
        return;
    }
    if (p.kind == ReduceKind::Row) {
        RowArgs a{};
        a.in = in;
        a.out = out;
        a.partial = sc.partial;
        a.counters = sc.counters;
        a.kept = p.kept;
        a.redo = p.red;
        a.redo.n = p.red.n - 1;
        a.K = p.K;
        const int64_t rin = p.red.size[p.red.n - 1];
        a.rout = p.R / rin;
        a.rin_v = rin / p.vec;
        a.sr = p.red.stride[p.red.n - 1];
        a.qchunk = (a.rout + p.split_q - 1) / p.split_q;
        a.ichunk = (a.rin_v + p.split_i - 1) / p.split_i;
        a.count = count;
        a.tpr = p.tpr;
        a.tpr_log2 = ilog2(p.tpr);
        a.rpb = p.rpb;
        a.split_q = p.split_q;
        a.split_i = p.split_i;
        a.init_out = init_out;
        dim3 grid((unsigned)((p.K + p.rpb - 1) / p.rpb), (unsigned)p.split);
        dim3 block((unsigned)(p.tpr * p.rpb));
        if (p.vec == FULL && FULL > 1) row_reduce_kernel<Op, FULL><<<grid, block, 0, st>>>(a);
        else row_reduce_kernel<Op, 1><<<grid, block, 0, st>>>(a);
        return;
    }
    ColArgs a{};
    a.in = in;
    a.out = out;
    a.partial = sc.partial;
    a.counters = sc.counters;
    a.kept_outer = p.kept;
    a.kept_outer.n = p.kept.n > 0 ? p.kept.n - 1 : 0;
    a.red = p.red;
    a.K = p.K;
    a.kin = p.kept.n ? p.kept.size[p.kept.n - 1] : 1;
    a.sk = p.kept.n ? p.kept.stride[p.kept.n - 1] : 0;
    a.R = p.R;
    a.chunk = p.chunk;
    a.count = count;
    a.split = p.split;
    a.init_out = init_out;
    const int64_t kv = p.K / p.vec;
    dim3 grid((unsigned)((kv + p.bx - 1) / p.bx), (unsigned)p.split);
    dim3 block((unsigned)p.bx, (unsigned)p.by);
    size_t smem = p.by > 1 ? (size_t)p.bx * p.by * p.vec * sizeof(typename Op::Acc) : 0;
    if (p.vec == FULL && FULL > 1) col_reduce_kernel<Op, FULL><<<grid, block, smem, st>>>(a);
    else col_reduce_kernel<Op, 1><<<grid, block, smem, st>>>(a);
}

// Instantiate launch_reduce_t for every dtype of one op family.
#define HPT_FOR_ALL_DTYPES(X) \
    X(HPT_BOOL) X(HPT_I8) X(HPT_I16) X(HPT_I32) X(HPT_I64) X(HPT_U8) X(HPT_U16) X(HPT_U32) \
    X(HPT_U64) X(HPT_F16) X(HPT_BF16) X(HPT_F32) X(HPT_F64)

}  // namespace hpt
