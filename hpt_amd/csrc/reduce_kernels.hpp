// The reduction kernels of libhpt_hip and their launcher.
//
//   row kernels   lanes walk the reduced index space of one output (a reduced
//                 dim owns the smallest stride): 128-bit streaming loads along
//                 the row, combine over the lanes of a wavefront by cross-lane
//                 shuffles, over wavefronts through LDS.
//   col kernels   lanes walk neighbouring outputs (a kept dim owns the smallest
//                 stride): every lane accumulates its own VEC outputs while it
//                 strides over the reduced range; thread rows meet in LDS.
//
// Each family has a lean form for the layouts that matter most (one reduced
// dim, at most two kept dims, 32-bit extents: every benchmark configuration)
// and a general form that walks up to 8 + 8 coalesced dims with 64-bit
// arithmetic. The lean kernels exist because these launches last 15-50 us and
// run thousands of short-lived workgroups: a long prologue of index arithmetic
// costs a measurable share of the HBM bandwidth.
//
// When there are too few outputs to fill 256 CUs, several workgroups share an
// output: each writes a partial accumulator and a second, tiny kernel folds the
// partials in a fixed order (bit-identical from run to run). Two launches beat
// the single-launch "last workgroup folds" scheme here: its device-scope fence
// writes back the L2 and its counter is one contended address, and both
// serialise (measured: 155 us against 19 us for a 100 MB full sum).
//
// These replace the eight kernel variants per op of the reference's device
// path (hpt-cudakernels/src/reduce/reduce_template.hpp:8-198) and the CPU
// kernels hpt/src/backends/cpu/kernels/reduce.rs:153-791.
#pragma once

#include "reduce_entry.hpp"
#include "reduce_ops.hpp"

namespace hpt {

template <class Op>
__device__ __forceinline__ void write_out(void* out, int64_t o, typename Op::Acc acc, int init_out,
                                          double count) {
    typename Op::Out* p = (typename Op::Out*)out + o;
    if (!init_out) acc = Op::comb(Op::from_out(*p), acc);
    *p = Op::post(acc, count);
}

// N neighbouring outputs of one lane, overwritten (init_out) with 128-bit stores. `p` must be
// aligned to min(16, N * sizeof(Out)) bytes; the caller checks the base and o is a multiple of N.
template <class Op, int N>
__device__ __forceinline__ void write_out_pack(void* out, int64_t o, const typename Op::Acc (&acc)[N], double count) {
    using Out = typename Op::Out;
    constexpr int PER = 16 / sizeof(Out) < N ? 16 / sizeof(Out) : N;  // outputs per store
    Out* p = (Out*)out + o;
#pragma unroll
    for (int j0 = 0; j0 < N; j0 += PER) {
        Pack<Out, PER> v;
#pragma unroll
        for (int j = 0; j < PER; ++j) v.v[j] = Op::post(acc[j0 + j], count);
        store_pack<Out, PER>(p + j0, v);
    }
}

// ---- lean row kernel ---------------------------------------------------------
// out[row] = reduce over i in [0, rin) of in[row * row_stride + i * sr].
struct RowLeanArgs {
    const void* in;
    void* out;       // outputs, or partial accumulators when split > 1
    int64_t row_stride;
    double count;
    int K;           // rows
    int rin_v;       // row length in vectors
    int rin;         // row length in elements (RAG)
    int sr;          // element stride along the row (1 when VEC > 1)
    int ichunk;      // vectors per split
    int tpr, tpr_log2, rpb, split, init_out;
};

// SS = 2: the row's elements sit at every second position; full vectors are
// loaded and the odd positions dropped (see row_reg_kernel).
// RAG: contiguous rows of any length that start anywhere. A row's elements before its first
// 16-byte boundary and after its last whole vector are folded one by one (by the first split's
// lanes); the vectors between are aligned.
// UA: short or strided-pitch rows off the grid: unaligned 128-bit loads from the row start on; the
// last vector of a row is taken from the row's END backwards and the elements it shares with the
// vector before are skipped, so no load leaves the row.
// IL > 1 (whole aligned vectors, IL divides VEC): a row is a contiguous [rin / IL, IL] slab reduced over its first
// dim; element e of the row belongs to output e % IL of the row, which is its place in its vector, and to index
// e / IL along the reduced dim. A thread keeps IL accumulators; output k of a row is out[row * IL + k].
template <class Op, int VEC, int SS = 1, bool RAG = false, bool UA = false, int IL = 1>
__global__ void __launch_bounds__(1024) row_lean_kernel(const RowLeanArgs a) {
    static_assert(!UA || (VEC > 1 && SS == 1 && !RAG), "UA is a full-vector mode of its own");
    static_assert(IL == 1 || (VEC % IL == 0 && SS == 1 && !RAG && !UA), "interleaved rows are whole aligned vectors");
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int UV = VEC / SS;
    __shared__ Acc smem[16 * IL];
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int row = blockIdx.x * a.rpb + ty;
    const bool valid = row < a.K;
    Acc accs[IL];
#pragma unroll
    for (int k = 0; k < IL; ++k) accs[k] = Op::identity();
    Acc& acc = accs[0];
    if (valid) {
        const T* p = (const T*)a.in + (int64_t)row * a.row_stride;
        int nvec = a.rin_v, head = 0;
        if constexpr (RAG) {
            head = min((int)(((16 - ((uintptr_t)p & 15)) & 15) / sizeof(T)), a.rin);
            nvec = (a.rin - head) / VEC;
            // (a lane meets its indices in growing order: head, vectors, tail)
            if (blockIdx.y == 0)
                for (int i = tx; i < head; i += tpr) fold_in<Op>(acc, p[i], i);
            p += head;
        }
        const int i0 = blockIdx.y * a.ichunk;
        const int i1 = min(nvec, i0 + a.ichunk);
        int iv = i0 + tx;
        if constexpr (VEC > 1) {
            auto load = [&](int i) {
                if constexpr (UA) return load_pack_unaligned<T, VEC>(p + min(i * VEC, a.rin - VEC));
                else return load_pack_stream<T, VEC>(p + (int64_t)i * VEC);
            };
            auto fold = [&](const Pack<T, VEC>& v, int i) {
                if constexpr (UA) {
                    const int e = i * VEC, from = min(e, a.rin - VEC);
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (from + j >= e) fold_in<Op>(acc, v.v[j], from + j);
                } else if constexpr (IL > 1) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) fold_in<Op>(accs[j % IL], v.v[j], i * (VEC / IL) + j / IL);
                } else {
#pragma unroll
                    for (int j = 0; j < UV; ++j) fold_in<Op>(acc, v.v[j * SS], head + i * UV + j);
                }
            };
            // batches of four loads in flight per lane before any is consumed
            for (; iv + 3 * tpr < i1; iv += 4 * tpr) {
                Pack<T, VEC> v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = load(iv + u * tpr);
#pragma unroll
                for (int u = 0; u < 4; ++u) fold(v[u], iv + u * tpr);
            }
            for (; iv < i1; iv += tpr) fold(load(iv), iv);
        } else {
#pragma unroll 4
            for (; iv < i1; iv += tpr) fold_in<Op>(acc, p[(int64_t)iv * a.sr], iv);
        }
        if constexpr (RAG) {
            if (blockIdx.y == 0)
                for (int i = nvec * VEC + tx; i < a.rin - head; i += tpr) fold_in<Op>(acc, p[i], head + i);
        }
    }
#pragma unroll
    for (int k = 0; k < IL; ++k) accs[k] = group_reduce<Op>(accs[k], tpr < 64 ? tpr : 64);
    if (tpr > 64) {
        const int wpr = tpr >> 6;  // wavefronts per row
        if ((threadIdx.x & 63) == 0) {
#pragma unroll
            for (int k = 0; k < IL; ++k) smem[(threadIdx.x >> 6) * IL + k] = accs[k];
        }
        __syncthreads();
        if (tx == 0)
            for (int w = 1; w < wpr; ++w) {
#pragma unroll
                for (int k = 0; k < IL; ++k) accs[k] = Op::comb(accs[k], smem[(ty * wpr + w) * IL + k]);
            }
    }
    if (tx == 0 && valid) {
        if constexpr (IL > 1) {
#pragma unroll
            for (int k = 0; k < IL; ++k) write_out<Op>(a.out, (int64_t)row * IL + k, accs[k], a.init_out, a.count);
        } else {
            if (a.split == 1) write_out<Op>(a.out, row, acc, a.init_out, a.count);
            else ((Acc*)a.out)[(int64_t)row * a.split + blockIdx.y] = acc;
        }
    }
}

// ---- rows that are [R, L] slabs, L no divisor of the vector -----------------------------------
// out[row * L + k] = reduce over c of in[row * rin + c * L + k], rin = R * L elements per row, rows back to back
// (a reduction over the middle axis of a contiguous [B, R, 3]: lanes along L idle, and the flat walk takes two
// launches and a workgroup per period). A row's lanes walk it with 128-bit loads; only the first `act` = the largest
// multiple of L lanes take part, so that a lane's vectors all start at the same place modulo L, (tx * VEC) % L: the
// lane keeps one accumulator per vector place and rotates them into the L outputs once, at the end. Rows start
// anywhere (unaligned loads); the elements after a row's last whole vector are folded one by one.
struct RowModArgs {
    const void* in;
    void* out;
    double count;
    int K;    // rows
    int rin;  // row length in elements, R * L
    int tpr, tpr_log2, rpb, init_out;
};

template <class Op, int VEC, int L>
__global__ void __launch_bounds__(256) row_mod_kernel(const RowModArgs a) {
    static_assert(VEC > 1 && VEC % L != 0 && L >= 3 && L <= 7, "inner dims that divide the vector run as interleaved rows");
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    __shared__ Acc smem[4 * L];
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int row = blockIdx.x * a.rpb + ty;
    const bool valid = row < a.K;
    const int act = tpr / L * L;
    Acc acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::identity();
    Acc cls[L];
#pragma unroll
    for (int k = 0; k < L; ++k) cls[k] = Op::identity();
    if (valid && tx < act) {
        const T* p = (const T*)a.in + (int64_t)row * a.rin;
        const int nvec = a.rin / VEC;
        auto fold = [&](const Pack<T, VEC>& v, int i) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v.v[j], (i * VEC + j) / L);
        };
        int iv = tx;
        for (; iv + 3 * act < nvec; iv += 4 * act) {
            Pack<T, VEC> v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = load_pack_unaligned<T, VEC>(p + (int64_t)(iv + u * act) * VEC);
#pragma unroll
            for (int u = 0; u < 4; ++u) fold(v[u], iv + u * act);
        }
        for (; iv < nvec; iv += act) fold(load_pack_unaligned<T, VEC>(p + (int64_t)iv * VEC), iv);
        // the lane's vector places as outputs: place j is output (tx * VEC + j) % L
        const int r = tx * VEC % L;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const int k = (r + j) % L;
#pragma unroll
            for (int kk = 0; kk < L; ++kk)
                if (kk == k) cls[kk] = Op::comb(cls[kk], acc[j]);
        }
        // fewer than VEC elements after the last whole vector
        const int e = nvec * VEC + tx;
        if (e < a.rin) {
            const T x = p[e];
#pragma unroll
            for (int kk = 0; kk < L; ++kk)
                if (kk == e % L) fold_in<Op>(cls[kk], x, e / L);
        }
    }
#pragma unroll
    for (int k = 0; k < L; ++k) cls[k] = group_reduce<Op>(cls[k], tpr < 64 ? tpr : 64);
    if (tpr > 64) {
        const int wpr = tpr >> 6;  // wavefronts per row (<= 4)
        if ((threadIdx.x & 63) == 0) {
#pragma unroll
            for (int k = 0; k < L; ++k) smem[(threadIdx.x >> 6) * L + k] = cls[k];
        }
        __syncthreads();
        if (tx == 0)
            for (int w = 1; w < wpr; ++w) {
#pragma unroll
                for (int k = 0; k < L; ++k) cls[k] = Op::comb(cls[k], smem[(ty * wpr + w) * L + k]);
            }
    }
    if (tx == 0 && valid) {
#pragma unroll
        for (int k = 0; k < L; ++k) write_out<Op>(a.out, (int64_t)row * L + k, cls[k], a.init_out, a.count);
    }
}

// ---- general row kernel ---------------------------------------------------------
struct RowArgs {
    const void* in;
    void* out;       // outputs, or partial accumulators when split > 1
    Dims kept;       // output index -> input offset
    Dims redo;       // outer reduced dims (all reduced dims but the innermost)
    int64_t K;       // outputs
    int64_t rout;    // product of redo sizes
    int64_t rin_v;   // innermost reduced length, in vectors
    int64_t rin;     // innermost reduced length, in elements (UA)
    int64_t sr;      // innermost reduced stride in elements (1 when VEC > 1)
    int64_t qchunk;  // outer reduced indices per split
    int64_t ichunk;  // inner vectors per split
    double count;    // elements reduced per output (mean)
    int tpr, tpr_log2, rpb, split_q, split_i, init_out;
    // > 0: workgroup x takes row block (x % 8) * xcd_chunk + x / 8 (gridDim.x = 8 * xcd_chunk). Workgroups are
    // dealt round-robin to the chip's eight XCDs, each with an L2 of its own: numbered this way, the row blocks
    // that run on one XCD at a time are neighbours, and when neighbouring rows' runs share cache lines (runs of
    // 320 bytes laid back to back) a line is fetched from memory once instead of once per XCD that needs it.
    int xcd_chunk;
};

// Vector iv of a run of `rin` contiguous elements at p. UA (runs that are not whole, aligned
// vectors): an unaligned load; the run's last vector is taken from its end backwards and the
// elements it shares with the vector before are skipped.
template <class T, int VEC, bool UA>
__device__ __forceinline__ Pack<T, VEC> row_vec_load(const T* p, int64_t iv, int64_t rin) {
    if constexpr (UA) return load_pack_unaligned<T, VEC>(p + min(iv * VEC, rin - VEC));
    else return load_pack_stream<T, VEC>(p + iv * VEC);
}
template <class Op, int VEC, bool UA>
__device__ __forceinline__ void row_vec_fold(typename Op::Acc& acc, const Pack<typename Op::In, VEC>& v, int64_t iv,
                                             int64_t rin) {
    const int64_t e = iv * VEC, from = UA ? min(e, rin - VEC) : e;
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        if (!UA || from + j >= e) fold_in<Op>(acc, v.v[j], from + j);
}

template <class Op, int VEC, bool UA>
__device__ __forceinline__ void row_step(typename Op::Acc& acc, const typename Op::In* p, int64_t iv,
                                         int64_t sr, int64_t rin) {
    using T = typename Op::In;
    if constexpr (VEC > 1) row_vec_fold<Op, VEC, UA>(acc, row_vec_load<T, VEC, UA>(p, iv, rin), iv, rin);
    else fold_in<Op>(acc, p[iv * sr], iv);
}

template <class Op, int VEC, bool UA = false>
__global__ void __launch_bounds__(1024) row_reduce_kernel(const RowArgs a) {
    static_assert(!UA || VEC > 1, "UA is a full-vector mode");
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    __shared__ Acc smem[16];

    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int64_t rb = a.xcd_chunk > 0 ? (int64_t)(blockIdx.x & 7) * a.xcd_chunk + (blockIdx.x >> 3) : (int64_t)blockIdx.x;
    const int64_t row = rb * a.rpb + ty;
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
        if (q1 - q0 <= 1) {
            if (q0 < q1) {
                const T* p = base + offset_of(a.redo, q0);
#pragma unroll 4
                for (int64_t iv = i0 + tx; iv < i1; iv += tpr) row_step<Op, VEC, UA>(acc, p, iv, a.sr, a.rin);
            }
        } else if (ni > 0) {
            // Several outer reduced indices, each with an inner run of ni vectors (the sums of a
            // batch norm: [N, C, H*W] over N and H*W): the lanes walk the (outer, inner) pairs as ONE
            // flat range, so a run that is not a multiple of the group size wastes no lanes, with
            // four loads in flight per lane. The pair of a lane advances by a fixed (outer, inner)
            // step: one division up front, none in the loop.
            const int64_t total = (q1 - q0) * ni;
            int64_t dq, di;
            if (((uint64_t)(tx | ni) >> 32) == 0) {
                dq = (uint32_t)tx / (uint32_t)ni;
                di = (uint32_t)tx - (uint32_t)dq * (uint32_t)ni;
            } else {
                dq = tx / ni;
                di = tx - dq * ni;
            }
            const int64_t step_q = tpr / ni, step_i = tpr - step_q * ni;
            auto advance = [&]() {
                dq += step_q;
                di += step_i;
                if (di >= ni) {
                    di -= ni;
                    ++dq;
                }
            };
            int64_t t = tx;
            for (; t + 3 * (int64_t)tpr < total; t += 4 * (int64_t)tpr) {
                const T* p[4];
                int64_t iv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    p[u] = base + offset_of(a.redo, q0 + dq);
                    iv[u] = i0 + di;
                    advance();
                }
                if constexpr (VEC > 1) {
                    Pack<T, VEC> v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = row_vec_load<T, VEC, UA>(p[u], iv[u], a.rin);
#pragma unroll
                    for (int u = 0; u < 4; ++u) row_vec_fold<Op, VEC, UA>(acc, v[u], iv[u], a.rin);
                } else {
                    T v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = p[u][iv[u] * a.sr];
#pragma unroll
                    for (int u = 0; u < 4; ++u) fold_in<Op>(acc, v[u], iv[u]);
                }
            }
            for (; t < total; t += tpr) {
                row_step<Op, VEC, UA>(acc, base + offset_of(a.redo, q0 + dq), i0 + di, a.sr, a.rin);
                advance();
            }
        }
    }

    acc = group_reduce<Op>(acc, tpr < 64 ? tpr : 64);
    if (tpr > 64) {
        const int wpr = tpr >> 6;
        if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (tx == 0)
            for (int w = 1; w < wpr; ++w) acc = Op::comb(acc, smem[ty * wpr + w]);
    }
    if (tx == 0 && valid) {
        const int split = a.split_q * a.split_i;
        if (split == 1) write_out<Op>(a.out, row, acc, a.init_out, a.count);
        else ((Acc*)a.out)[row * split + blockIdx.y] = acc;
    }
}

// ---- column kernels ---------------------------------------------------------------
// Fold the `by` thread rows of a workgroup into row 0.
template <class Op, int VEC>
__device__ __forceinline__ void fold_thread_rows(typename Op::Acc (&acc)[VEC], typename Op::Acc* smem) {
    const int bx = blockDim.x, by = blockDim.y;
    const int tx = threadIdx.x, ty = threadIdx.y;
    if (by == 1) return;
    if (by <= 4) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) smem[((size_t)ty * bx + tx) * VEC + j] = acc[j];
        __syncthreads();
        if (ty == 0) {
            for (int y = 1; y < by; ++y) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = Op::comb(acc[j], smem[((size_t)y * bx + tx) * VEC + j]);
            }
        }
        return;
    }
    // Many thread rows (a narrow inner dim): halve them step by step; rows [s, 2s) hand their
    // values to rows [0, s) through LDS. The pairing is fixed, so the result is deterministic.
    int top = 1;
    while (top < by) top <<= 1;
    for (int s = top >> 1; s >= 1; s >>= 1) {
        if (ty >= s && ty < 2 * s) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) smem[((size_t)(ty - s) * bx + tx) * VEC + j] = acc[j];
        }
        __syncthreads();
        if (ty < s && ty + s < by) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = Op::comb(acc[j], smem[((size_t)ty * bx + tx) * VEC + j]);
        }
        __syncthreads();
    }
}

// Short rows laid back to back (a contiguous [K, R] matrix, R * sizeof(T) <= 1 KiB): a workgroup
// stages `rows_per_wg` consecutive rows (16 KiB, a multiple of VEC rows so that the tile starts
// on a 16-byte boundary) in LDS with aligned 128-bit loads, then groups of `tpr` lanes reduce
// the rows out of LDS. HBM sees only whole, aligned lines whatever R is.
struct RowTileArgs {
    const void* in;
    void* out;
    int64_t K;   // rows
    double count;
    int R;       // row length
    int rows_per_wg;
    int tpr, tpr_log2;
    int init_out;
};

template <class Op, int VEC>
__global__ void __launch_bounds__(256) row_tile_kernel(const RowTileArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int NV = 4;  // vectors per thread: 256 * 4 * 16 bytes = 16 KiB
    __shared__ __align__(16) unsigned char tile_raw[256 * NV * 16];
    T* tile = reinterpret_cast<T*>(tile_raw);
    const int t = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t left = a.K - row0;
    const int nrows = left < a.rows_per_wg ? (int)left : a.rows_per_wg;
    const int n = nrows * a.R;  // elements of this tile
    const T* src = (const T*)a.in + row0 * a.R;
    Pack<T, VEC> v[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e + VEC <= n) {
            v[u] = load_pack_stream<T, VEC>(src + e);
        } else {  // the tensor's last, partial vector
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                if (e + j < n) v[u].v[j] = src[e + j];
        }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e < n) store_pack<T, VEC>(tile + e, v[u]);
    }
    __syncthreads();
    const int tx = t & (a.tpr - 1);
    const int g = t >> a.tpr_log2;
    const int groups = 256 >> a.tpr_log2;
    for (int r = g; r < nrows; r += groups) {
        Acc acc = Op::identity();
        const T* row = tile + r * a.R;
        for (int c = tx; c < a.R; c += a.tpr) fold_in<Op>(acc, row[c], c);
        acc = group_reduce<Op>(acc, a.tpr);
        if (tx == 0) write_out<Op>(a.out, row0 + r, acc, a.init_out, a.count);
    }
}

// Small groups laid back to back (a contiguous [outer, R, kin] tensor reduced over R with R * kin
// small: [N, 2, 3], [N, 3, 16], [N, 4, 12]): lanes along kin would leave most of a wavefront idle and a
// lane per output reads single elements at a stride. As in row_tile_kernel a workgroup stages 16 KiB of
// whole groups in LDS with aligned 128-bit loads; then one lane per output folds its R elements out of LDS.
struct GroupTileArgs {
    const void* in;
    void* out;
    int64_t groups;  // outer
    double count;
    int R, kin;
    int groups_per_wg;
    int init_out;
};

template <class Op, int VEC, bool PADDED>
__global__ void __launch_bounds__(256) group_tile_kernel(const GroupTileArgs a) {
    constexpr bool padded = PADDED;
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int NV = 4;  // vectors per thread: 256 * 4 * 16 bytes = 16 KiB
    // One pad slot of 4 bytes (one 8-byte element) after every 128 bytes of the tile: the lanes of a
    // wavefront start whole groups apart, and a group of 128 bytes or a multiple would put them all on
    // the same LDS bank.
    constexpr int PER = 128 / sizeof(T);                     // elements between pad slots
    constexpr int PAD = sizeof(T) >= 4 ? 1 : 4 / sizeof(T);  // elements per pad slot
    // (PADDED only where the groups' starts would collide: the pad costs the vector LDS accesses)
    auto pad = [](int e) { return PADDED ? e + e / PER * PAD : e; };
    __shared__ __align__(16) unsigned char tile_raw[256 * NV * 16 + (256 * NV * 16 / 128) * 8];
    T* tile = reinterpret_cast<T*>(tile_raw);
    const int t = threadIdx.x;
    const int G = a.R * a.kin;
    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t left = a.groups - g0;
    const int ngroups = left < a.groups_per_wg ? (int)left : a.groups_per_wg;
    const int n = ngroups * G;  // elements of this tile
    const T* src = (const T*)a.in + g0 * G;
    Pack<T, VEC> v[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e + VEC <= n) {
            v[u] = load_pack_stream<T, VEC>(src + e);
        } else {  // the tensor's last, partial vector
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                if (e + j < n) v[u].v[j] = src[e + j];
        }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e < n) {
            if constexpr (!padded) {
                store_pack<T, VEC>(tile + e, v[u]);
            } else {
                T* q = tile + pad(e);  // a 16-byte vector never straddles a pad slot
#pragma unroll
                for (int j = 0; j < VEC; ++j) q[j] = v[u].v[j];
            }
        }
    }
    __syncthreads();
    const int nout = ngroups * a.kin;
    for (int o = t; o < nout; o += 256) {
        const int g = o / a.kin, i = o - g * a.kin;
        const int base = g * G + i;
        Acc acc = Op::identity();
        for (int r = 0; r < a.R; ++r) fold_in<Op>(acc, tile[pad(base + r * a.kin)], r);
        write_out<Op>(a.out, g0 * a.kin + o, acc, a.init_out, a.count);
    }
}

// Lean form: outputs are (outer, inner) with inner the lane dim; one reduced dim.
// out[outer * kin + inner] = reduce over r of in[outer * so + r * rs + inner * sk].
struct ColLeanArgs {
    const void* in;
    void* out;       // outputs, or partials [split][K] when split > 1
    int64_t so;      // stride of the outer kept dim
    int64_t rs;      // stride of the reduced dim
    int64_t K;       // outputs
    double count;
    int kin_v;       // inner kept length in vectors
    int sk;          // inner kept stride in elements (1 when VEC > 1)
    int R;           // reduced length
    int split, init_out;
    int64_t oso, osi;  // output strides of the outer / inner kept index (kin and 1 unless the kept dims were swapped)
    int vec_out;       // the outputs of a lane may be stored as vectors: overwrite mode, unit stride, aligned
    int kin;           // inner kept length in elements (UA: kin_v = ceil(kin / VEC))
};

// UA: the rows are not whole, aligned vectors. A lane takes VEC neighbouring outputs all the same, with
// unaligned 128-bit loads; the last lane of a row, which has fewer, loads them one by one.
template <class Op, int VEC, int SS = 1, bool UA = false>
__global__ void __launch_bounds__(1024) col_lean_kernel(const ColLeanArgs a) {
    static_assert(!UA || (VEC > 1 && SS == 1), "UA is a full-vector mode");
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    constexpr int UV = VEC / SS;  // outputs per lane (SS = 2: every second position of a vector)
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tx = threadIdx.x, ty = threadIdx.y, by = blockDim.y;
    const int cv = blockIdx.x * blockDim.x + tx;  // vector column in the inner dim
    const int outer = blockIdx.y;
    const bool valid = cv < a.kin_v;
    // UA: outputs of this lane (VEC except in the last lane of a row)
    const int cnt = UA ? (a.kin - cv * VEC < VEC ? a.kin - cv * VEC : VEC) : UV;
    Acc acc[UV];
#pragma unroll
    for (int j = 0; j < UV; ++j) acc[j] = Op::identity();
    auto load = [&](const T* p) {
        Pack<T, VEC> v;
        if constexpr (UA) {
            if (cnt == VEC) {
                v = load_pack_unaligned<T, VEC>(p);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v.v[j] = j < cnt ? p[j] : p[0];
            }
        } else if constexpr (VEC > 1) {
            v = load_pack_stream<T, VEC>(p);
        } else {
            v.v[0] = *p;
        }
        return v;
    };
    if (valid) {
        const T* base = (const T*)a.in + (int64_t)outer * a.so + (int64_t)cv * (VEC > 1 ? VEC : a.sk);
        // The reduced range is dealt out round-robin: thread row ty of workgroup z takes
        // r = z * by + ty, then steps by (by * splits). Wavefronts that run at the same
        // time therefore read neighbouring rows, which keeps a power-of-two row pitch
        // from sending them all to the same memory channels.
        const int step = by * a.split;
        int r = blockIdx.z * by + ty;
        // batches of eight loads in flight per lane before any is consumed: with one
        // wavefront per 64 columns this is what keeps the memory pipeline full
        for (; r + 7 * step < a.R; r += 8 * step) {
            Pack<T, VEC> v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = load(base + (int64_t)(r + u * step) * a.rs);
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int j = 0; j < UV; ++j) fold_in<Op>(acc[j], v[u].v[j * SS], r + u * step);
        }
        for (; r < a.R; r += step) {
            const Pack<T, VEC> v = load(base + (int64_t)r * a.rs);
#pragma unroll
            for (int j = 0; j < UV; ++j) fold_in<Op>(acc[j], v.v[j * SS], r);
        }
    }
    fold_thread_rows<Op, UV>(acc, (Acc*)smem_raw);
    if (ty == 0 && valid) {
        if constexpr (UA) {
            // (the lanes of a row do not all have VEC outputs: element by element)
            const int64_t ov = (int64_t)outer * a.kin + (int64_t)cv * VEC;  // in the kernel's numbering
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if (j >= cnt) break;
                if (a.split == 1)
                    write_out<Op>(a.out, (int64_t)outer * a.oso + ((int64_t)cv * VEC + j) * a.osi, acc[j], a.init_out, a.count);
                else
                    ((Acc*)a.out)[(int64_t)blockIdx.z * a.K + ov + j] = acc[j];
            }
            return;
        }
        const int64_t o0 = ((int64_t)outer * a.kin_v + cv) * UV;
        if (a.split == 1) {
            if (UV > 1 && a.vec_out) {
                // a lane's UV outputs are neighbours in memory: whole vectors (the outputs are half the
                // traffic when few elements are reduced into each)
                write_out_pack<Op, UV>(a.out, (int64_t)outer * a.oso + (int64_t)cv * UV, acc, a.count);
            } else {
#pragma unroll
                for (int j = 0; j < UV; ++j)
                    write_out<Op>(a.out, (int64_t)outer * a.oso + ((int64_t)cv * UV + j) * a.osi, acc[j], a.init_out,
                                  a.count);
            }
        } else {
#pragma unroll
            for (int j = 0; j < UV; ++j) ((Acc*)a.out)[(int64_t)blockIdx.z * a.K + o0 + j] = acc[j];
        }
    }
}

// A contiguous [R, kin] slab per outer index whose rows are not whole vectors, walked as a flat
// array: thread t owns elements [t * VEC, t * VEC + VEC) of every period of L = threads * VEC
// elements. L is a multiple of kin, so slot (t, j) always sees column (t * VEC + j) % kin and
// row (t * VEC + j) / kin + period * (L / kin). All loads are aligned 128-bit vectors whatever kin is.
struct ColFlatArgs {
    const void* in;
    void* out;      // outputs, or partials [split][K] when split > 1
    int64_t so;     // stride of the outer kept dim
    int64_t total;  // elements per outer index: R * kin
    int64_t K;      // outputs: outer * kin
    double count;
    int kin;        // inner kept length (columns)
    int threads;    // threads that take part (a multiple of kin / gcd(kin, VEC))
    int split, init_out;
};

// UA: the slabs do not start on 16-byte boundaries (an odd slab size): the same vectors, unaligned.
template <class Op, int VEC, bool UA = false>
__global__ void __launch_bounds__(1024) col_flat_kernel(const ColFlatArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Acc* smem = (Acc*)smem_raw;
    auto flat_load = [](const T* p) {
        if constexpr (UA) return load_pack_unaligned<T, VEC>(p);
        else return load_pack_stream<T, VEC>(p);
    };
    const int t = threadIdx.x;
    const int outer = blockIdx.y;
    const int L = a.threads * VEC;
    const int rows_per_period = L / a.kin;
    const int p0 = t * VEC;
    Acc acc[VEC];
    int row[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        acc[j] = Op::identity();
        row[j] = (p0 + j) / a.kin;
    }
    if (t < a.threads) {
        const T* base = (const T*)a.in + (int64_t)outer * a.so;
        const int64_t whole = a.total / L;  // periods that lie wholly inside the slab
        const int split = a.split;
        int64_t it = blockIdx.z;  // periods are dealt round-robin over the workgroups of a slab
        // Batches of four vectors, two batches alternating: the next batch is in flight while the
        // current one is folded in. (Its loads are issued unconditionally, from a repeated address
        // on the last round: a load under a branch would make the wait before the fold a full one.)
        auto load4 = [&](Pack<T, VEC>(&v)[4], int64_t i0) {
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = flat_load(base + (i0 + u * split) * L + p0);
        };
        auto fold4 = [&](const Pack<T, VEC>(&v)[4], int64_t i0) {
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    fold_in<Op>(acc[j], v[u].v[j], row[j] + (int)(i0 + u * split) * rows_per_period);
        };
        const int64_t step = 4 * (int64_t)split;
        if (it + 3 * split < whole) {
            Pack<T, VEC> va[4], vb[4];
            load4(va, it);
            for (;;) {
                int64_t nx = it + step;
                bool more = nx + 3 * split < whole;
                load4(vb, more ? nx : it);
                fold4(va, it);
                it = nx;
                if (!more) break;
                nx = it + step;
                more = nx + 3 * split < whole;
                load4(va, more ? nx : it);
                fold4(vb, it);
                it = nx;
                if (!more) break;
            }
        }
        for (; it < whole; it += split) {
            Pack<T, VEC> v = flat_load(base + it * L + p0);
#pragma unroll
            for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v.v[j], row[j] + (int)it * rows_per_period);
        }
        if (it == whole) {  // the last, partial period: element by element
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int64_t pos = whole * L + p0 + j;
                if (pos < a.total) fold_in<Op>(acc[j], base[pos], row[j] + (int)whole * rows_per_period);
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) smem[p0 + j] = acc[j];
    }
    __syncthreads();
    // Slot p holds column p % kin: fold the L / kin slot rows pairwise, upper half into lower half.
    int top = 1;
    while (top < rows_per_period) top <<= 1;
    for (int s = top >> 1; s >= 1; s >>= 1) {
        const int n = s * a.kin;
        for (int i = t; i < n; i += blockDim.x)
            if (i + n < L) smem[i] = Op::comb(smem[i], smem[i + n]);
        __syncthreads();
    }
    for (int c = t; c < a.kin; c += blockDim.x) {
        const int64_t o = (int64_t)outer * a.kin + c;
        if (a.split == 1) write_out<Op>(a.out, o, smem[c], a.init_out, a.count);
        else ((Acc*)a.out)[(int64_t)blockIdx.z * a.K + o] = smem[c];
    }
}

// The same flat walk for rows wider than a workgroup can cover: the period (phases rows, the
// shortest run after which row starts repeat their alignment) is spread over gridDim.x workgroups.
// Each vector slot is then a single (row phase, column) pair; the partials are [slice][phase][K].
struct ColFlatWideArgs {
    const void* in;
    void* partial;
    int64_t so;      // stride of the outer kept dim
    int64_t total;   // elements per outer index: R * kin
    int64_t K;       // outputs: outer * kin
    int kin;         // inner kept length (columns)
    int vecs;        // vectors per period: kin * phases / VEC
    int phases;      // rows per period
    int slices;      // workgroups along the reduced range
};

template <class Op, int VEC>
__global__ void __launch_bounds__(1024) col_flat_wide_kernel(const ColFlatWideArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    const int q = blockIdx.x * blockDim.x + threadIdx.x;  // vector within the period
    if (q >= a.vecs) return;
    const int outer = blockIdx.y;
    const int64_t L = (int64_t)a.vecs * VEC;
    const int p0 = q * VEC;
    Acc acc[VEC];
    int row[VEC], col[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        acc[j] = Op::identity();
        row[j] = (p0 + j) / a.kin;
        col[j] = (p0 + j) - row[j] * a.kin;
    }
    const T* base = (const T*)a.in + (int64_t)outer * a.so;
    const int64_t whole = a.total / L;
    const int slices = a.slices;
    int64_t it = blockIdx.z;
    // two alternating batches of four vectors, as in col_flat_kernel
    auto load4 = [&](Pack<T, VEC>(&v)[4], int64_t i0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = load_pack_stream<T, VEC>(base + (i0 + u * slices) * L + p0);
    };
    auto fold4 = [&](const Pack<T, VEC>(&v)[4], int64_t i0) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v[u].v[j], row[j] + (int)(i0 + u * slices) * a.phases);
    };
    const int64_t step = 4 * (int64_t)slices;
    if (it + 3 * slices < whole) {
        Pack<T, VEC> va[4], vb[4];
        load4(va, it);
        for (;;) {
            int64_t nx = it + step;
            bool more = nx + 3 * slices < whole;
            load4(vb, more ? nx : it);
            fold4(va, it);
            it = nx;
            if (!more) break;
            nx = it + step;
            more = nx + 3 * slices < whole;
            load4(va, more ? nx : it);
            fold4(vb, it);
            it = nx;
            if (!more) break;
        }
    }
    for (; it < whole; it += slices) {
        Pack<T, VEC> v = load_pack_stream<T, VEC>(base + it * L + p0);
#pragma unroll
        for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v.v[j], row[j] + (int)it * a.phases);
    }
    if (it == whole) {  // the last, partial period
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const int64_t pos = whole * L + p0 + j;
            if (pos < a.total) fold_in<Op>(acc[j], base[pos], row[j] + (int)whole * a.phases);
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        ((Acc*)a.partial)[((int64_t)blockIdx.z * a.phases + row[j]) * a.K + (int64_t)outer * a.kin + col[j]] = acc[j];
}

struct ColArgs {
    const void* in;
    void* out;        // outputs, or partials [split][K] when split > 1
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

template <class Op, int VEC>
__global__ void __launch_bounds__(1024) col_reduce_kernel(const ColArgs a) {
    using T = typename Op::In;
    using Acc = typename Op::Acc;
    extern __shared__ __align__(16) unsigned char smem_raw[];

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
        int64_t r = r0 + ty;
        for (; r + 7 * by < r1; r += 8 * by) {  // eight reduced positions in flight per lane
            const T* p[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) p[u] = base + offset_of(a.red, r + u * by);
            if constexpr (VEC > 1) {
                Pack<T, VEC> v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = load_pack_stream<T, VEC>(p[u]);
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v[u].v[j], r + u * by);
            } else {
                T v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = *p[u];
#pragma unroll
                for (int u = 0; u < 8; ++u) fold_in<Op>(acc[0], v[u], r + u * by);
            }
        }
        for (; r < r1; r += by) {
            const T* p = base + offset_of(a.red, r);
            if constexpr (VEC > 1) {
                Pack<T, VEC> v = load_pack_stream<T, VEC>(p);
#pragma unroll
                for (int j = 0; j < VEC; ++j) fold_in<Op>(acc[j], v.v[j], r);
            } else {
                fold_in<Op>(acc[0], *p, r);
            }
        }
    }
    fold_thread_rows<Op, VEC>(acc, (Acc*)smem_raw);
    if (ty == 0 && valid) {
        if (a.split == 1) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) write_out<Op>(a.out, o0 + j, acc[j], a.init_out, a.count);
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) ((Acc*)a.out)[(int64_t)blockIdx.y * a.K + o0 + j] = acc[j];
        }
    }
}

// ---- second stage: fold the partials of the outputs that were split ---------------
// finish_rows_kernel: few outputs with many partials each (row splits; partial s of
// output o at part[o * split + s]): a workgroup folds one output.
template <class Op>
__global__ void __launch_bounds__(256) finish_rows_kernel(const void* part_, void* out, int split, int init_out,
                                                          double count) {
    using Acc = typename Op::Acc;
    const Acc* part = (const Acc*)part_;
    __shared__ Acc smem[16];
    const int64_t o = blockIdx.x;
    Acc acc = Op::identity();
    for (int s = threadIdx.x; s < split; s += blockDim.x) acc = Op::comb(acc, part[o * split + s]);
    acc = block_reduce<Op>(acc, smem);
    if (threadIdx.x == 0) write_out<Op>(out, o, acc, init_out, count);
}

// finish_rows_thin_kernel: the same partials when every output has only a few (split <= 16: sum([0, 2, 3]) of
// [64, 128, 56, 56] has 128 outputs of 4): a thread folds one output, in the order of the partials, and the whole
// launch is one or two workgroups instead of one per output.
template <class Op>
__global__ void __launch_bounds__(256) finish_rows_thin_kernel(const void* part_, void* out, int64_t K, int split, int init_out,
                                                               double count) {
    using Acc = typename Op::Acc;
    const Acc* part = (const Acc*)part_;
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= K) return;
    Acc v[16];
#pragma unroll
    for (int s = 0; s < 16; ++s)
        if (s < split) v[s] = part[o * split + s];
    Acc acc = v[0];
#pragma unroll
    for (int s = 1; s < 16; ++s)
        if (s < split) acc = Op::comb(acc, v[s]);
    write_out<Op>(out, o, acc, init_out, count);
}

// finish_cols_kernel: many outputs (column splits; partial s of output o at
// part[s * K + o]): 64 neighbouring outputs per workgroup, the partials of each dealt
// over blockDim.y thread rows so that no thread walks a long chain of dependent
// loads, then folded through LDS.
template <class Op>
__global__ void __launch_bounds__(1024) finish_cols_kernel(const void* part_, void* out, int64_t K, int split,
                                                           int init_out, double count, int64_t kin, int64_t oso,
                                                           int64_t osi) {
    using Acc = typename Op::Acc;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Acc* sm = (Acc*)smem_raw;
    const Acc* part = (const Acc*)part_;
    const int tx = threadIdx.x, ty = threadIdx.y, by = blockDim.y;
    const int64_t o = (int64_t)blockIdx.x * 64 + tx;
    const bool valid = o < K;
    Acc acc = Op::identity();
    if (valid) {
        // eight partials in flight per thread (the kernel is a chain of load latencies otherwise)
        const Acc* p = part + o;
        int s = ty;
        for (; s + 7 * by < split; s += 8 * by) {
            Acc v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p[(int64_t)(s + u * by) * K];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = Op::comb(acc, v[u]);
        }
        for (; s < split; s += by) acc = Op::comb(acc, p[(int64_t)s * K]);
    }
    if (by > 1) {
        sm[ty * 64 + tx] = acc;
        __syncthreads();
        if (ty == 0)
            for (int y = 1; y < by; ++y) acc = Op::comb(acc, sm[y * 64 + tx]);
    }
    // output o of the kernel's (outer, inner) numbering sits at outer * oso + inner * osi
    if (ty == 0 && valid) write_out<Op>(out, (o / kin) * oso + (o % kin) * osi, acc, init_out, count);
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
    using Acc = typename Op::Acc;
    constexpr int FULL = 16 / sizeof(T);
    const double count = (double)p.R;
    if (p.kind == ReduceKind::Empty) return;
    if (p.kind == ReduceKind::Identity) {
        int64_t blocks = (p.K + 255) / 256;
        identity_fill_kernel<Op><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(out, p.K, init_out, count);
        return;
    }
    const bool vec = p.vec == FULL && FULL > 1;
    void* stage1_out = p.split > 1 ? sc.partial : out;
    if (p.kind == ReduceKind::Col && p.group_tile > 0) {
        if constexpr (FULL > 1) {
            GroupTileArgs a{};
            a.in = in;
            a.out = out;
            a.groups = p.kept.size[0];
            a.count = count;
            a.R = (int)p.R;
            a.kin = (int)p.kept.size[1];
            a.groups_per_wg = p.group_tile;
            a.init_out = init_out;
            // a narrow inner dim with groups of a multiple of 32 bytes: the lanes' group starts collide in LDS
            // (a very narrow inner dim with groups of a multiple of 128 bytes: 16 or more of a wavefront's lanes
            // would start on the same LDS bank. Measured: f32 [N, 16, 2] softmax 2.2 -> 5.8 TB/s padded; wider inner
            // dims or other group sizes lose up to a quarter to the pad's scalar LDS accesses.)
            const bool padded = a.kin * (int)sizeof(T) <= 16 && (a.R * a.kin * (int)sizeof(T)) % 128 == 0;
            const dim3 grid((unsigned)((a.groups + p.group_tile - 1) / p.group_tile));
            if (padded) group_tile_kernel<Op, FULL, true><<<grid, dim3(256), 0, st>>>(a);
            else group_tile_kernel<Op, FULL, false><<<grid, dim3(256), 0, st>>>(a);
        }
        return;
    }
    if (p.kind == ReduceKind::Row && p.row_tile > 0) {
        if constexpr (FULL > 1) {
            RowTileArgs a{};
            a.in = in;
            a.out = out;
            a.K = p.K;
            a.count = count;
            a.R = (int)p.R;
            a.rows_per_wg = p.row_tile;
            a.tpr = p.tpr;
            a.tpr_log2 = ilog2(p.tpr);
            a.init_out = init_out;
            row_tile_kernel<Op, FULL><<<dim3((unsigned)((p.K + p.row_tile - 1) / p.row_tile)), dim3(256), 0, st>>>(a);
        }
        return;
    }
    if (p.kind == ReduceKind::Row && p.mod_rows > 0) {
        if constexpr (FULL > 1) {
            if (p.vec != FULL || p.split != 1 || p.K % p.mod_rows != 0 || p.tpr * p.rpb != 256 || p.tpr < 64 ||
                p.R * p.mod_rows >= (1ll << 30))
                fail(HPT_ERR_KERNEL, "rows of [R, L] slabs: 256-thread workgroups of whole rows");
            const int64_t rows = p.K / p.mod_rows;
            const dim3 grid((unsigned)((rows + p.rpb - 1) / p.rpb));
            RowModArgs a{};
            a.in = in;
            a.out = out;
            a.count = count;
            a.K = (int)rows;
            a.rin = (int)(p.R * p.mod_rows);
            a.tpr = p.tpr;
            a.tpr_log2 = ilog2(p.tpr);
            a.rpb = p.rpb;
            a.init_out = init_out;
            switch (p.mod_rows) {
                case 3: row_mod_kernel<Op, FULL, 3><<<grid, dim3(256), 0, st>>>(a); return;
                // (eight-byte elements: four is no divisor of their two-element vector)
                case 4: if constexpr (FULL == 2) { row_mod_kernel<Op, FULL, 4><<<grid, dim3(256), 0, st>>>(a); return; } break;
                case 5: row_mod_kernel<Op, FULL, 5><<<grid, dim3(256), 0, st>>>(a); return;
                case 6: row_mod_kernel<Op, FULL, 6><<<grid, dim3(256), 0, st>>>(a); return;
                case 7: row_mod_kernel<Op, FULL, 7><<<grid, dim3(256), 0, st>>>(a); return;
                default: break;
            }
        }
        fail(HPT_ERR_KERNEL, "rows of [R, L] slabs: L = %d", p.mod_rows);
    }
    if (p.kind == ReduceKind::Row && p.interleave > 1) {
        // rows that are [R, interleave] slabs: the lean kernel over rows of R * interleave elements
        if (!p.lean || !vec || p.split != 1 || p.sstride != 1 || p.ragged || p.unaligned || FULL % p.interleave != 0 ||
            p.K % p.interleave != 0 || (p.R * p.interleave) % FULL != 0)
            fail(HPT_ERR_KERNEL, "interleaved rows need whole aligned vectors and one workgroup per row");
        const int64_t rows = p.K / p.interleave;
        const dim3 grid((unsigned)((rows + p.rpb - 1) / p.rpb));
        const dim3 block((unsigned)(p.tpr * p.rpb));
        RowLeanArgs a{};
        a.in = in;
        a.out = out;
        a.row_stride = p.R * p.interleave;
        a.count = count;
        a.K = (int)rows;
        a.rin_v = (int)(p.R * p.interleave / FULL);
        a.rin = (int)(p.R * p.interleave);
        a.sr = 1;
        a.ichunk = a.rin_v;
        a.tpr = p.tpr;
        a.tpr_log2 = ilog2(p.tpr);
        a.rpb = p.rpb;
        a.split = 1;
        a.init_out = init_out;
        if constexpr (FULL >= 2) {
            if (p.interleave == 2) { row_lean_kernel<Op, FULL, 1, false, false, 2><<<grid, block, 0, st>>>(a); return; }
        }
        if constexpr (FULL >= 4) {
            if (p.interleave == 4) { row_lean_kernel<Op, FULL, 1, false, false, 4><<<grid, block, 0, st>>>(a); return; }
        }
        if constexpr (FULL >= 8) {
            if (p.interleave == 8) { row_lean_kernel<Op, FULL, 1, false, false, 8><<<grid, block, 0, st>>>(a); return; }
        }
        fail(HPT_ERR_KERNEL, "interleaved rows: %d outputs per row", p.interleave);
    }
    if (p.kind == ReduceKind::Row) {
        dim3 grid((unsigned)((p.K + p.rpb - 1) / p.rpb), (unsigned)p.split);
        dim3 block((unsigned)(p.tpr * p.rpb));
        const int64_t rin = p.red.size[p.red.n - 1];
        if (p.lean) {
            RowLeanArgs a{};
            a.in = in;
            a.out = stage1_out;
            a.row_stride = p.kept.n ? p.kept.stride[0] : 0;
            a.count = count;
            a.K = (int)p.K;
            a.rin_v = (int)((rin + (p.unaligned ? p.vec - 1 : 0)) / (p.vec / p.sstride));
            a.rin = (int)rin;
            a.sr = (int)p.red.stride[0];
            a.ichunk = (a.rin_v + p.split - 1) / p.split;
            a.tpr = p.tpr;
            a.tpr_log2 = ilog2(p.tpr);
            a.rpb = p.rpb;
            a.split = p.split;
            a.init_out = init_out;
            if (vec && p.sstride == 2) row_lean_kernel<Op, FULL, 2><<<grid, block, 0, st>>>(a);
            else if (vec && p.ragged) row_lean_kernel<Op, FULL, 1, true><<<grid, block, 0, st>>>(a);
            else if (vec && p.unaligned) row_lean_kernel<Op, FULL, 1, false, true><<<grid, block, 0, st>>>(a);
            else if (vec) row_lean_kernel<Op, FULL><<<grid, block, 0, st>>>(a);
            else row_lean_kernel<Op, 1><<<grid, block, 0, st>>>(a);
        } else {
            RowArgs a{};
            a.in = in;
            a.out = stage1_out;
            a.kept = p.kept;
            a.redo = p.red;
            a.redo.n = p.red.n - 1;
            a.K = p.K;
            a.rout = p.R / rin;
            a.rin_v = (rin + (p.unaligned ? p.vec - 1 : 0)) / p.vec;
            a.rin = rin;
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
            // neighbouring outputs whose runs lie within a few lines of each other: number the row blocks per XCD
            if (p.kept.n >= 1 && grid.x >= 64) {
                const int64_t ks = p.kept.stride[p.kept.n - 1] < 0 ? -p.kept.stride[p.kept.n - 1] : p.kept.stride[p.kept.n - 1];
                if (ks * (int64_t)sizeof(T) * p.rpb < 4096) {
                    a.xcd_chunk = (int)((grid.x + 7) / 8);
                    grid.x = (unsigned)a.xcd_chunk * 8;
                }
            }
            if (vec && p.unaligned) row_reduce_kernel<Op, FULL, true><<<grid, block, 0, st>>>(a);
            else if (vec) row_reduce_kernel<Op, FULL><<<grid, block, 0, st>>>(a);
            else row_reduce_kernel<Op, 1><<<grid, block, 0, st>>>(a);
        }
        if (p.split > 1 && p.split <= 16)
            finish_rows_thin_kernel<Op><<<dim3((unsigned)((p.K + 255) / 256)), dim3(256), 0, st>>>(sc.partial, out, p.K, p.split,
                                                                                                   init_out, count);
        else if (p.split > 1)
            finish_rows_kernel<Op><<<dim3((unsigned)p.K), dim3(256), 0, st>>>(sc.partial, out, p.split, init_out,
                                                                              count);
        return;
    }
    // Col
    if (p.flat_xb > 0) {
        if constexpr (FULL > 1) {
            const int nk = p.kept.n;
            const int64_t kin = p.kept.size[nk - 1];
            const int64_t outer = nk > 1 ? p.kept.size[0] : 1;
            ColFlatWideArgs a{};
            a.in = in;
            a.partial = sc.partial;
            a.so = nk > 1 ? p.kept.stride[0] : 0;
            a.total = kin * p.R;
            a.K = p.K;
            a.kin = (int)kin;
            a.vecs = (int)(kin * p.flat_phases / FULL);
            a.phases = p.flat_phases;
            a.slices = p.split / p.flat_phases;
            col_flat_wide_kernel<Op, FULL><<<dim3((unsigned)p.flat_xb, (unsigned)outer, (unsigned)a.slices),
                                             dim3((unsigned)p.flat_t), 0, st>>>(a);
        }
    } else if (p.flat_t > 0) {
        if constexpr (FULL > 1) {
            const int nk = p.kept.n;
            const int64_t kin = p.kept.size[nk - 1];
            const int64_t outer = nk > 1 ? p.kept.size[0] : 1;
            ColFlatArgs a{};
            a.in = in;
            a.out = stage1_out;
            a.so = nk > 1 ? p.kept.stride[0] : 0;
            a.total = kin * p.R;
            a.K = p.K;
            a.count = count;
            a.kin = (int)kin;
            a.threads = p.flat_t;
            a.split = p.split;
            a.init_out = init_out;
if (p.unaligned)             col_flat_kernel<Op, FULL, true><<<dim3(1, (unsigned)outer, (unsigned)p.split), dim3((unsigned)p.bx),
                                        (size_t)p.flat_t * FULL * sizeof(Acc), st>>>(a);
            else             col_flat_kernel<Op, FULL><<<dim3(1, (unsigned)outer, (unsigned)p.split), dim3((unsigned)p.bx),
                                        (size_t)p.flat_t * FULL * sizeof(Acc), st>>>(a);
        }
    } else {
        const int64_t kv = p.K / p.vec;
        dim3 block((unsigned)p.bx, (unsigned)p.by);
        size_t smem = p.by > 1 ? (size_t)p.bx * p.by * (p.vec / p.sstride) * sizeof(Acc) : 0;
        if (p.lean) {
            ColLeanArgs a{};
            const int nk = p.kept.n;
            const int64_t kin = nk ? p.kept.size[nk - 1] : 1;
            a.in = in;
            a.out = stage1_out;
            a.so = nk > 1 ? p.kept.stride[0] : 0;
            a.rs = p.red.n ? p.red.stride[0] : 0;
            a.K = p.K;
            a.count = count;
            a.kin_v = (int)((kin + (p.unaligned ? p.vec - 1 : 0)) / (p.vec / p.sstride));
            a.kin = (int)kin;
            a.sk = nk ? (int)p.kept.stride[nk - 1] : 1;
            a.R = (int)p.R;
            a.split = p.split;
            a.init_out = init_out;
            const int64_t outer = nk > 1 ? p.kept.size[0] : 1;
            a.oso = p.kept_swapped ? 1 : kin;
            a.osi = p.kept_swapped ? outer : 1;
            {
                using Out = typename Op::Out;
                const int uv = p.vec / p.sstride;
                const size_t chunk = std::min<size_t>(16, (size_t)uv * sizeof(Out));
                // every lane's first output index, outer * kin + cv * uv, must be a multiple of uv: kin is
                a.vec_out = init_out && !p.kept_swapped && uv > 1 && kin % uv == 0 && ((uintptr_t)out % chunk) == 0;
            }
            dim3 grid((unsigned)((a.kin_v + p.bx - 1) / p.bx), (unsigned)outer, (unsigned)p.split);
            if (vec && p.sstride == 2) col_lean_kernel<Op, FULL, 2><<<grid, block, smem, st>>>(a);
            else if (vec && p.unaligned) {
                if constexpr (FULL > 1) col_lean_kernel<Op, FULL, 1, true><<<grid, block, smem, st>>>(a);
            } else if (vec) col_lean_kernel<Op, FULL><<<grid, block, smem, st>>>(a);
            else col_lean_kernel<Op, 1><<<grid, block, smem, st>>>(a);
        } else {
            ColArgs a{};
            a.in = in;
            a.out = stage1_out;
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
            dim3 grid((unsigned)((kv + p.bx - 1) / p.bx), (unsigned)p.split);
            if (vec) col_reduce_kernel<Op, FULL><<<grid, block, smem, st>>>(a);
            else col_reduce_kernel<Op, 1><<<grid, block, smem, st>>>(a);
        }
    }
    if (p.split > 1) {
        int fy = 1;  // thread rows sharing an output's partials: about two partials per thread
        while (fy < 16 && fy * 2 < p.split) fy <<= 1;
        // (swapped kept dims: the partials are in the kernel's numbering, the outputs in the caller's)
        const int64_t kin = p.kept_swapped ? p.kept.size[1] : p.K;
        const int64_t oso = p.kept_swapped ? 1 : 0, osi = p.kept_swapped ? p.kept.size[0] : 1;
        finish_cols_kernel<Op><<<dim3((unsigned)((p.K + 63) / 64)), dim3(64, (unsigned)fy),
                                 fy > 1 ? (size_t)fy * 64 * sizeof(Acc) : 0, st>>>(sc.partial, out, p.K, p.split,
                                                                                    init_out, count, kin, oso, osi);
    }
}

// Instantiate launch_reduce_t for every dtype of one op family.
#define HPT_FOR_ALL_DTYPES(X) \
    X(HPT_BOOL) X(HPT_I8) X(HPT_I16) X(HPT_I32) X(HPT_I64) X(HPT_U8) X(HPT_U16) X(HPT_U32) \
    X(HPT_U64) X(HPT_F16) X(HPT_BF16) X(HPT_F32) X(HPT_F64)

}  // namespace hpt
