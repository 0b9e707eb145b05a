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

#include "device_utils.hpp"
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

// exp / log in the compute type. Half tensors, whose results are rounded to 8 or 11 significant
// bits anyway, use the hardware exp2 / log2 on the scaled argument; f32 tensors (tolerance 1e-5
// against the CPU path) the exactly reduced form (exp_reduced, device_utils.hpp).
template <class T> __device__ __forceinline__ float exp_ct(float x) {
    if constexpr (sizeof(T) == 2) return __expf(x);
    else return exp_reduced<true>(x);  // every exponential of a softmax is of x - max <= 0
}
template <class T> __device__ __forceinline__ double exp_ct(double x) { return exp(x); }
template <class T> __device__ __forceinline__ float log_ct(float x) {
    if constexpr (sizeof(T) == 2) return __logf(x);
    else return logf(x);
}
template <class T> __device__ __forceinline__ double log_ct(double x) { return log(x); }
__device__ __forceinline__ float fma_ct(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double fma_ct(double a, double b, double c) { return fma(a, b, c); }
__device__ __forceinline__ float rsqrt_ct(float x) { return 1.0f / sqrtf(x); }
__device__ __forceinline__ double rsqrt_ct(double x) { return 1.0 / sqrt(x); }

template <class CT> __device__ __forceinline__ CT neg_inf() {
    if constexpr (sizeof(CT) == 8) return -__builtin_huge_val();
    else return -__builtin_huge_valf();
}

// Type the layernorm row statistics are combined in ACROSS lanes. Each lane sums
// its own (few) elements in the compute type; f32 rows then combine the lane
// sums in f64 and carry the mean as an f32 (hi, lo) pair, so that x - mean is
// accurate to an ulp of the difference even when the row's offset dwarfs its
// spread. No per-element f64 arithmetic is involved.
template <class T> struct StatType { using type = float; };
template <> struct StatType<float> { using type = double; };
template <> struct StatType<double> { using type = double; };

// (The kernels that sum exponentials one lane at a time carry that sum in StatType too: a long chain
// of f32 additions next to a total near 1, as when one element dominates its row, loses ~6e-8 per step,
// which shows in log_softmax results close to zero.)

// All-reduce over the `tpr` lanes that share a row: shuffles inside a wavefront,
// LDS across the wavefronts of the row. Every thread of the workgroup must call it.
template <class Op, class A>
__device__ __forceinline__ A row_all_reduce(A v, int tpr, int ty, A* smem) {
    v = group_reduce<Op>(v, tpr < 64 ? tpr : 64);
    if (tpr > 64) {
        const int wpr = tpr >> 6;
        __syncthreads();
        if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
        __syncthreads();
        A r = smem[ty * wpr];
        for (int w = 1; w < wpr; ++w) r = Op::comb(r, smem[ty * wpr + w]);
        v = r;
    }
    return v;
}

// The same for N values at once (one exchange through LDS for all of them; smem holds 16 * G * N values).
// G > 1: neighbouring lanes hold DIFFERENT statistics - lane l those of number l % G - and only lanes with the same
// l % G are folded: the butterflies start at distance G.
template <class Op, class A, int N, int G = 1>
__device__ __forceinline__ void row_all_reduce_n(A (&v)[N], int tpr, int ty, A* smem) {
    static_assert(G == 1 || G == 2 || G == 4, "up to four lanes side by side (the wavefronts' partials are folded by one wavefront's lanes)");
    const int width = tpr < 64 ? tpr : 64;
#pragma unroll
    for (int k = 0; k < N; ++k) {
        if constexpr (G == 1) {
            v[k] = group_reduce<Op>(v[k], width);
        } else {
#pragma unroll
            for (int d = G; d < 64; d <<= 1)
                if (d < width) v[k] = Op::comb(v[k], shfl_xor_any(v[k], d));
        }
    }
    if (tpr > 64) {
        const int wpr = tpr >> 6;
        const int lane = threadIdx.x & 63;
        __syncthreads();
        if (lane < G) {
#pragma unroll
            for (int k = 0; k < N; ++k) smem[((threadIdx.x >> 6) * G + lane) * N + k] = v[k];
        }
        __syncthreads();
        // (lanes take one wavefront's values each and a butterfly over them folds the wavefronts: N reads and
        // N * log2(wpr) shuffles per thread instead of N * wpr reads)
        const int w = (lane / G) & (wpr - 1), g = lane % G;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            A r = smem[((ty * wpr + w) * G + g) * N + k];
            if constexpr (G == 1) {
                r = group_reduce<Op>(r, wpr);
            } else {
#pragma unroll
                for (int d = G; d < 64; d <<= 1)
                    if (d < G * wpr) r = Op::comb(r, shfl_xor_any(r, d));
            }
            v[k] = r;
        }
    }
}

// ---- rows held in registers ---------------------------------------------------
// grid.x workgroups walk the rows in steps of gridDim.x * rpb, so that gamma and
// beta are fetched once per thread (they index by column, and a thread keeps its
// columns) instead of once per row, and the launch prologue is paid once.
// SS = 2 reads a row whose elements sit at every second position (a [:, ::2] view):
// full 128-bit vectors are loaded and the odd positions dropped, which moves the
// same cache lines as a scalar gather with a fraction of the instructions. (A
// 16-byte aligned vector that holds one valid element never leaves that element's
// page, so the unused half of the last vector is safe to touch.)
// SHIFT (VEC > 1, SS = 1): rows whose START is only element-aligned (odd row lengths: 197, 4097,
// 50257). A row is covered by the 16-byte ALIGNED vectors that contain it: vector iv holds the
// row's elements iv * VEC - m ... + VEC - 1, m = the row's misalignment in elements; positions
// outside the row are masked, whole vectors are stored whole and the two end vectors element by
// element. Input, output and residual rows share m (the caller checks bases and pitches mod 16
// bytes). Layernorm keeps gamma / beta per thread, so a thread's rows must share m as well: the
// launch makes the row step of the walk a multiple of VEC.
// PF: always issue the next row's loads before the current row's statistics (see kPrefetch below);
// the launch then caps the grid so that workgroups do walk rows.
// GB = 2 (layernorm rows of more vectors per thread than leave room for gamma / beta beside them): gamma / beta are
// read again for every row, vector by vector in the last sweep, from L2 (they are 2 x cols elements, which every
// workgroup keeps reading). A workgroup then needs nothing from one row to the next.
// GB = 1, "GBL" (layernorm of 2-byte types, long rows): gamma / beta live in LDS instead of registers (loaded
// once per workgroup, read per row), which leaves room for four vectors of the row per thread where
// the register form holds two: half as many threads per row, twice as many rows in flight.
// IL > 1 (softmax kinds): a "row" is a contiguous [cols / IL, IL] slab and the softmax runs over its first dim - IL
// interleaved softmaxes, element e of the row belonging to number e % IL. IL divides VEC: that is the element's place
// in its vector, and a thread keeps IL (max, sum) pairs. IL = 2 vectors: a thread's vectors all hold the same VEC
// numbers (threads per row are even), its neighbour the other VEC, and only threads two apart are folded together. Loads and stores are those of a plain row (softmax over the middle axis of a contiguous
// [B, C, 2], [B, C, 4], [B, C, 8 heads]).
template <int KIND, class T, int VEC, int NCHUNK, int SS = 1, bool SHIFT = false, bool PF = false, int GB = 0, int IL = 1>
__global__ void __launch_bounds__(1024) row_reg_kernel(const NormArgs a) {
    constexpr int ML = IL < 0 ? -IL : 0;  // interleaved softmaxes whose number is no divisor of the vector (3, 5, 6, 7)
    static_assert(IL == 1 || (!norm_is_layer(KIND) && !norm_is_causal(KIND) && SS == 1 && !SHIFT && VEC > 1 &&
                              (ML ? (ML >= 3 && ML <= 7 && VEC % ML != 0) : (VEC % IL == 0 || IL % VEC == 0))),
                  "interleaved rows: a plain softmax of whole vectors");
    constexpr int NS = ML ? VEC : (IL < VEC ? IL : VEC);  // statistics a thread keeps
    constexpr int IG = IL > VEC ? IL / VEC : 1;            // neighbouring threads that hold different ones
    constexpr bool GBL = GB == 1;  // gamma / beta in LDS
    constexpr bool GBG = GB == 2;  // gamma / beta from global memory, every row
    static_assert(GB == 0 || (norm_is_layer(KIND) && VEC > 1 && SS == 1 && !SHIFT), "gamma / beta outside registers: an aligned layernorm form");
    static_assert(!SHIFT || (VEC > 1 && SS == 1), "SHIFT is a full-vector mode");
    constexpr int UV = VEC / SS;  // useful elements per vector
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    __shared__ __align__(8) unsigned char smem_stat[16 * (ML ? ML : IL) * sizeof(double)];
    CT* smem = reinterpret_cast<CT*>(smem_stat);
    ST* ssmem = reinterpret_cast<ST*>(smem_stat);
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int nv = SHIFT ? (int)((a.cols + 2 * (VEC - 1)) / VEC) : (int)(a.cols / UV);  // SHIFT: upper bound
    // Vector c of this thread. ML: only the largest multiple of ML lanes of a row take part, so that all of a lane's
    // vectors start at the same place modulo ML, (tx * VEC) % ML; the other lanes hold nothing.
    const int tstep = ML ? tpr / (ML ? ML : 1) * ML : tpr;
    auto vec_of = [&](int c) -> int {
        if constexpr (ML > 0) return tx < tstep ? c * tstep + tx : nv;
        else return c * tpr + tx;
    };
    const int cols = (int)a.cols;
    // misalignment, in elements, of a row that starts at p
    auto shift_of = [](const T* p) -> int { return SHIFT ? (int)(((uintptr_t)p / sizeof(T)) % VEC) : 0; };
    constexpr bool kSoft = !norm_is_layer(KIND);
    constexpr bool kLog = norm_is_log(KIND);
    constexpr bool kCausal = norm_is_causal(KIND);
    constexpr bool kRes = KIND == NORM_ADD_LAYERNORM;
    const CT fill = kSoft ? neg_inf<CT>() : (CT)0;

    // this thread's columns never change: keep gamma / beta in registers (or, GBL, in LDS)
    extern __shared__ __align__(16) unsigned char gb_raw[];
    T* lds_gamma = reinterpret_cast<T*>(gb_raw);
    T* lds_beta = lds_gamma + (GBL ? (size_t)nv * UV : 0);
    Pack<T, UV> gam[GB ? 1 : NCHUNK], bet[GB ? 1 : NCHUNK];
    if constexpr (!kSoft && !GB) {
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int iv = vec_of(c);
#pragma unroll
            for (int j = 0; j < UV; ++j) {
                gam[c].v[j] = Elem<T>::narrow((CT)1);
                bet[c].v[j] = Elem<T>::narrow((CT)0);
            }
            if constexpr (SHIFT) {
                // every row this thread will see has the misalignment of its first one
                const int64_t row = (int64_t)blockIdx.x * a.rpb + ty;
                const int m = shift_of((const T*)a.out + (row < a.rows ? row : 0) * a.cols);
                const int e0 = iv * VEC - m;
                if (e0 >= 0 && e0 + VEC <= cols) {
                    if (a.gamma) gam[c] = load_pack_unaligned<T, UV>((const T*)a.gamma + e0);
                    if (a.beta) bet[c] = load_pack_unaligned<T, UV>((const T*)a.beta + e0);
                } else {
#pragma unroll
                    for (int j = 0; j < UV; ++j)
                        if ((unsigned)(e0 + j) < (unsigned)cols) {
                            if (a.gamma) gam[c].v[j] = ((const T*)a.gamma)[e0 + j];
                            if (a.beta) bet[c].v[j] = ((const T*)a.beta)[e0 + j];
                        }
                }
            } else if (iv < nv) {
                if constexpr (VEC > 1) {
                    if (a.gamma) gam[c] = load_pack<T, UV>((const T*)a.gamma + (int64_t)iv * UV);
                    if (a.beta) bet[c] = load_pack<T, UV>((const T*)a.beta + (int64_t)iv * UV);
                } else {
                    if (a.gamma) gam[c].v[0] = ((const T*)a.gamma)[iv];
                    if (a.beta) bet[c].v[0] = ((const T*)a.beta)[iv];
                }
            }
        }
    }

    // Where registers allow (2-byte elements, few values per thread), the loads of the
    // NEXT row this workgroup will take are issued before the current row's statistics
    // and stores, so that the memory pipeline never drains between rows. With 4-byte
    // elements the extra live registers cost more than the overlap gains (measured).
    // Rows that take 512 or 1024 threads leave room for one or two workgroups per compute unit, so
    // nothing else hides a row's load -> reduce -> reduce -> store chain: there (PF) the prefetch
    // pays for every type (f32 [3355, 10000] softmax: 3.2 TB/s without).
    constexpr bool kPrefetch = ((sizeof(T) == 2 && NCHUNK * UV <= ((kSoft || GB) ? 32 : 16)) || PF) && !kRes;
    const int64_t row_step = (int64_t)gridDim.x * a.rpb;
    Pack<T, VEC> raw[NCHUNK];
    Pack<T, UV> raw_res[kRes ? NCHUNK : 1];
    // causal kinds: row q of each (q_rows x cols) matrix keeps columns 0 .. q + causal_offset;
    // the rest is never read and counts as -inf
    // the scalar operand of the unfused mul_ has the tensor's dtype
    const CT scale_t = kCausal ? Elem<T>::widen(Elem<T>::narrow((CT)a.scale)) : (CT)1;
    auto row_limit = [&](int64_t row) -> int64_t {
        if constexpr (kCausal) {
            // (rows and q_rows fit 32 bits whenever this kernel runs: a row fits registers)
            const int64_t q = ((uint64_t)(row | a.q_rows) >> 32) == 0 ? (int64_t)((uint32_t)row % (uint32_t)a.q_rows)
                                                                      : row % a.q_rows;
            const int64_t lim = q + a.causal_offset + 1;
            return lim < 0 ? 0 : (lim < a.cols ? lim : a.cols);
        } else {
            return a.cols;
        }
    };
    auto issue_loads = [&](int64_t row0) {
        const int64_t row = row0 + ty;
        if (row >= a.rows) return;
        const T* in_row = (const T*)a.in + offset_of(a.kept_in, row);
        const int m = shift_of(in_row);
        in_row -= m;
        const int nv_row = (kCausal || SHIFT) ? (int)((row_limit(row) + m + UV - 1) / UV) : nv;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int iv = vec_of(c);
            if (iv < nv_row) {
                if constexpr (VEC > 1) raw[c] = load_pack_stream<T, VEC>(in_row + (int64_t)iv * VEC);
                else raw[c].v[0] = in_row[(int64_t)iv * a.sa];
                if constexpr (kRes) {
                    const T* res_row = (const T*)a.residual + row * a.cols - m;
                    if constexpr (VEC > 1) raw_res[c] = load_pack_stream<T, UV>(res_row + (int64_t)iv * UV);
                    else raw_res[c].v[0] = res_row[iv];
                }
            }
        }
    };
    if constexpr (kPrefetch) issue_loads((int64_t)blockIdx.x * a.rpb);
    // (gamma / beta are staged while the first row's loads are in flight)
    if constexpr (GBL) {
        for (int i = threadIdx.x; i < nv; i += blockDim.x) {
            Pack<T, UV> g, b;
#pragma unroll
            for (int j = 0; j < UV; ++j) {
                g.v[j] = Elem<T>::narrow((CT)1);
                b.v[j] = Elem<T>::narrow((CT)0);
            }
            if (a.gamma) g = load_pack<T, UV>((const T*)a.gamma + (int64_t)i * UV);
            if (a.beta) b = load_pack<T, UV>((const T*)a.beta + (int64_t)i * UV);
            store_pack<T, UV>(lds_gamma + (size_t)i * UV, g);
            store_pack<T, UV>(lds_beta + (size_t)i * UV, b);
        }
        __syncthreads();
    }
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < a.rows; row0 += row_step) {
        if constexpr (!kPrefetch) issue_loads(row0);
        const int64_t row = row0 + ty;
        const bool valid = row < a.rows;
        T* out_row = (T*)a.out + (valid ? row * a.cols : 0);
        const int limit = valid ? (int)row_limit(row) : 0;  // cols <= 8192 vectors here
        const int sh = shift_of(out_row);
        // is element j of vector iv inside the row (and, for the causal kinds, kept)?
        auto inside = [&](int iv, int j) -> bool {
            if constexpr (SHIFT) return (unsigned)(iv * UV + j - sh) < (unsigned)limit;
            else return iv < nv && (!kCausal || iv * UV + j < limit);
        };

        CT x[NCHUNK][UV];
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int iv = vec_of(c);
            if constexpr (kCausal && !SHIFT) {
                // A chunk (the tpr vectors the row's lanes hold side by side) lies wholly below the diagonal, wholly
                // above it, or across it. Only the one across it needs a test per element; the masked half of the
                // logits costs no arithmetic at all. (With the tests on every element the two-byte kernel was bound
                // by its instructions, not by memory: bf16 [32, 2048, 2048] with nothing masked took 104 us where the
                // plain softmax of the same bytes takes 85.)
                const int c_lo = c * tpr * UV;
                if (!valid || c_lo >= limit) {
#pragma unroll
                    for (int j = 0; j < UV; ++j) x[c][j] = fill;
                    continue;
                }
                if (c_lo + tpr * UV <= limit) {
#pragma unroll
                    for (int j = 0; j < UV; ++j)
                        x[c][j] = Elem<T>::widen(Elem<T>::narrow(Elem<T>::widen(raw[c].v[j * SS]) * scale_t));
                    continue;
                }
            }
#pragma unroll
            for (int j = 0; j < UV; ++j) {
                const bool have = valid && inside(iv, j);
                CT e = have ? Elem<T>::widen(raw[c].v[j * SS]) : fill;
                // the fused forms round the intermediate (in + residual, scale * in) to the tensor's
                // dtype, as the separate add / mul_ of the unfused sequence would have stored it
                if constexpr (kRes) e = have ? Elem<T>::widen(Elem<T>::narrow(e + Elem<T>::widen(raw_res[c].v[j]))) : fill;
                if constexpr (kCausal) e = have ? Elem<T>::widen(Elem<T>::narrow(e * scale_t)) : fill;
                x[c][j] = e;
            }
        }
        if constexpr (kPrefetch) issue_loads(row0 + row_step);

        if constexpr (kSoft) {
            CT mv[NS];
#pragma unroll
            for (int k = 0; k < NS; ++k) mv[k] = neg_inf<CT>();
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
                for (int j = 0; j < UV; ++j) mv[j % NS] = MaxC<CT>::comb(mv[j % NS], x[c][j]);
            // ML: place j of this lane's vectors belongs to softmax (tx * VEC + j) % ML
            const int rot = ML ? tx * VEC % (ML ? ML : 1) : 0;
            if constexpr (IL == 1) {
                mv[0] = row_all_reduce<MaxC<CT>>(mv[0], tpr, ty, smem);
            } else if constexpr (ML > 0) {
                CT cm[ML];
#pragma unroll
                for (int k = 0; k < ML; ++k) cm[k] = neg_inf<CT>();
#pragma unroll
                for (int j = 0; j < VEC; ++j)
#pragma unroll
                    for (int k = 0; k < ML; ++k)
                        if (k == (rot + j) % ML) cm[k] = MaxC<CT>::comb(cm[k], mv[j]);
                row_all_reduce_n<MaxC<CT>, CT, ML, 1>(cm, tpr, ty, smem);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
#pragma unroll
                    for (int k = 0; k < ML; ++k)
                        if (k == (rot + j) % ML) mv[j] = cm[k];
            } else {
                row_all_reduce_n<MaxC<CT>, CT, NS, IG>(mv, tpr, ty, smem);
            }
            CT sv[NS];
#pragma unroll
            for (int k = 0; k < NS; ++k) sv[k] = 0;
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c) {
                // causal kinds: a chunk that lies wholly above the diagonal (the same for every lane
                // of the row) is all -inf: its exponentials are 0 without computing them. A row with
                // no key at all takes the ordinary way and comes out NaN, as -inf - -inf does.
                if (kCausal && limit > 0 && c * tpr * UV - sh >= limit) {
#pragma unroll
                    for (int j = 0; j < UV; ++j) x[c][j] = kLog ? neg_inf<CT>() : (CT)0;
                    continue;
                }
#pragma unroll
                for (int j = 0; j < UV; ++j) {
                    CT d = x[c][j] - mv[j % NS];
                    CT e = exp_ct<T>(d);
                    sv[j % NS] += e;
                    x[c][j] = kLog ? d : e;
                }
            }
            if constexpr (IL == 1) {
                sv[0] = row_all_reduce<SumC<CT>>(sv[0], tpr, ty, smem);
            } else if constexpr (ML > 0) {
                CT cs[ML];
#pragma unroll
                for (int k = 0; k < ML; ++k) cs[k] = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j)
#pragma unroll
                    for (int k = 0; k < ML; ++k)
                        if (k == (rot + j) % ML) cs[k] += sv[j];
                row_all_reduce_n<SumC<CT>, CT, ML, 1>(cs, tpr, ty, smem);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
#pragma unroll
                    for (int k = 0; k < ML; ++k)
                        if (k == (rot + j) % ML) sv[j] = cs[k];
            } else {
                row_all_reduce_n<SumC<CT>, CT, NS, IG>(sv, tpr, ty, smem);
            }
            CT kv[NS];
#pragma unroll
            for (int k = 0; k < NS; ++k) kv[k] = kLog ? log_ct<T>(sv[k]) : (CT)1 / sv[k];
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
                for (int j = 0; j < UV; ++j)
                    x[c][j] = kLog ? x[c][j] - kv[j % NS] : x[c][j] * kv[j % NS];
        } else {
            // (the lane's own sum is taken in the wide type too: a lane may hold the whole of a short row,
            // and a row whose spread is small against its offset loses digits of the mean that matter)
            ST s = 0;
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
                for (int j = 0; j < UV; ++j) s += (ST)x[c][j];
            // mean = sum / cols, as a reciprocal multiply plus one correction step
            // (exact quotient for the cases that matter, e.g. constant rows)
            const ST sum = row_all_reduce<SumC<ST>>(s, tpr, ty, ssmem);
            const ST m0 = sum * (ST)a.inv_cols;
            const ST mean = fma_ct(fma_ct(-m0, (ST)a.cols, sum), (ST)a.inv_cols, m0);
            const CT mean_hi = (CT)mean;
            const CT mean_lo = (CT)(mean - (ST)mean_hi);  // 0 when ST is no wider than CT
            CT q = 0;
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c) {
                const bool in_row_c = (c * tpr + tx) < nv;
#pragma unroll
                for (int j = 0; j < UV; ++j) {
                    const bool in_row_e = SHIFT ? inside(c * tpr + tx, j) : in_row_c;
                    const CT d = in_row_e ? (x[c][j] - mean_hi) - mean_lo : (CT)0;
                    x[c][j] = d;
                    q += d * d;
                }
            }
            const ST var = row_all_reduce<SumC<ST>>((ST)q, tpr, ty, ssmem) * (ST)a.inv_cols;
            const CT rstd = rsqrt_ct((CT)var + (CT)a.eps);
            if constexpr (GBG) {
                // (the pointers are made opaque per row, or the loads would be hoisted out of the row loop and
                // gamma / beta would sit in registers after all)
                const T* gp = (const T*)a.gamma;
                const T* bp = (const T*)a.beta;
                asm volatile("" : "+s"(gp), "+s"(bp));
#pragma unroll
                for (int c = 0; c < NCHUNK; ++c) {
                    const int iv = vec_of(c);
                    if (iv < nv) {
                        Pack<T, UV> g, b;
#pragma unroll
                        for (int j = 0; j < UV; ++j) {
                            g.v[j] = Elem<T>::narrow((CT)1);
                            b.v[j] = Elem<T>::narrow((CT)0);
                        }
                        if (gp) g = load_pack<T, UV>(gp + (size_t)iv * UV);
                        if (bp) b = load_pack<T, UV>(bp + (size_t)iv * UV);
#pragma unroll
                        for (int j = 0; j < UV; ++j)
                            x[c][j] = x[c][j] * rstd * Elem<T>::widen(g.v[j]) + Elem<T>::widen(b.v[j]);
                    }
                }
            } else if constexpr (GBL) {
#pragma unroll
                for (int c = 0; c < NCHUNK; ++c) {
                    const int iv = vec_of(c);
                    if (iv < nv) {
                        const Pack<T, UV> g = load_pack<T, UV>(lds_gamma + (size_t)iv * UV);
                        const Pack<T, UV> b = load_pack<T, UV>(lds_beta + (size_t)iv * UV);
#pragma unroll
                        for (int j = 0; j < UV; ++j)
                            x[c][j] = x[c][j] * rstd * Elem<T>::widen(g.v[j]) + Elem<T>::widen(b.v[j]);
                    }
                }
            } else {
#pragma unroll
                for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
                    for (int j = 0; j < UV; ++j)
                        x[c][j] = x[c][j] * rstd * Elem<T>::widen(gam[c].v[j]) + Elem<T>::widen(bet[c].v[j]);
            }
        }

        if (valid) {
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c) {
                const int iv = vec_of(c);
                if constexpr (SHIFT) {
                    const int e0 = iv * VEC - sh;
                    if (e0 + VEC > 0 && e0 < cols) {
                        Pack<T, UV> o;
#pragma unroll
                        for (int j = 0; j < UV; ++j) o.v[j] = Elem<T>::narrow(x[c][j]);
                        if (e0 >= 0 && e0 + VEC <= cols) {
                            store_pack_stream<T, UV>(out_row + e0, o);
                        } else {
#pragma unroll
                            for (int j = 0; j < UV; ++j)
                                if ((unsigned)(e0 + j) < (unsigned)cols) out_row[e0 + j] = o.v[j];
                        }
                    }
                } else if (iv < nv) {
                    if constexpr (VEC > 1) {
                        Pack<T, UV> o;
#pragma unroll
                        for (int j = 0; j < UV; ++j) o.v[j] = Elem<T>::narrow(x[c][j]);
                        store_pack_stream<T, UV>(out_row + (int64_t)iv * UV, o);
                    } else {
                        out_row[iv] = Elem<T>::narrow(x[c][0]);
                    }
                }
            }
        }
    }
}

// ---- long rows of 2-byte elements: the raw row in registers ---------------------------------
// softmax / log_softmax over aligned rows of 98305 ... 131072 f16 / bf16 elements (a vocabulary of
// 128256). The row kernel above keeps the widened row (f32) between its sweeps, which is 64 registers
// per thread at eight vectors and does not fit at sixteen. Here only the RAW row stays (4 registers
// per vector: 64 at sixteen vectors per thread, 1024 threads per row) and every sweep widens again:
// max, then the sum of exponentials, then the result, the exponential taken twice. One HBM read and
// one write where the streaming kernel reads twice.
template <int KIND, class T, int NCHUNK>
__global__ void __launch_bounds__(1024) row_raw_kernel(const NormArgs a) {
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "a softmax kernel");
    constexpr int VEC = 16 / sizeof(T);
    constexpr bool kLog = KIND == NORM_LOGSOFTMAX;
    using CT = typename Elem<T>::Wide;
    __shared__ CT smem[16];
    const int tx = threadIdx.x;
    const int nv = (int)a.cols / VEC;
    Pack<T, VEC> raw[NCHUNK];
    // (2-byte types: keep the compiler from holding the widened copies of one sweep for the next)
    auto forget = [](Pack<T, VEC>& v) {
        if constexpr (sizeof(T) == 2) asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&v)));
    };
    for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const T* in_row = (const T*)a.in + offset_of(a.kept_in, row);
        T* out_row = (T*)a.out + row * a.cols;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int iv = c * 1024 + tx;
            if (iv < nv) raw[c] = load_pack_stream<T, VEC>(in_row + (int64_t)iv * VEC);
        }
        CT m = neg_inf<CT>();
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
            if (c * 1024 + tx < nv)
#pragma unroll
                for (int j = 0; j < VEC; ++j) m = MaxC<CT>::comb(m, Elem<T>::widen(raw[c].v[j]));
        m = row_all_reduce<MaxC<CT>>(m, 1024, 0, smem);
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) forget(raw[c]);
        CT s = 0;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
            if (c * 1024 + tx < nv)
#pragma unroll
                for (int j = 0; j < VEC; ++j) s += exp_ct<T>(Elem<T>::widen(raw[c].v[j]) - m);
        s = row_all_reduce<SumC<CT>>(s, 1024, 0, smem);
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) forget(raw[c]);
        const CT k = kLog ? log_ct<T>(s) : (CT)1 / s;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int iv = c * 1024 + tx;
            if (iv < nv) {
                Pack<T, VEC> o;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const CT d = Elem<T>::widen(raw[c].v[j]) - m;
                    o.v[j] = Elem<T>::narrow(kLog ? d - k : exp_ct<T>(d) * k);
                }
                store_pack_stream<T, VEC>(out_row + (int64_t)iv * VEC, o);
            }
        }
    }
}

// ---- long rows that stay on chip: the row in registers AND LDS -----------------------------------
// softmax / log_softmax over rows too long for the register kernel's eight vectors per thread: f32 rows
// of 32769 ... 131072 elements and two-byte rows of 32769 ... 196608 (logits over a vocabulary: 50257,
// 50304, 65536, 100277, 128256, 151936), and rows of odd length (row starts off the 16-byte grid) from
// 2049 vectors on, which the register kernel does not take.
// NREG vectors per thread live in registers, up to NLDS more in LDS (every thread reads back only the
// slots it filled, so the LDS part needs no barrier: it is a second register file). One HBM read and
// one write where the streaming kernel reads twice. The LDS part arrives by LDS-direct loads
// (global_load_lds_dwordx4: a wavefront's 64 lanes fill 1 KiB of LDS from the wavefront's base on), so
// no register is held for it while it is on its way and NREG can take what the register file has.
// Shapes: NT = 256 or 512 threads with 24 + 8 vectors of a four-byte type (16 + 8 of a two-byte type)
// and 128 registers each, so that two (512) or four (256) workgroups share a compute unit and one's
// arithmetic overlaps the other's loads and stores; NT = 512 with 48 + 16 (32 + 16) vectors and 256
// registers each for the longest rows, one workgroup per compute unit. (Shifted four-byte rows: 20 + 8
// and 44 + 16, which leaves the row-end masks their registers.)
// Four-byte types: the summing sweep overwrites the held row with exp(x - max) (softmax) or x - max
// (log_softmax), so the exponential is taken once per element either way. Two-byte types keep the
// raw row (rounding the intermediate to 16 bits would cost accuracy) and take the exponential twice.
// SHIFT: rows that start off 16-byte boundaries (a vocabulary of 50257): a row is covered by aligned
// vectors that contain it; positions outside the row count as -inf and the two end vectors are stored
// element by element. Input and output rows share their misalignment.
template <int KIND, class T, int NREG, int NLDS, bool SHIFT, int NT, int MINW>
__global__ void __launch_bounds__(NT, MINW) row_lds_kernel(const NormArgs a) {
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "a softmax kernel");
    static_assert(NLDS * NT * 16 <= 144 * 1024, "LDS of a compute unit");
    constexpr int VEC = 16 / sizeof(T);
    constexpr bool kKeep = sizeof(T) >= 4;  // the held row may be overwritten with intermediates
    constexpr bool kLog = KIND == NORM_LOGSOFTMAX;
    // the walks over the LDS part stay loops (LDS takes a run-time index; unrolled, their reads are
    // hoisted over the register part's work and push it out of the register file)
    constexpr int kLdsUnroll = 2;
    using CT = typename Elem<T>::Wide;
    __shared__ CT smem[16];
    __shared__ __align__(16) unsigned char lds_raw[NLDS * NT * 16];
    Pack<T, VEC>* lds = reinterpret_cast<Pack<T, VEC>*>(lds_raw);
    const int tx = threadIdx.x;
    const int cols = (int)a.cols;
    // SHIFT: the vector grid starts on the 128-byte line that holds the row's first element, so a
    // wavefront's 1 KiB of loads or stores covers eight whole lines, not nine partial ones
    constexpr int LINE = 128 / sizeof(T);
    auto shift_of = [](const T* p) -> int { return SHIFT ? (int)(((uintptr_t)p / sizeof(T)) % LINE) : 0; };
    // (2-byte types: keep the compiler from holding the widened copies of one sweep for the next)
    auto forget = [](Pack<T, VEC>& v) {
        if constexpr (sizeof(T) == 2) asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&v)));
    };
    for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const T* in_row = (const T*)a.in + offset_of(a.kept_in, row);
        T* out_row = (T*)a.out + row * a.cols;
        const int sh = shift_of(out_row);
        const int nv = SHIFT ? (cols + sh + VEC - 1) / VEC : cols / VEC;
        auto mask_ends = [&](Pack<T, VEC>& v, int iv) {
            if constexpr (SHIFT) {
                if (iv * VEC < sh || iv == nv - 1) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if ((unsigned)(iv * VEC + j - sh) >= (unsigned)cols) v.v[j] = Elem<T>::narrow(neg_inf<CT>());
                }
            }
        };
        // (a vector that lies wholly before the row is not loaded: only a vector that holds an element of
        // the row is sure to stay on that element's page)
        auto touches = [&](int iv) { return !SHIFT || (iv + 1) * VEC > sh; };
        // an address is the chunk's start (the same for every lane: a scalar) plus the lane's 32-bit offset;
        // forty-odd 64-bit addresses per lane, computed ahead of the row loop, would not fit beside the row
        auto chunk_of = [](auto* p, int c) { return p + (int64_t)c * (NT * VEC); };
        const unsigned lane_off = (unsigned)tx * VEC;
        // The LDS part arrives by LDS-direct loads, which the LOAD counter tracks, not the LDS one. Whether the compiler
        // waits for them before an ordinary LDS read of the same slot depends on what it can prove about the two
        // addresses (a working build that issued the loads from inside a lambda lost that wait, and the sweeps read slots
        // that had not arrived). The wait is therefore written out, before the first LDS read of a row.
        auto wait_for_lds_part = [] { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
        Pack<T, VEC> reg[NREG];
        {
#pragma unroll kLdsUnroll
            for (int c = 0; c < NLDS; ++c) {
                const int iv = (NREG + c) * NT + tx;
                if (iv < nv && touches(iv))
                    __builtin_amdgcn_global_load_lds(
                        (const __attribute__((address_space(1))) void*)(chunk_of(in_row - sh, NREG + c) + lane_off),
                        (__attribute__((address_space(3))) void*)(lds + c * NT + (tx & ~63)), 16, 0, 0);
            }
#pragma unroll
            for (int c = 0; c < NREG; ++c) {
                const int iv = c * NT + tx;
                if (iv < nv && touches(iv)) reg[c] = load_pack_stream<T, VEC>(chunk_of(in_row - sh, c) + lane_off);
            }
            if constexpr (SHIFT) {
                wait_for_lds_part();
#pragma unroll kLdsUnroll
                for (int c = 0; c < NLDS; ++c) {
                    const int iv = (NREG + c) * NT + tx;
                    if (iv < nv && (iv * VEC < sh || iv == nv - 1)) {
                        Pack<T, VEC> v = lds[c * NT + tx];
                        mask_ends(v, iv);
                        lds[c * NT + tx] = v;
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < NREG; ++c) mask_ends(reg[c], c * NT + tx);
        CT m = neg_inf<CT>();
#pragma unroll
        for (int c = 0; c < NREG; ++c)
            if (c * NT + tx < nv)
#pragma unroll
                for (int j = 0; j < VEC; ++j) m = MaxC<CT>::comb(m, Elem<T>::widen(reg[c].v[j]));
        if constexpr (!SHIFT) wait_for_lds_part();
#pragma unroll kLdsUnroll
        for (int c = 0; c < NLDS; ++c)
            if ((NREG + c) * NT + tx < nv) {
                const Pack<T, VEC> v = lds[c * NT + tx];
#pragma unroll
                for (int j = 0; j < VEC; ++j) m = MaxC<CT>::comb(m, Elem<T>::widen(v.v[j]));
            }
        m = row_all_reduce<MaxC<CT>>(m, NT, 0, smem);
#pragma unroll
        for (int c = 0; c < NREG; ++c) forget(reg[c]);
        CT s = 0;
#pragma unroll
        for (int c = 0; c < NREG; ++c)
            if (c * NT + tx < nv)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const CT d = Elem<T>::widen(reg[c].v[j]) - m;
                    const CT e = exp_ct<T>(d);
                    s += e;
                    if constexpr (kKeep) reg[c].v[j] = Elem<T>::narrow(kLog ? d : e);
                }
#pragma unroll kLdsUnroll
        for (int c = 0; c < NLDS; ++c)
            if ((NREG + c) * NT + tx < nv) {
                Pack<T, VEC> v = lds[c * NT + tx];
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const CT d = Elem<T>::widen(v.v[j]) - m;
                    const CT e = exp_ct<T>(d);
                    s += e;
                    if constexpr (kKeep) v.v[j] = Elem<T>::narrow(kLog ? d : e);
                }
                if constexpr (kKeep) lds[c * NT + tx] = v;
            }
        s = row_all_reduce<SumC<CT>>(s, NT, 0, smem);
#pragma unroll
        for (int c = 0; c < NREG; ++c) forget(reg[c]);
        const CT k = kLog ? log_ct<T>(s) : (CT)1 / s;
        auto finish = [&](Pack<T, VEC> v, int iv) {
            Pack<T, VEC> o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const CT x = Elem<T>::widen(v.v[j]);
                if constexpr (kKeep) o.v[j] = Elem<T>::narrow(kLog ? x - k : x * k);
                else o.v[j] = Elem<T>::narrow(kLog ? (x - m) - k : exp_ct<T>(x - m) * k);
            }
            const int e0 = iv * VEC - sh;
            T* dst = chunk_of(out_row - sh, (iv - tx) / NT) + lane_off;
            if (!SHIFT || (e0 >= 0 && e0 + VEC <= cols)) {
                store_pack_stream<T, VEC>(dst, o);
            } else {  // the row's two end vectors leave element by element
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if ((unsigned)(e0 + j) < (unsigned)cols) out_row[e0 + j] = o.v[j];
            }
        };
#pragma unroll
        for (int c = 0; c < NREG; ++c)
            if (c * NT + tx < nv) finish(reg[c], c * NT + tx);
#pragma unroll kLdsUnroll
        for (int c = 0; c < NLDS; ++c)
            if ((NREG + c) * NT + tx < nv) finish(lds[c * NT + tx], (NREG + c) * NT + tx);
    }
}

// ---- short rows laid back to back: whole tiles through LDS ---------------------------------
// A contiguous [rows, cols] matrix with short rows (cols <= 512): a workgroup brings a.rpb
// consecutive rows (16 KiB; a multiple of VEC rows, so the tile starts on a 16-byte boundary
// whatever cols is) into LDS with aligned 128-bit loads, groups of `tpr` lanes normalise the rows
// in place (EPL elements per lane, at most eight, held in registers between the passes), and the tile
// leaves with aligned 128-bit stores. HBM sees whole lines only, in both directions.
// EPL is what a lane of THIS row length has (rows of 257 over 64 lanes: 5): sweeps unrolled to eight would run
// three steps with every lane masked off - f32 [130561, 257] softmax 59.4 -> 48.0 us, [260111, 129] 54.6 -> 49.0,
// f16 [130561, 257] 38.0 -> 34.5. (Stopping the unrolled sweeps at run time instead costs more than the idle steps:
// f16 [170327, 197] 28.5 -> 36.7 us.)
template <int KIND, class T, int VEC, int EPL = 8>
__global__ void __launch_bounds__(256) norm_tile_kernel(const NormArgs a) {
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX || KIND == NORM_LAYERNORM, "plain kinds only");
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    constexpr bool kSoft = !norm_is_layer(KIND);
    constexpr bool kLog = norm_is_log(KIND);
    constexpr int NV = 4;   // vectors per thread: 256 * 4 * 16 bytes = 16 KiB
    __shared__ __align__(16) unsigned char tile_raw[256 * NV * 16];
    T* tile = reinterpret_cast<T*>(tile_raw);
    const int t = threadIdx.x;
    const int R = (int)a.cols;
    const int64_t row0 = (int64_t)blockIdx.x * a.rpb;
    const int64_t left = a.rows - row0;
    const int nrows = left < a.rpb ? (int)left : a.rpb;
    const int n = nrows * R;
    const T* src = (const T*)a.in + row0 * R;
    T* dst = (T*)a.out + row0 * R;
    const int tpr = a.tpr;
    const int tx = t & (tpr - 1);
    const int g = t >> a.tpr_log2;
    const int groups = 256 >> a.tpr_log2;
    // gamma / beta first: their trip to L2 then runs beside the tile's loads instead of after the barrier.
    // (Every lane loads from an index inside the row, with no branch around a load, so the loads go out together:
    // with a test per element the compiler waited for each 2-byte load before the next - fourteen trips to L2 per
    // workgroup, a quarter of the f16 launch: [170327, 197] 40.7 us against 29.3 without gamma / beta.)
    T graw[kSoft ? 1 : EPL], braw[kSoft ? 1 : EPL];
    if constexpr (!kSoft) {
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            graw[i] = Elem<T>::narrow((CT)1);
            braw[i] = Elem<T>::narrow((CT)0);
        }
        if (a.gamma) {
#pragma unroll
            for (int i = 0; i < EPL; ++i) graw[i] = ((const T*)a.gamma)[min(tx + i * tpr, R - 1)];
        }
        if (a.beta) {
#pragma unroll
            for (int i = 0; i < EPL; ++i) braw[i] = ((const T*)a.beta)[min(tx + i * tpr, R - 1)];
        }
    }
    {
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
    }
    __syncthreads();
    const CT fill = kSoft ? neg_inf<CT>() : (CT)0;
    // a lane keeps its columns from row to row: gamma / beta, fetched before the tile, are widened once
    CT gam[kSoft ? 1 : EPL], bet[kSoft ? 1 : EPL];
    if constexpr (!kSoft) {
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            gam[i] = Elem<T>::widen(graw[i]);
            bet[i] = Elem<T>::widen(braw[i]);
        }
    }
    for (int r = g; r < nrows; r += groups) {
        T* row = tile + r * R;
        CT x[EPL];
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            // Read from an index clamped into the row, all lanes, then select. (Behind a test per element the 2-byte LDS
            // reads went out one at a time, each waited for before the next; and a value that only the kept side of a
            // select uses is moved back behind the test, so the reads are pinned first.)
            const int c = tx + i * tpr;
            x[i] = Elem<T>::widen(row[c < R ? c : R - 1]);
        }
#pragma unroll
        for (int i = 0; i < EPL; ++i) asm volatile("" : "+v"(x[i]));
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int c = tx + i * tpr;
            x[i] = c < R ? x[i] : fill;
        }
        if constexpr (kSoft) {
            CT m = neg_inf<CT>();
#pragma unroll
            for (int i = 0; i < EPL; ++i) m = MaxC<CT>::comb(m, x[i]);
            m = group_reduce<MaxC<CT>>(m, tpr);
            CT s = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i) {
                const CT d = x[i] - m;
                const CT e = exp_ct<T>(d);
                s += e;
                x[i] = kLog ? d : e;
            }
            s = group_reduce<SumC<CT>>(s, tpr);
            const CT k = kLog ? log_ct<T>(s) : (CT)1 / s;
#pragma unroll
            for (int i = 0; i < EPL; ++i) x[i] = kLog ? x[i] - k : x[i] * k;
        } else {
            // (a row may be three elements: the lane's own sum is taken in the wide type too, or the
            // mean of a row whose spread is small against its offset loses digits that matter)
            ST s = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i) s += (ST)x[i];
            const ST sum = group_reduce<SumC<ST>>(s, tpr);
            const ST m0 = sum * (ST)a.inv_cols;
            const ST mean = fma_ct(fma_ct(-m0, (ST)a.cols, sum), (ST)a.inv_cols, m0);
            const CT mean_hi = (CT)mean;
            const CT mean_lo = (CT)(mean - (ST)mean_hi);
            CT q = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i) {
                const CT d = tx + i * tpr < R ? (x[i] - mean_hi) - mean_lo : (CT)0;
                x[i] = d;
                q += d * d;
            }
            const ST var = group_reduce<SumC<ST>>((ST)q, tpr) * (ST)a.inv_cols;
            const CT rstd = rsqrt_ct((CT)var + (CT)a.eps);
#pragma unroll
            for (int i = 0; i < EPL; ++i) x[i] = x[i] * rstd * gam[i] + bet[i];
        }
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int c = tx + i * tpr;
            if (c < R) row[c] = Elem<T>::narrow(x[i]);
        }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e + VEC <= n) {
            store_pack_stream<T, VEC>(dst + e, load_pack<T, VEC>(tile + e));
        } else {
            for (int j = 0; j < VEC; ++j)
                if (e + j < n) dst[e + j] = tile[e + j];
        }
    }
}

// ---- small [cols, L] groups laid back to back: softmax over the middle axis through LDS --------
// A contiguous [batch, cols, L] tensor with cols * L small ([N, 4, 64], [N, 2, 3], [B, T, 4, 12]),
// softmax over cols: a workgroup brings a.rpb whole groups (16 KiB, a multiple of VEC groups) into
// LDS with aligned 128-bit loads, one lane per (group, inner position) normalises its column of
// `cols` elements at stride L in place, and the tile leaves with aligned 128-bit stores.
template <int KIND, class T, int VEC, bool PADDED>
__global__ void __launch_bounds__(256) norm_group_tile_kernel(const NormArgs a, int L, int64_t batch) {
    constexpr bool padded = PADDED;
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "a softmax kernel");
    using CT = typename Elem<T>::Wide;
    constexpr bool kLog = norm_is_log(KIND);
    constexpr int NV = 4;  // vectors per thread: 256 * 4 * 16 bytes = 16 KiB
    // The tile is kept with one pad slot of 4 bytes (one 8-byte element) after every 128 bytes: the lanes
    // of a wavefront walk columns whose starts are a whole group apart, and a group of 128 bytes or a
    // multiple would put them all on the same LDS bank.
    constexpr int PER = 128 / sizeof(T);                     // elements between pad slots
    constexpr int PAD = sizeof(T) >= 4 ? 1 : 4 / sizeof(T);  // elements per pad slot
    // (PADDED only where the groups' starts would collide: the pad costs the vector LDS accesses)
    auto pad = [](int e) { return PADDED ? e + e / PER * PAD : e; };
    __shared__ __align__(16) unsigned char tile_raw[256 * NV * 16 + (256 * NV * 16 / 128) * 8];
    T* tile = reinterpret_cast<T*>(tile_raw);
    const int t = threadIdx.x;
    const int C = (int)a.cols;
    const int G = C * L;
    const int64_t g0 = (int64_t)blockIdx.x * a.rpb;
    const int64_t left = batch - g0;
    const int ngroups = left < a.rpb ? (int)left : a.rpb;
    const int n = ngroups * G;
    const T* src = (const T*)a.in + g0 * G;
    T* dst = (T*)a.out + g0 * G;
    {
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
    }
    __syncthreads();
    const int npos = ngroups * L;
    for (int o = t; o < npos; o += 256) {
        const int g = o / L, i = o - g * L;
        const int base = g * G + i;
        CT m = neg_inf<CT>();
        for (int c = 0; c < C; ++c) m = MaxC<CT>::comb(m, Elem<T>::widen(tile[pad(base + c * L)]));
        using ST = typename StatType<T>::type;
        ST total = 0;
        for (int c = 0; c < C; ++c) total += (ST)exp_ct<T>(Elem<T>::widen(tile[pad(base + c * L)]) - m);
        const CT s = (CT)total;
        const CT k = kLog ? log_ct<T>(s) : (CT)1 / s;
        for (int c = 0; c < C; ++c) {
            T* q = tile + pad(base + c * L);
            const CT d = Elem<T>::widen(*q) - m;
            *q = Elem<T>::narrow(kLog ? d - k : exp_ct<T>(d) * k);
        }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int e = (t + u * 256) * VEC;
        if (e + VEC <= n) {
            Pack<T, VEC> o;
            if constexpr (!padded) {
                o = load_pack<T, VEC>(tile + e);
            } else {
                const T* q = tile + pad(e);
#pragma unroll
                for (int j = 0; j < VEC; ++j) o.v[j] = q[j];
            }
            store_pack_stream<T, VEC>(dst + e, o);
        } else {
            for (int j = 0; j < VEC; ++j)
                if (e + j < n) dst[e + j] = tile[pad(e + j)];
        }
    }
}

// ---- mid-sized [cols, L] slabs with a narrow inner dim: one workgroup per slab, through LDS -----
// softmax over the middle axis of a contiguous [batch, cols, L] with L narrow (3 ... 64 elements) and
// slabs of 2 ... 64 KiB ([B, 1000, 3], [B, 768, 60], [B, 1024, 33]: attention pooling over a
// sequence with a few heads). Lanes along L idle, a lane per inner position holds up to 64 values
// and reads 2-byte pieces. Here a workgroup brings its whole slab into LDS with 128-bit loads
// (unaligned when the slab starts off a 16-byte boundary), groups of `tpc` lanes share a column
// and walk it at stride L, and the slab leaves with 128-bit stores.
template <int KIND, class T, int VEC>
__global__ void __launch_bounds__(256) norm_slab_kernel(const NormArgs a, int L, int tpc_log2) {
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "a softmax kernel");
    using CT = typename Elem<T>::Wide;
    constexpr bool kLog = norm_is_log(KIND);
    extern __shared__ __align__(16) unsigned char slab_raw[];
    T* tile = reinterpret_cast<T*>(slab_raw);
    const int t = threadIdx.x;
    const int C = (int)a.cols;
    const int n = C * L;
    const T* src = (const T*)a.in + (int64_t)blockIdx.x * n;
    T* dst = (T*)a.out + (int64_t)blockIdx.x * n;
    const int nvec = n / VEC;
    for (int iv = t; iv < nvec; iv += 256) store_pack<T, VEC>(tile + iv * VEC, load_pack_unaligned<T, VEC>(src + iv * VEC));
    for (int e = nvec * VEC + t; e < n; e += 256) tile[e] = src[e];
    __syncthreads();
    const int tpc = 1 << tpc_log2;
    const int lane = t & (tpc - 1);
    const int ngrp = 256 >> tpc_log2;
    for (int i = t >> tpc_log2; i < L; i += ngrp) {
        T* p = tile + i;
        CT m = neg_inf<CT>();
        for (int c = lane; c < C; c += tpc) m = MaxC<CT>::comb(m, Elem<T>::widen(p[c * L]));
        m = group_reduce<MaxC<CT>>(m, tpc);
        using ST = typename StatType<T>::type;
        ST total = 0;
        for (int c = lane; c < C; c += tpc) total += (ST)exp_ct<T>(Elem<T>::widen(p[c * L]) - m);
        const CT s = (CT)group_reduce<SumC<ST>>(total, tpc);
        const CT k = kLog ? log_ct<T>(s) : (CT)1 / s;
        for (int c = lane; c < C; c += tpc) {
            const CT d = Elem<T>::widen(p[c * L]) - m;
            p[c * L] = Elem<T>::narrow(kLog ? d - k : exp_ct<T>(d) * k);
        }
    }
    __syncthreads();
    for (int iv = t; iv < nvec; iv += 256) store_pack_unaligned<T, VEC>(dst + iv * VEC, load_pack<T, VEC>(tile + iv * VEC));
    for (int e = nvec * VEC + t; e < n; e += 256) dst[e] = tile[e];
}

// ---- streaming rows: online statistics, then a second sweep ------------------

// running (max, sum of exp(x - max)); the sum may be carried in a wider type ST
template <class CT, class ST = CT> struct SoftStat {
    CT m;
    ST s;
};
template <class T, class CT, class ST = CT> struct SoftStatOp {
    __device__ static __forceinline__ SoftStat<CT, ST> comb(SoftStat<CT, ST> a, SoftStat<CT, ST> b) {
        SoftStat<CT, ST> r;
        r.m = MaxC<CT>::comb(a.m, b.m);
        // a side that has seen nothing (m = -inf, s = 0) must not produce inf - inf
        ST sa = a.s == (ST)0 ? (ST)0 : a.s * (ST)exp_ct<T>(a.m - r.m);
        ST sb = b.s == (ST)0 ? (ST)0 : b.s * (ST)exp_ct<T>(b.m - r.m);
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

// SHIFT (VEC > 1 only): rows contiguous along the axis whose START is only element-aligned (odd
// row lengths: 50257-wide logits). Vectors are taken at 16-byte aligned addresses all the same:
// vector iv of a row covers its elements iv * VEC - m ... + VEC - 1, m = the row's misalignment,
// and positions outside 0 .. cols - 1 are masked. (An aligned vector that holds one valid
// element lies in that element's page, so the over-read at both ends is safe.) Input, output
// and residual rows share m: the caller checks that their bases and row pitches agree mod 16 bytes.
//
// TI: the INPUT's element type when it is not the output's. NormalizationOps promote a non-float input to
// FloatBinaryType<T> inside the op (hpt/src/backends/cpu/tensor_internal/normalization.rs:205-221); here the
// conversion is part of the load - TI -> T with one rounding, exactly what a separate `astype` would
// have stored, then widened to the compute type - so an integer tensor is normalised in one launch
// and no promoted copy goes through HBM.
template <class T, class TI> __device__ __forceinline__ typename Elem<T>::Wide promoted_input(TI x) {
    using CT = typename Elem<T>::Wide;
    if constexpr (std::is_same<T, TI>::value) {
        return Elem<T>::widen(x);
    } else {
        static_assert(!Elem<TI>::is_float && Elem<T>::is_float, "promotion is integer -> float");
        const CT f = (CT)Elem<TI>::cmp(x);  // (bool: 0 or 1)
        if constexpr (sizeof(T) < sizeof(CT)) return Elem<T>::widen(Elem<T>::narrow(f));
        else return f;
    }
}

template <int KIND, class T, int VEC, bool SHIFT = false, class TI = T>
__global__ void __launch_bounds__(1024) row_stream_kernel(const NormArgs a) {
    static_assert(!SHIFT || VEC > 1, "SHIFT is a vector mode");
    static_assert(std::is_same<T, TI>::value || (!SHIFT && KIND <= NORM_LAYERNORM),
                  "promoted inputs: plain kinds, rows on the vector grid");
    using CT = typename Elem<T>::Wide;
    __shared__ __align__(16) unsigned char smem_raw[16 * 3 * sizeof(double)];
    const int tpr = a.tpr;
    const int tx = threadIdx.x & (tpr - 1);
    const int ty = threadIdx.x >> a.tpr_log2;
    const int64_t row = (int64_t)blockIdx.x * a.rpb + ty;
    const bool valid = row < a.rows;
    const TI* in_row = (const TI*)a.in + (valid ? offset_of(a.kept_in, row) : 0);
    T* out_row = (T*)a.out + (valid ? offset_of(a.kept_out, row) : 0);
    const int m = SHIFT ? (int)(((uintptr_t)in_row / sizeof(T)) % VEC) : 0;
    const int64_t nv = SHIFT ? (a.cols + m + VEC - 1) / VEC : a.cols / VEC;
    // is element j of vector iv inside the row?
    auto inside = [&](int64_t iv, int j) {
        if constexpr (!SHIFT) return true;
        const int64_t e = iv * VEC + j - m;
        return e >= 0 && e < a.cols;
    };
    const bool one_dim = a.norm_in.n <= 1;
    constexpr bool kLog = norm_is_log(KIND);
    constexpr bool kCausal = norm_is_causal(KIND);
    constexpr bool kRes = KIND == NORM_ADD_LAYERNORM;
    // causal kinds: this row keeps columns 0 .. limit - 1; the rest is never read and counts as -inf
    int64_t limit = a.cols;
    if constexpr (kCausal) {
        limit = valid ? row % a.q_rows + a.causal_offset + 1 : 0;
        limit = limit < 0 ? 0 : (limit < a.cols ? limit : a.cols);
    }
    const int64_t nv_lim = kCausal ? (limit + m + VEC - 1) / VEC : nv;
    // the scalar operand of the unfused mul_ has the tensor's dtype
    const CT scale_t = kCausal ? Elem<T>::widen(Elem<T>::narrow((CT)a.scale)) : (CT)1;
    const T* res_row = kRes ? (const T*)a.residual + (valid ? row * a.cols : 0) : nullptr;

    // The fused forms round the intermediate (in + residual, scale * in) to the tensor's dtype, as
    // the separate add / mul_ of the unfused sequence would have stored it.
    auto load = [&](int64_t iv, CT* x) {
        if constexpr (VEC > 1) {
            Pack<TI, VEC> v = load_pack<TI, VEC>(in_row - m + iv * VEC);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[j] = promoted_input<T, TI>(v.v[j]);
            if constexpr (kRes) {
                Pack<T, VEC> r = load_pack<T, VEC>(res_row - m + iv * VEC);
#pragma unroll
                for (int j = 0; j < VEC; ++j) x[j] = Elem<T>::widen(Elem<T>::narrow(x[j] + Elem<T>::widen(r.v[j])));
            }
        } else {
            const int64_t off = one_dim ? iv * a.sa : offset_of(a.norm_in, iv);
            x[0] = promoted_input<T, TI>(in_row[off]);
            if constexpr (kRes) x[0] = Elem<T>::widen(Elem<T>::narrow(x[0] + Elem<T>::widen(res_row[iv])));
        }
        if constexpr (kCausal) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                x[j] = iv * VEC + j - m < limit ? Elem<T>::widen(Elem<T>::narrow(x[j] * scale_t)) : neg_inf<CT>();
        }
    };
    auto store = [&](int64_t iv, const CT* y) {
        if constexpr (VEC > 1) {
            Pack<T, VEC> o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o.v[j] = Elem<T>::narrow(y[j]);
            if constexpr (SHIFT) {
                const int64_t e0 = iv * VEC - m;
                if (e0 >= 0 && e0 + VEC <= a.cols) {
                    store_pack<T, VEC>(out_row + e0, o);
                } else {  // the partial vectors at both ends of the row
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (e0 + j >= 0 && e0 + j < a.cols) out_row[e0 + j] = o.v[j];
                }
            } else {
                store_pack<T, VEC>(out_row + iv * VEC, o);
            }
        } else {
            out_row[iv * a.out_axis_stride] = Elem<T>::narrow(y[0]);
        }
    };

    if constexpr (!norm_is_layer(KIND)) {
        // A lane may sum a whole row by itself here (tpr = 1: thousands of terms one after the
        // other), so f32 rows carry the sum of exponentials in f64: sequential f32 addition would
        // lose about sqrt(n) ulps, which shows in log_softmax values near zero.
        using ST = typename StatType<T>::type;
        SoftStat<CT, ST> st{neg_inf<CT>(), (ST)0};
        if (valid) {
            auto take = [&](int64_t iv, CT* x) {
                if constexpr (SHIFT) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (!inside(iv, j)) x[j] = neg_inf<CT>();
                }
                CT cm = x[0];
#pragma unroll
                for (int j = 1; j < VEC; ++j) cm = MaxC<CT>::comb(cm, x[j]);
                if (cm > st.m) {
                    st.s = st.s == (ST)0 ? (ST)0 : st.s * (ST)exp_ct<T>(st.m - cm);
                    st.m = cm;
                }
                if (st.m > neg_inf<CT>()) {
                    CT part = 0;  // the few elements of one vector add up in the compute type
#pragma unroll
                    for (int j = 0; j < VEC; ++j) part += exp_ct<T>(x[j] - st.m);
                    st.s += (ST)part;
                }
            };
            // four vectors in flight per thread (one per iteration left the memory pipeline mostly idle)
            int64_t iv = tx;
            for (; iv + 3 * tpr < nv_lim; iv += 4 * tpr) {
                CT x[4][VEC];
#pragma unroll
                for (int u = 0; u < 4; ++u) load(iv + u * tpr, x[u]);
#pragma unroll
                for (int u = 0; u < 4; ++u) take(iv + u * tpr, x[u]);
            }
            for (; iv < nv_lim; iv += tpr) {
                CT x[VEC];
                load(iv, x);
                take(iv, x);
            }
        }
        st = stat_all_reduce<SoftStatOp<T, CT, ST>>(st, tpr, (SoftStat<CT, ST>*)smem_raw);
        if (!valid) return;
        const CT k = kLog ? log_ct<T>((CT)st.s) : (CT)((ST)1 / st.s);
        auto finish = [&](int64_t iv, CT* x) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                CT d = x[j] - st.m;
                x[j] = kLog ? d - k : exp_ct<T>(d) * k;
            }
            store(iv, x);
        };
        // The second sweep runs BACKWARDS: the end of the row is what the first sweep read last and
        // what the L2 still holds.
        auto fetch = [&](int64_t iv, CT* x) {
            if (iv < nv_lim) {
                load(iv, x);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) x[j] = neg_inf<CT>();
            }
        };
        // (Shifted rows measured slower that way and keep the forward order.)
        const int64_t cnt = tx < nv ? (nv - tx + tpr - 1) / tpr : 0;  // vectors of this thread
        auto at = [&](int64_t i) { return tx + (SHIFT ? cnt - 1 - i : i) * tpr; };
        int64_t left = cnt;
        for (; left >= 4; left -= 4) {
            CT x[4][VEC];
#pragma unroll
            for (int u = 0; u < 4; ++u) fetch(at(left - 1 - u), x[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) finish(at(left - 1 - u), x[u]);
        }
        for (; left > 0; --left) {
            CT x[VEC];
            fetch(at(left - 1), x);
            finish(at(left - 1), x);
        }
    } else {
        using ST = typename StatType<T>::type;
        MomentStat<ST> st{(ST)0, (ST)0, (ST)0};
        if (valid) {
            // Per lane: sums of (x - k) and (x - k)^2 around the first element k it
            // sees, in the compute type (no division per element, no cancellation
            // against a far origin), turned into (count, mean, M2) once at the end.
            CT k = 0, s1 = 0, s2 = 0;
            int64_t n = 0;
            bool first = true;
            auto take = [&](int64_t iv, CT* x) {
                if (first) {
                    k = x[0];  // the first element of the row this lane sees
                    if constexpr (SHIFT) {
                        if (iv == 0) {
#pragma unroll
                            for (int j = 1; j < VEC; ++j)
                                if (j == m) k = x[j];
                        }
                    }
                    first = false;
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const bool in_row_j = inside(iv, j);
                    const CT d = in_row_j ? x[j] - k : (CT)0;
                    s1 += d;
                    s2 += d * d;
                    n += in_row_j;
                }
            };
            int64_t iv = tx;
            for (; iv + 3 * tpr < nv; iv += 4 * tpr) {  // four vectors in flight per thread
                CT x[4][VEC];
#pragma unroll
                for (int u = 0; u < 4; ++u) load(iv + u * tpr, x[u]);
#pragma unroll
                for (int u = 0; u < 4; ++u) take(iv + u * tpr, x[u]);
            }
            for (; iv < nv; iv += tpr) {
                CT x[VEC];
                load(iv, x);
                take(iv, x);
            }
            if (n > 0) {
                st.n = (ST)n;
                st.mean = (ST)k + (ST)s1 / st.n;
                st.m2 = (ST)s2 - (ST)s1 * (ST)s1 / st.n;
                if (st.m2 < (ST)0) st.m2 = 0;
            }
        }
        st = stat_all_reduce<MomentStatOp<ST>>(st, tpr, (MomentStat<ST>*)smem_raw);
        if (!valid) return;
        const CT mean_hi = (CT)st.mean;
        const CT mean_lo = (CT)(st.mean - (ST)mean_hi);
        const CT rstd = rsqrt_ct((CT)(st.m2 * (ST)a.inv_cols) + (CT)a.eps);
        auto finish = [&](int64_t iv, CT* x) {
            if constexpr (VEC > 1 && !SHIFT) {
                // aligned rows: gamma / beta come as vectors too (the caller checked their alignment)
                Pack<T, VEC> g, b;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    g.v[j] = Elem<T>::narrow((CT)1);
                    b.v[j] = Elem<T>::narrow((CT)0);
                }
                if (a.gamma) g = load_pack<T, VEC>((const T*)a.gamma + iv * VEC);
                if (a.beta) b = load_pack<T, VEC>((const T*)a.beta + iv * VEC);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    x[j] = ((x[j] - mean_hi) - mean_lo) * rstd * Elem<T>::widen(g.v[j]) + Elem<T>::widen(b.v[j]);
            } else if (SHIFT && iv * VEC - m >= 0 && iv * VEC - m + VEC <= a.cols) {
                // a whole vector of a shifted row: its gamma / beta run starts off a boundary by m
                const int64_t e0 = iv * VEC - m;
                Pack<T, VEC> g, b;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    g.v[j] = Elem<T>::narrow((CT)1);
                    b.v[j] = Elem<T>::narrow((CT)0);
                }
                if (a.gamma) g = load_pack_unaligned<T, VEC>((const T*)a.gamma + e0);
                if (a.beta) b = load_pack_unaligned<T, VEC>((const T*)a.beta + e0);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    x[j] = ((x[j] - mean_hi) - mean_lo) * rstd * Elem<T>::widen(g.v[j]) + Elem<T>::widen(b.v[j]);
            } else {
                // (the end vectors of a shifted row, or single elements: gamma / beta from indices clamped into the row,
                // no branch around a load - with a test per element the compiler waits for every load in turn, and the
                // wavefronts that hold a row's two ends kept the whole row waiting)
                T g[VEC], b[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    g[j] = Elem<T>::narrow((CT)1);
                    b[j] = Elem<T>::narrow((CT)0);
                }
                const int64_t c0 = iv * VEC - m;
                if (a.gamma) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const int64_t col = c0 + j;
                        g[j] = ((const T*)a.gamma)[col < 0 ? 0 : (col < a.cols ? col : a.cols - 1)];
                    }
                }
                if (a.beta) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const int64_t col = c0 + j;
                        b[j] = ((const T*)a.beta)[col < 0 ? 0 : (col < a.cols ? col : a.cols - 1)];
                    }
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    x[j] = ((x[j] - mean_hi) - mean_lo) * rstd * Elem<T>::widen(g[j]) + Elem<T>::widen(b[j]);
            }
            store(iv, x);
        };
        // backwards, as in the softmax branch: the row's end is the part the L2 still holds
        const int64_t cnt = tx < nv ? (nv - tx + tpr - 1) / tpr : 0;
        auto at = [&](int64_t i) { return tx + (SHIFT ? cnt - 1 - i : i) * tpr; };
        int64_t left = cnt;
        for (; left >= 4; left -= 4) {
            CT x[4][VEC];
#pragma unroll
            for (int u = 0; u < 4; ++u) load(at(left - 1 - u), x[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) finish(at(left - 1 - u), x[u]);
        }
        for (; left > 0; --left) {
            CT x[VEC];
            load(at(left - 1), x);
            finish(at(left - 1), x);
        }
    }
}

// ---- few, very long rows: a row is shared by many workgroups ------------------------------
// One workgroup per row leaves most of the chip idle when there are fewer rows than compute
// units (a batch of 32 rows of 131072 logits). Here S workgroups take a slice of the row each:
//   row_split_stats_kernel     partial statistics of a slice: softmax (max, sum of exp(x - max)),
//                              layernorm sums of (x - k), (x - k)^2 with k the row's first element
//   row_split_apply_kernel     folds the S partials of its row into (max, 1/sum or ln sum) or
//                              (mean_hi, mean_lo, rstd), re-reads the slice and writes the result
// Input rows are contiguous along the axis (any row offsets), the output is contiguous.
struct RowSplitArgs {
    const void* in;
    void* out;
    const void* gamma;
    const void* beta;
    const void* residual;  // NORM_ADD_LAYERNORM
    void* part;            // [rows][S] partials (16 bytes each at most)
    Dims kept_in;
    int64_t rows, cols;
    int64_t chunk_v;       // vectors per slice
    double eps, inv_cols;
    int S;
};

template <class ST> struct SumPair {
    ST a, b;
};
template <class ST> struct SumPairOp {
    __device__ static __forceinline__ SumPair<ST> comb(SumPair<ST> x, SumPair<ST> y) { return SumPair<ST>{x.a + y.a, x.b + y.b}; }
};

// UA: rows whose length or start is off the 16-byte grid. The vectors are unaligned, and a row's last
// vector is taken from the row's end backwards: it shares its first `skip` elements with the vector
// before (the statistics leave them out, the last pass does not store them).
template <int VEC, bool UA> __device__ __forceinline__ int64_t row_split_vectors(int64_t cols) {
    return UA ? (cols + VEC - 1) / VEC : cols / VEC;
}
template <int VEC, bool UA> __device__ __forceinline__ int64_t row_split_start(int64_t iv, int64_t cols) {
    return UA ? min(iv * VEC, cols - VEC) : iv * VEC;
}
template <class T, int VEC, bool UA> __device__ __forceinline__ Pack<T, VEC> row_split_pack(const T* p) {
    if constexpr (UA) return load_pack_unaligned<T, VEC>(p);
    else return load_pack<T, VEC>(p);
}

// the VEC elements of a row from element e0 on, with the residual added where the kind says so
template <int KIND, class T, int VEC, bool UA>
__device__ __forceinline__ void row_split_load(const RowSplitArgs& a, const T* in_row, int64_t row, int64_t e0,
                                               typename Elem<T>::Wide (&x)[VEC]) {
    const Pack<T, VEC> v = row_split_pack<T, VEC, UA>(in_row + e0);
#pragma unroll
    for (int j = 0; j < VEC; ++j) x[j] = Elem<T>::widen(v.v[j]);
    if constexpr (KIND == NORM_ADD_LAYERNORM) {
        const Pack<T, VEC> r = row_split_pack<T, VEC, UA>((const T*)a.residual + row * a.cols + e0);
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[j] = Elem<T>::widen(Elem<T>::narrow(x[j] + Elem<T>::widen(r.v[j])));
    }
}

template <int KIND, class T, int VEC, bool UA>
__global__ void __launch_bounds__(256) row_split_stats_kernel(const RowSplitArgs a) {
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    __shared__ __align__(16) unsigned char smem_raw[16 * 2 * sizeof(double)];
    const int64_t row = blockIdx.y;
    const T* in_row = (const T*)a.in + offset_of(a.kept_in, row);
    const int64_t nv = row_split_vectors<VEC, UA>(a.cols);
    const int64_t v0 = (int64_t)blockIdx.x * a.chunk_v, v1 = min(nv, v0 + a.chunk_v);
    if constexpr (!norm_is_layer(KIND)) {
        SoftStat<CT, ST> st{neg_inf<CT>(), (ST)0};
        for (int64_t iv = v0 + threadIdx.x; iv < v1; iv += 256) {
            CT x[VEC];
            const int64_t e0 = row_split_start<VEC, UA>(iv, a.cols);
            row_split_load<KIND, T, VEC, UA>(a, in_row, row, e0, x);
            if constexpr (UA) {
                const int skip = (int)(iv * VEC - e0);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (j < skip) x[j] = neg_inf<CT>();
            }
            CT cm = x[0];
#pragma unroll
            for (int j = 1; j < VEC; ++j) cm = MaxC<CT>::comb(cm, x[j]);
            if (cm > st.m) {
                st.s = st.s == (ST)0 ? (ST)0 : st.s * (ST)exp_ct<T>(st.m - cm);
                st.m = cm;
            }
            if (st.m > neg_inf<CT>()) {
                CT part = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) part += exp_ct<T>(x[j] - st.m);
                st.s += (ST)part;
            }
        }
        st = block_reduce<SoftStatOp<T, CT, ST>>(st, (SoftStat<CT, ST>*)smem_raw);
        if (threadIdx.x == 0) ((SoftStat<CT, ST>*)a.part)[row * a.S + blockIdx.x] = st;
    } else {
        // the shift k is the row's first element (after the residual, if any): the same for every slice
        CT k;
        {
            CT x0[VEC];
            row_split_load<KIND, T, VEC, UA>(a, in_row, row, 0, x0);
            k = x0[0];
        }
        CT s1 = 0, s2 = 0;
        for (int64_t iv = v0 + threadIdx.x; iv < v1; iv += 256) {
            CT x[VEC];
            const int64_t e0 = row_split_start<VEC, UA>(iv, a.cols);
            row_split_load<KIND, T, VEC, UA>(a, in_row, row, e0, x);
            const int skip = UA ? (int)(iv * VEC - e0) : 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const CT d = (!UA || j >= skip) ? x[j] - k : (CT)0;
                s1 += d;
                s2 += d * d;
            }
        }
        SumPair<ST> sp{(ST)s1, (ST)s2};
        sp = block_reduce<SumPairOp<ST>>(sp, (SumPair<ST>*)smem_raw);
        if (threadIdx.x == 0) ((SumPair<ST>*)a.part)[row * a.S + blockIdx.x] = sp;
    }
}

// The last pass: every workgroup of a row folds the row's S partials itself (at most 512, in the same
// order, so all of them arrive at the same bits; a launch of its own for that would cost more than the
// few hundred loads), then re-reads its slice and writes the result.
template <int KIND, class T, int VEC, bool UA>
__global__ void __launch_bounds__(256) row_split_apply_kernel(const RowSplitArgs a) {
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    __shared__ __align__(16) unsigned char smem_raw[16 * 2 * sizeof(double)];
    const int64_t row = blockIdx.y;
    const T* in_row = (const T*)a.in + offset_of(a.kept_in, row);
    T* out_row = (T*)a.out + row * a.cols;
    CT p0, p1, p2;
    if constexpr (!norm_is_layer(KIND)) {
        SoftStat<CT, ST> st{neg_inf<CT>(), (ST)0};
        for (int i = threadIdx.x; i < a.S; i += 256) st = SoftStatOp<T, CT, ST>::comb(st, ((const SoftStat<CT, ST>*)a.part)[row * a.S + i]);
        st = block_reduce<SoftStatOp<T, CT, ST>>(st, (SoftStat<CT, ST>*)smem_raw);
        p0 = st.m;
        p1 = norm_is_log(KIND) ? log_ct<T>((CT)st.s) : (CT)((ST)1 / st.s);
        p2 = 0;
    } else {
        SumPair<ST> sp{(ST)0, (ST)0};
        for (int i = threadIdx.x; i < a.S; i += 256) sp = SumPairOp<ST>::comb(sp, ((const SumPair<ST>*)a.part)[row * a.S + i]);
        sp = block_reduce<SumPairOp<ST>>(sp, (SumPair<ST>*)smem_raw);
        CT x0[VEC];
        row_split_load<KIND, T, VEC, UA>(a, in_row, row, 0, x0);
        const ST mean = (ST)x0[0] + sp.a * (ST)a.inv_cols;
        ST m2 = sp.b - sp.a * sp.a * (ST)a.inv_cols;
        if (m2 < (ST)0) m2 = 0;
        p0 = (CT)mean;
        p1 = (CT)(mean - (ST)p0);
        p2 = rsqrt_ct((CT)(m2 * (ST)a.inv_cols) + (CT)a.eps);
    }
    const int64_t nv = row_split_vectors<VEC, UA>(a.cols);
    const int64_t v0 = (int64_t)blockIdx.x * a.chunk_v, v1 = min(nv, v0 + a.chunk_v);
    for (int64_t iv = v0 + threadIdx.x; iv < v1; iv += 256) {
        CT x[VEC];
        const int64_t e0 = row_split_start<VEC, UA>(iv, a.cols);
        row_split_load<KIND, T, VEC, UA>(a, in_row, row, e0, x);
        Pack<T, VEC> o;
        if constexpr (norm_is_layer(KIND)) {
            Pack<T, VEC> g, b;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                g.v[j] = Elem<T>::narrow((CT)1);
                b.v[j] = Elem<T>::narrow((CT)0);
            }
            if (a.gamma) g = row_split_pack<T, VEC, UA>((const T*)a.gamma + e0);
            if (a.beta) b = row_split_pack<T, VEC, UA>((const T*)a.beta + e0);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                o.v[j] = Elem<T>::narrow(((x[j] - p0) - p1) * p2 * Elem<T>::widen(g.v[j]) + Elem<T>::widen(b.v[j]));
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const CT d = x[j] - p0;
                o.v[j] = Elem<T>::narrow(norm_is_log(KIND) ? d - p1 : exp_ct<T>(d) * p1);
            }
        }
        if constexpr (UA) {
            const int skip = (int)(iv * VEC - e0);
            if (skip == 0) {
                store_pack_unaligned<T, VEC>(out_row + e0, o);
            } else {  // the row's last vector: only the elements that are its own
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (j >= skip) out_row[e0 + j] = o.v[j];
            }
        } else if constexpr (VEC > 1) store_pack_stream<T, VEC>(out_row + e0, o);
        else out_row[e0] = o.v[0];
    }
}

}  // namespace hpt
