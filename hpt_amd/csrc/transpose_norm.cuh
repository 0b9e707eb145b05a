// Softmax / log_softmax / layernorm when the INPUT is contiguous along the rows
// (the dim that is kept) and strided along the normalised axis, while the
// OUTPUT is contiguous along the axis: the permute([1, 0]) view of a row-major
// matrix. A row does not sit contiguously anywhere in the input, so:
//
//   transposed_stats_kernel     walks the input in address order (lanes along the
//       rows, 1 KiB per wavefront and column) and keeps VEC running row
//       statistics per lane (online max + rescaled sum, or shifted sums ->
//       (n, mean, M2)); S workgroups share the axis so that the chip is full.
//   transposed_finalize_kernel  folds the S partials of each row into the three
//       numbers the last pass needs.
//   transposed_apply_kernel     reads the input a second time (it is still in the
//       256 MB Infinity Cache for the shapes this matters for) in tiles of
//       (8*VEC rows) x (8*VEC cols) per wavefront: lane (rg, cl) loads VEC
//       vectors of VEC consecutive rows, normalises them, and stores VEC
//       vectors of VEC consecutive columns. Both sides move whole 128-byte
//       lines; the transpose is only a renaming of registers: no LDS.
//
// Arithmetic is that of norm_kernels.cuh (the CPU reference's
// hpt/src/backends/cpu/kernels/softmax.rs:81-201 column form and
// hpt/src/backends/cpu/tensor_internal/normalization.rs:126-201).
#pragma once

#include "norm_kernels.cuh"

namespace hpt {

struct TransposedArgs {
    const void* in;
    void* out;
    const void* gamma;
    const void* beta;
    void* stats;      // [batch][S][R] partial statistics
    void* params;     // [batch][3][R] per-row numbers for the last pass
    int64_t sa;       // input stride along the normalised axis
    int64_t bi;       // input stride of the batch dim
    double eps, inv_cols;
    int R;            // rows per batch (contiguous in the input)
    int cols;         // length of the normalised axis
    int S;            // workgroups sharing the axis in the statistics pass
    int cols_per_split;
};

// A partial row statistic over some of the columns.
//   softmax  : (max, sum of exp(x - max)); merged with SoftStatOp.
//   layernorm: (sum of (x - k), sum of (x - k)^2) with k the row's FIRST element,
//              the same shift for every partial of the row, so that partials
//              merge by plain addition and only the last step divides.
template <class CT> struct ShiftedSums {
    CT s1, s2;
};
template <int KIND, class T> struct RowPartial {
    using CT = typename Elem<T>::Wide;
    using type = typename std::conditional<KIND == NORM_LAYERNORM, ShiftedSums<CT>, SoftStat<CT>>::type;
};

// Pass 1: partial row statistics. Lanes run along the rows (a wavefront reads 1 KiB
// of consecutive rows per column), so every lane owns its VEC rows outright: no
// cross-lane merge. Every wavefront takes its own columns; the four wavefronts of a
// workgroup meet in LDS and write one partial per row: partial y of row r goes to
// stats[b][y][r], y = blockIdx.y.
template <int KIND, class T>
__global__ void __launch_bounds__(256) transposed_stats_kernel(const TransposedArgs a) {
    using CT = typename Elem<T>::Wide;
    using Part = typename RowPartial<KIND, T>::type;
    constexpr int VEC = 16 / sizeof(T);
    constexpr int NW = 4;

    const int lane = threadIdx.x & 63;
    // the wavefront index is uniform: say so, and the column arithmetic stays scalar
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // lanes past the last row keep going (they meet the others at the barrier below) on row 0
    const bool valid = (blockIdx.x * 64 + lane) * VEC < a.R;
    const int r0 = valid ? (blockIdx.x * 64 + lane) * VEC : 0;
    // Columns are dealt out round-robin over all P = 4 S wavefronts that share these
    // rows: wavefront p takes columns p, p + P, ... Wavefronts running at the same time
    // then read neighbouring columns, which keeps a power-of-two column pitch from
    // sending them all to the same memory channels.
    const int P = a.S * NW;
    const int pid = blockIdx.y * NW + w;
    const T* base = (const T*)a.in + (int64_t)blockIdx.z * a.bi + r0;

    // per row: softmax (m, s); layernorm s = sum (x - k), s2 = sum (x - k)^2, k = x[row][0]
    CT m[VEC], s[VEC], s2[VEC];
    if constexpr (KIND == NORM_LAYERNORM) {
        Pack<T, VEC> f = load_pack<T, VEC>(base);
#pragma unroll
        for (int k = 0; k < VEC; ++k) m[k] = Elem<T>::widen(f.v[k]);
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) m[k] = neg_inf<CT>();
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        s[k] = 0;
        s2[k] = 0;
    }
    auto fold = [&](const Pack<T, VEC>* v, auto cnt_tag) {
        constexpr int CNT = decltype(cnt_tag)::value;
        if constexpr (KIND == NORM_LAYERNORM) {
#pragma unroll
            for (int i = 0; i < CNT; ++i)
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const CT d = Elem<T>::widen(v[i].v[k]) - m[k];
                    s[k] += d;
                    s2[k] += d * d;
                }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                CT bm = neg_inf<CT>();
#pragma unroll
                for (int i = 0; i < CNT; ++i) bm = MaxC<CT>::comb(bm, Elem<T>::widen(v[i].v[k]));
                if (bm > m[k]) {
                    s[k] = s[k] == (CT)0 ? (CT)0 : s[k] * exp_ct<T>(m[k] - bm);
                    m[k] = bm;
                }
                if (m[k] > neg_inf<CT>()) {
#pragma unroll
                    for (int i = 0; i < CNT; ++i) s[k] += exp_ct<T>(Elem<T>::widen(v[i].v[k]) - m[k]);
                }
            }
        }
    };
    const int64_t stepb = (int64_t)P * a.sa;
    const T* p = base + (int64_t)pid * a.sa;
    int c = pid;
    for (; c + 7 * P < a.cols; c += 8 * P) {  // eight columns in flight per lane
        Pack<T, VEC> v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = load_pack<T, VEC>(p + i * stepb);
        p += 8 * stepb;
        // keep the scheduler from sinking loads into the arithmetic: all eight stay in flight
        __builtin_amdgcn_sched_barrier(0);
        fold(v, std::integral_constant<int, 8>{});
    }
    for (; c < a.cols; c += P) {
        Pack<T, VEC> v = load_pack<T, VEC>(p);
        p += stepb;
        fold(&v, std::integral_constant<int, 1>{});
    }

    // The four wavefronts hold partials of the same rows: fold them through LDS so
    // that one partial per row and workgroup goes to memory.
    __shared__ Part sm[NW - 1][VEC][64];
    Part t[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        if constexpr (KIND == NORM_LAYERNORM) {
            t[k].s1 = s[k];
            t[k].s2 = s2[k];
        } else {
            t[k].m = m[k];
            t[k].s = s[k];
        }
    }
    if (w > 0) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) sm[w - 1][k][lane] = t[k];
    }
    __syncthreads();
    if (w > 0 || !valid) return;
    Part* dst = (Part*)a.stats + ((int64_t)blockIdx.z * a.S + blockIdx.y) * a.R + r0;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
#pragma unroll
        for (int o = 0; o < NW - 1; ++o) {
            const Part u = sm[o][k][lane];
            if constexpr (KIND == NORM_LAYERNORM) {
                t[k].s1 += u.s1;
                t[k].s2 += u.s2;
            } else {
                t[k] = SoftStatOp<T, CT>::comb(t[k], u);
            }
        }
        dst[k] = t[k];
    }
}

// Pass 2 (tiny): fold the partials of every row and turn them into the three
// numbers the last pass needs: softmax (max, 1/sum or ln(sum), -), layernorm
// (mean_hi, mean_lo, 1/sqrt(var + eps)). params is [batch][3][R]. Sixteen lanes
// share a row (blockDim = (16 rows, 16)) and meet in LDS.
template <int KIND, class T>
__global__ void __launch_bounds__(256) transposed_finalize_kernel(const TransposedArgs a) {
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    using Part = typename RowPartial<KIND, T>::type;
    constexpr int LY = 16;
    __shared__ ST sm0[LY][16], sm1[LY][16];
    const int r = blockIdx.x * 16 + threadIdx.x;
    const bool ok = r < a.R;
    const int P = a.S;
    ST acc0, acc1;  // layernorm: sums of s1, s2; softmax: running max, rescaled sum
    if constexpr (KIND == NORM_LAYERNORM) { acc0 = 0; acc1 = 0; }
    else { acc0 = (ST)neg_inf<CT>(); acc1 = 0; }
    if (ok) {
        const Part* sp = (const Part*)a.stats + (int64_t)blockIdx.z * P * a.R + r;
        for (int p = threadIdx.y; p < P; p += LY) {
            const Part t = sp[(int64_t)p * a.R];
            if constexpr (KIND == NORM_LAYERNORM) {
                acc0 += (ST)t.s1;
                acc1 += (ST)t.s2;
            } else {
                SoftStat<CT> x{(CT)acc0, (CT)acc1};
                x = SoftStatOp<T, CT>::comb(x, t);
                acc0 = x.m;
                acc1 = x.s;
            }
        }
    }
    sm0[threadIdx.y][threadIdx.x] = acc0;
    sm1[threadIdx.y][threadIdx.x] = acc1;
    __syncthreads();
    if (threadIdx.y > 0 || !ok) return;
    for (int y = 1; y < LY; ++y) {
        if constexpr (KIND == NORM_LAYERNORM) {
            acc0 += sm0[y][threadIdx.x];
            acc1 += sm1[y][threadIdx.x];
        } else {
            SoftStat<CT> x{(CT)acc0, (CT)acc1}, t{(CT)sm0[y][threadIdx.x], (CT)sm1[y][threadIdx.x]};
            x = SoftStatOp<T, CT>::comb(x, t);
            acc0 = x.m;
            acc1 = x.s;
        }
    }
    CT* p = (CT*)a.params + (int64_t)blockIdx.z * 3 * a.R + r;
    if constexpr (KIND == NORM_LAYERNORM) {
        const ST k = (ST)Elem<T>::widen(((const T*)a.in)[(int64_t)blockIdx.z * a.bi + r]);
        const ST mean = k + acc0 * (ST)a.inv_cols;
        ST m2 = acc1 - acc0 * acc0 * (ST)a.inv_cols;
        if (m2 < (ST)0) m2 = 0;
        const CT hi = (CT)mean;
        p[0] = hi;
        p[a.R] = (CT)(mean - (ST)hi);
        p[2 * (int64_t)a.R] = rsqrt_ct((CT)(m2 * (ST)a.inv_cols) + (CT)a.eps);
    } else {
        p[0] = (CT)acc0;
        p[a.R] = KIND == NORM_SOFTMAX ? (CT)1 / (CT)acc1 : log_ct<T>((CT)acc1);
        p[2 * (int64_t)a.R] = 0;
    }
}

// Pass 3: normalise and transpose, one (8*VEC rows) x (8*VEC cols) tile per wavefront.
template <int KIND, class T>
__global__ void __launch_bounds__(256) transposed_apply_kernel(const TransposedArgs a) {
    using CT = typename Elem<T>::Wide;
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TR = 8 * VEC, TC = 8 * VEC;

    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int rg = lane & 7, cl = lane >> 3;
    // neighbouring workgroups take neighbouring row tiles: their 128-byte reads are
    // adjacent in memory
    const int r0 = blockIdx.x * TR + rg * VEC;
    const int c0 = (blockIdx.y * 4 + w) * TC + cl * VEC;
    if (r0 >= a.R || c0 >= a.cols) return;

    const CT* pp = (const CT*)a.params + (int64_t)blockIdx.z * 3 * a.R + r0;
    const Pack<CT, VEC> p0 = *reinterpret_cast<const Pack<CT, VEC>*>(pp);
    const Pack<CT, VEC> p1 = *reinterpret_cast<const Pack<CT, VEC>*>(pp + a.R);
    Pack<CT, VEC> p2 = p0;
    if constexpr (KIND == NORM_LAYERNORM) p2 = *reinterpret_cast<const Pack<CT, VEC>*>(pp + 2 * (int64_t)a.R);
    Pack<T, VEC> gam, bet;
    if constexpr (KIND == NORM_LAYERNORM) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            gam.v[i] = Elem<T>::narrow((CT)1);
            bet.v[i] = Elem<T>::narrow((CT)0);
        }
        if (a.gamma) gam = load_pack<T, VEC>((const T*)a.gamma + c0);
        if (a.beta) bet = load_pack<T, VEC>((const T*)a.beta + c0);
    }

    const T* base = (const T*)a.in + (int64_t)blockIdx.z * a.bi + r0;
    Pack<T, VEC> v[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = load_pack<T, VEC>(base + (int64_t)(c0 + i) * a.sa);

    T* out = (T*)a.out + ((int64_t)blockIdx.z * a.R + r0) * a.cols + c0;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        Pack<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const CT x = Elem<T>::widen(v[i].v[k]);
            CT y;
            if constexpr (KIND == NORM_LAYERNORM)
                y = ((x - p0.v[k]) - p1.v[k]) * p2.v[k] * Elem<T>::widen(gam.v[i]) + Elem<T>::widen(bet.v[i]);
            else if constexpr (KIND == NORM_SOFTMAX)
                y = exp_ct<T>(x - p0.v[k]) * p1.v[k];
            else
                y = (x - p0.v[k]) - p1.v[k];
            o.v[i] = Elem<T>::narrow(y);
        }
        store_pack_stream<T, VEC>(out + (int64_t)k * a.cols, o);
    }
}

}  // namespace hpt
