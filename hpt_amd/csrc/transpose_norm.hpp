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
// Arithmetic is that of norm_kernels.hpp (the CPU reference's
// hpt/src/backends/cpu/kernels/softmax.rs:81-201 column form and
// hpt/src/backends/cpu/tensor_internal/normalization.rs:126-201).
#pragma once

#include "norm_kernels.hpp"

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
//   softmax  : (max, sum of exp(x - max)), the sum in StatType; merged with SoftStatOp.
//   layernorm: (sum of (x - k), sum of (x - k)^2) with k the row's FIRST element,
//              the same shift for every partial of the row, so that partials
//              merge by plain addition and only the last step divides.
template <class CT> struct ShiftedSums {
    CT s1, s2;
};
template <int KIND, class T> struct RowPartial {
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;  // the sum of exponentials of f32 rows is carried in f64
    using type = typename std::conditional<KIND == NORM_LAYERNORM, ShiftedSums<CT>, SoftStat<CT, ST>>::type;
};

// Pass 1: partial row statistics. Lanes run along the rows (a wavefront reads 1 KiB
// of consecutive rows per column), so every lane owns its VEC rows outright: no
// cross-lane merge. Every wavefront takes its own columns; the wavefronts of a
// workgroup meet in LDS and write one partial per row: partial y of row r goes to
// stats[b][y][r], y = blockIdx.y.
// UA: the inner rows are not whole, aligned vectors (an odd inner length): the same vectors unaligned; the last
// lane of an inner row takes its vector from the row's end backwards, so no load leaves the row, and computes the
// rows it shares with the lane before a second time (the same bits, stored twice).
template <int KIND, class T, int VEC = 16 / sizeof(T), bool UA = false>
__global__ void __launch_bounds__(1024) transposed_stats_kernel(const TransposedArgs a) {
    using CT = typename Elem<T>::Wide;
    using Part = typename RowPartial<KIND, T>::type;
    using ST = typename StatType<T>::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int NW = blockDim.x >> 6;  // wavefronts per workgroup (1...16)

    const int lane = threadIdx.x & 63;
    // the wavefront index is uniform: say so, and the column arithmetic stays scalar
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // lanes past the last row keep going (they meet the others at the barrier below) on row 0
    const bool valid = (blockIdx.x * 64 + lane) * VEC < a.R;
    const int r0 = valid ? (UA ? min((int)(blockIdx.x * 64 + lane) * VEC, a.R - VEC) : (int)(blockIdx.x * 64 + lane) * VEC) : 0;
    // Columns are dealt out round-robin over all P = 4 S wavefronts that share these
    // rows: wavefront p takes columns p, p + P, ... Wavefronts running at the same time
    // then read neighbouring columns, which keeps a power-of-two column pitch from
    // sending them all to the same memory channels.
    const int P = a.S * NW;
    const int pid = blockIdx.y * NW + w;
    const T* base = (const T*)a.in + (int64_t)blockIdx.z * a.bi + r0;

    // per row: softmax (m, s); layernorm s = sum (x - k), s2 = sum (x - k)^2, k = x[row][0]
    CT m[VEC], s[VEC], s2[VEC];
    ST se[VEC];  // softmax: the sum of exponentials
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
        se[k] = 0;
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
                    se[k] = se[k] == (ST)0 ? (ST)0 : se[k] * (ST)exp_ct<T>(m[k] - bm);
                    m[k] = bm;
                }
                if (m[k] > neg_inf<CT>()) {
#pragma unroll
                    for (int i = 0; i < CNT; ++i) se[k] += (ST)exp_ct<T>(Elem<T>::widen(v[i].v[k]) - m[k]);
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
        for (int i = 0; i < 8; ++i) v[i] = UA ? load_pack_unaligned<T, VEC>(p + i * stepb) : load_pack<T, VEC>(p + i * stepb);
        p += 8 * stepb;
        // keep the scheduler from sinking loads into the arithmetic: all eight stay in flight
        __builtin_amdgcn_sched_barrier(0);
        fold(v, std::integral_constant<int, 8>{});
    }
    for (; c < a.cols; c += P) {
        Pack<T, VEC> v = UA ? load_pack_unaligned<T, VEC>(p) : load_pack<T, VEC>(p);
        p += stepb;
        fold(&v, std::integral_constant<int, 1>{});
    }

    // The wavefronts of a workgroup hold partials of the same rows: they meet in LDS
    // (sm[wavefront][k][lane]) and wavefront w folds row k = w, w + NW, ... of every lane, so
    // that one partial per row and workgroup goes to memory.
    Part* sm = (Part*)smem_raw;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        Part t;
        if constexpr (KIND == NORM_LAYERNORM) {
            t.s1 = s[k];
            t.s2 = s2[k];
        } else {
            t.m = m[k];
            t.s = se[k];
        }
        sm[(w * VEC + k) * 64 + lane] = t;
    }
    __syncthreads();
    if (!valid) return;
    Part* dst = (Part*)a.stats + ((int64_t)blockIdx.z * a.S + blockIdx.y) * a.R + r0;
    for (int k = w; k < VEC; k += NW) {
        Part t = sm[k * 64 + lane];
        for (int o = 1; o < NW; ++o) {
            const Part u = sm[(o * VEC + k) * 64 + lane];
            if constexpr (KIND == NORM_LAYERNORM) {
                t.s1 += u.s1;
                t.s2 += u.s2;
            } else {
                t = SoftStatOp<T, CT, ST>::comb(t, u);
            }
        }
        dst[k] = t;
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
        auto take = [&](const Part& t) {
            if constexpr (KIND == NORM_LAYERNORM) {
                acc0 += (ST)t.s1;
                acc1 += (ST)t.s2;
            } else {
                SoftStat<CT, ST> x{(CT)acc0, acc1};
                x = SoftStatOp<T, CT, ST>::comb(x, t);
                acc0 = x.m;
                acc1 = x.s;
            }
        };
        int p = threadIdx.y;
        for (; p + 3 * LY < P; p += 4 * LY) {  // four partials in flight (the kernel is a chain of load latencies)
            Part t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = sp[(int64_t)(p + u * LY) * a.R];
#pragma unroll
            for (int u = 0; u < 4; ++u) take(t[u]);
        }
        for (; p < P; p += LY) take(sp[(int64_t)p * a.R]);
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
            SoftStat<CT, ST> x{(CT)acc0, acc1}, t{(CT)sm0[y][threadIdx.x], sm1[y][threadIdx.x]};
            x = SoftStatOp<T, CT, ST>::comb(x, t);
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

// Pass 3: normalise and transpose in (8*VEC rows) x (8*VEC cols) register tiles. The four
// wavefronts of a workgroup take neighbouring row tiles (512 contiguous bytes of the input per
// column) and each wavefront takes two neighbouring column tiles (256 contiguous bytes of
// the output per row).
template <int KIND, class T>
__global__ void __launch_bounds__(256) transposed_apply_kernel(const TransposedArgs a) {
    using CT = typename Elem<T>::Wide;
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TR = 8 * VEC, TC = 8 * VEC, NC = 2;

    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int rg = lane & 7, cl = lane >> 3;
    const int r0 = (blockIdx.x * 4 + w) * TR + rg * VEC;
    const int c_base = blockIdx.y * (NC * TC) + cl * VEC;
    if (r0 >= a.R || c_base >= a.cols) return;

    const CT* pp = (const CT*)a.params + (int64_t)blockIdx.z * 3 * a.R + r0;
    const Pack<CT, VEC> p0 = *reinterpret_cast<const Pack<CT, VEC>*>(pp);
    const Pack<CT, VEC> p1 = *reinterpret_cast<const Pack<CT, VEC>*>(pp + a.R);
    Pack<CT, VEC> p2 = p0;
    if constexpr (KIND == NORM_LAYERNORM) p2 = *reinterpret_cast<const Pack<CT, VEC>*>(pp + 2 * (int64_t)a.R);

    const T* base = (const T*)a.in + (int64_t)blockIdx.z * a.bi + r0;
    Pack<T, VEC> v[NC][VEC], gam[NC], bet[NC];
    bool have[NC];
#pragma unroll
    for (int s = 0; s < NC; ++s) {
        const int c0 = c_base + s * TC;
        have[s] = c0 < a.cols;
        if (!have[s]) continue;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[s][i] = load_pack<T, VEC>(base + (int64_t)(c0 + i) * a.sa);
        if constexpr (KIND == NORM_LAYERNORM) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                gam[s].v[i] = Elem<T>::narrow((CT)1);
                bet[s].v[i] = Elem<T>::narrow((CT)0);
            }
            if (a.gamma) gam[s] = load_pack<T, VEC>((const T*)a.gamma + c0);
            if (a.beta) bet[s] = load_pack<T, VEC>((const T*)a.beta + c0);
        }
    }

    T* out = (T*)a.out + ((int64_t)blockIdx.z * a.R + r0) * a.cols + c_base;
#pragma unroll
    for (int k = 0; k < VEC; ++k)
#pragma unroll
        for (int s = 0; s < NC; ++s) {
            if (!have[s]) continue;
            Pack<T, VEC> o;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const CT x = Elem<T>::widen(v[s][i].v[k]);
                CT y;
                if constexpr (KIND == NORM_LAYERNORM)
                    y = ((x - p0.v[k]) - p1.v[k]) * p2.v[k] * Elem<T>::widen(gam[s].v[i]) + Elem<T>::widen(bet[s].v[i]);
                else if constexpr (KIND == NORM_SOFTMAX)
                    y = exp_ct<T>(x - p0.v[k]) * p1.v[k];
                else
                    y = (x - p0.v[k]) - p1.v[k];
                o.v[i] = Elem<T>::narrow(y);
            }
            store_pack_stream<T, VEC>(out + (int64_t)k * a.cols + s * TC, o);
        }
}

// ---- the normalised axis is strided in input AND output (softmax over a middle dim) ----------
// Same statistics and finalize passes (the rows are the contiguous inner kept dim, the
// "columns" the axis); the last pass keeps the layout: lanes along the inner dim, each thread
// holds the VEC per-row numbers in registers and walks a slice of the axis with batches of
// loads in flight. out is contiguous: [batch][cols][R].
template <int KIND, class T, int VEC, bool UA = false>
__global__ void __launch_bounds__(256) col_apply_kernel(const TransposedArgs a, int chunk) {
    using CT = typename Elem<T>::Wide;
    constexpr bool kLog = KIND == NORM_LOGSOFTMAX;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    int r0 = (blockIdx.x * 64 + tx) * VEC;
    if (r0 >= a.R) return;
    if constexpr (UA) r0 = min(r0, a.R - VEC);  // the row's last vector, from its end backwards
    const CT* pp = (const CT*)a.params + (int64_t)blockIdx.z * 3 * a.R + r0;
    const Pack<CT, VEC> p0 = UA ? load_pack_unaligned<CT, VEC>(pp) : *reinterpret_cast<const Pack<CT, VEC>*>(pp);
    const Pack<CT, VEC> p1 = UA ? load_pack_unaligned<CT, VEC>(pp + a.R) : *reinterpret_cast<const Pack<CT, VEC>*>(pp + a.R);
    const T* in = (const T*)a.in + (int64_t)blockIdx.z * a.bi + r0;
    T* out = (T*)a.out + (int64_t)blockIdx.z * a.cols * a.R + r0;
    const int c_end = min(a.cols, (int)(blockIdx.y + 1) * chunk);
    auto apply = [&](const Pack<T, VEC>& v, int c) {
        Pack<T, VEC> o;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const CT d = Elem<T>::widen(v.v[k]) - p0.v[k];
            o.v[k] = Elem<T>::narrow(kLog ? d - p1.v[k] : exp_ct<T>(d) * p1.v[k]);
        }
        if constexpr (UA) store_pack_unaligned<T, VEC>(out + (int64_t)c * a.R, o);
        else if constexpr (VEC > 1) store_pack_stream<T, VEC>(out + (int64_t)c * a.R, o);
        else out[(int64_t)c * a.R] = o.v[0];
    };
    auto fetch = [&](int c) {
        if constexpr (UA) return load_pack_unaligned<T, VEC>(in + (int64_t)c * a.sa);
        else return load_pack<T, VEC>(in + (int64_t)c * a.sa);
    };
    int c = blockIdx.y * chunk + ty;
    for (; c + 12 < c_end; c += 16) {  // four positions in flight per thread (thread rows are 4 apart)
        Pack<T, VEC> v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = fetch(c + 4 * u);
#pragma unroll
        for (int u = 0; u < 4; ++u) apply(v[u], c + 4 * u);
    }
    for (; c < c_end; c += 4) apply(fetch(c), c);
}

// ---- a SHORT strided axis: the whole axis in registers ---------------------------------------
// softmax over the channels of [B, C, H, W] (segmentation logits, C = 21; feature maps, C = 128):
// lanes run along the contiguous inner dim, EV elements each, and the threads that share an inner
// position (one for C <= NC; 2, 4, 8 or 16 thread rows for longer axes, channels dealt round-robin)
// load ALL C values of it: C strided vectors, every one of them in flight at once. Max, sum and
// result come from registers (thread rows meet in LDS), and C vectors are stored: one HBM read and
// one write. Only the raw values stay in registers (NC * EV * sizeof(T) <= 256 bytes per thread);
// the exponentials are computed twice (for the sum, then for the result) rather than kept.
struct ColRegArgs {
    const void* in;
    void* out;
    int64_t sa;     // input stride along the axis
    int64_t bi;     // input stride of the batch dim
    int64_t nvec;   // vectors per batch slab along the inner dim: L / EV (UA: rounded up)
    int64_t total;  // batch * nvec
    int64_t L;      // inner length
    int cols;       // axis length (<= NC << ty_log2)
    int ty_log2;    // log2 of the thread rows that share an inner position
};

// Make the compiler forget what it knows about a pack: between two sweeps over the raw values it
// would otherwise keep what the first sweep derived from them (the widened f32 copies of 2-byte
// elements, x - max) alive for the second, at up to twice the registers of the values themselves.
// Deriving again costs an instruction.
template <class T, int N> __device__ __forceinline__ void forget_pack(Pack<T, N>& v) {
    if constexpr (sizeof(T) * N == 16) asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&v)));
    else if constexpr (sizeof(T) * N == 8) asm volatile("" : "+v"(*reinterpret_cast<u32x2*>(&v)));
    else if constexpr (sizeof(T) * N == 4) asm volatile("" : "+v"(*reinterpret_cast<uint32_t*>(&v)));
    else if constexpr (sizeof(T) * N == 2) asm volatile("" : "+v"(*reinterpret_cast<uint16_t*>(&v)));
}

// UA: the inner dim is not whole, aligned vectors (an odd length, odd strides): unaligned vectors all the
// same; the last vector of an inner row is taken from the row's end backwards and stores only the
// elements that the vector before it does not cover.
template <int KIND, class T, int EV, int NC, bool UA = false>
__global__ void __launch_bounds__(256) col_reg_kernel(const ColRegArgs a) {
    static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "a softmax kernel");
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    constexpr bool kLog = KIND == NORM_LOGSOFTMAX;
    __shared__ CT sm[256 * EV];
    const int TY = 1 << a.ty_log2;
    const int TX = 256 >> a.ty_log2;
    const int tx = threadIdx.x & (TX - 1);
    const int ty = threadIdx.x >> (8 - a.ty_log2);
    const int64_t g = (int64_t)blockIdx.x * TX + tx;
    const bool valid = g < a.total;
    int64_t b = 0, q = 0;
    if (valid) {
        if (((uint64_t)(g | a.nvec) >> 32) == 0) {
            b = (uint32_t)g / (uint32_t)a.nvec;
            q = (uint32_t)g - (uint32_t)b * (uint32_t)a.nvec;
        } else {
            b = g / a.nvec;
            q = g - b * a.nvec;
        }
    }
    const int64_t e0 = UA ? min(q * EV, a.L - EV) : q * EV;
    const int skip = (int)(q * EV - e0);  // UA: leading elements that belong to the vector before
    const T* in = (const T*)a.in + b * a.bi + e0;
    T* out = (T*)a.out + b * a.cols * a.L + e0;
    // this thread's channels: ty, ty + TY, ...
    const int mine = valid ? (a.cols - ty + TY - 1) >> a.ty_log2 : 0;
    // A pair of f16 is held as its 32 bits until a sweep takes it apart: a loaded <2 x half> is split in the block of
    // its load, behind the test that guards it, and each of the 64 loads then waits for the one before.
    constexpr bool kBits = std::is_same<T, f16_t>::value && EV == 2;
    using Held = typename std::conditional<kBits, uint32_t, Pack<T, EV>>::type;
    Held raw[NC];
    auto get = [&](int i) -> Pack<T, EV> {
        if constexpr (kBits) return __builtin_bit_cast(Pack<T, EV>, raw[i]);
        else return raw[i];
    };
    auto forget = [&](int i) {
        if constexpr (kBits) asm volatile("" : "+v"(raw[i]));
        else forget_pack(raw[i]);
    };
#pragma unroll
    for (int i = 0; i < NC; ++i)
        if (i < mine) {
            const T* src = in + (int64_t)(ty + (i << a.ty_log2)) * a.sa;
            if constexpr (kBits) {
                if constexpr (UA) __builtin_memcpy(&raw[i], src, 4);
                else raw[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src));
            } else if constexpr (UA) {
                raw[i] = load_pack_unaligned<T, EV>(src);
            } else {
                raw[i] = load_pack_stream<T, EV>(src);
            }
        }
    // (Nothing may look inside a loaded value before every load is out: left alone, the compiler widens a 2-byte value
    // right behind its load, inside the branch that guards it, and so waits for each of the 64 loads before it issues
    // the next.)
#pragma unroll
    for (int i = 0; i < NC; ++i) forget(i);
    // All-reduce over the thread rows of an inner position. With TX < 64 a wavefront holds 64 / TX of
    // them, TX lanes apart: those meet in a shuffle butterfly, and only one partial row per wavefront
    // goes through LDS (for sixteen thread rows, 4 LDS reads per value instead of 16). Every thread of
    // an inner position ends with the same bits: the butterfly adds the same pairs in every lane.
    const int rpw = TX < 64 ? 64 / TX : 1;  // thread rows per wavefront
    const int nrow = TY / rpw;              // partial rows left after the butterfly
    const int prow = ty / rpw;
    auto across = [&](CT(&v)[EV], auto op) {
        if (TY == 1) return;
        if (TX <= 16)
#pragma unroll
            for (int k = 0; k < EV; ++k) v[k] = op(v[k], shfl_xor_any(v[k], 16));
        if (TX <= 32)
#pragma unroll
            for (int k = 0; k < EV; ++k) v[k] = op(v[k], shfl_xor_any(v[k], 32));
        if (nrow == 1) return;
#pragma unroll
        for (int k = 0; k < EV; ++k) sm[(prow * TX + tx) * EV + k] = v[k];
        __syncthreads();
#pragma unroll
        for (int k = 0; k < EV; ++k) {
            CT r = sm[tx * EV + k];
            for (int y = 1; y < nrow; ++y) r = op(r, sm[(y * TX + tx) * EV + k]);
            v[k] = r;
        }
        __syncthreads();
    };
    CT m[EV], kk[EV], sf[EV];
    ST s[EV];  // this thread's sum of exponentials, carried in the wider type
#pragma unroll
    for (int k = 0; k < EV; ++k) {
        m[k] = neg_inf<CT>();
        s[k] = 0;
    }
#pragma unroll
    for (int i = 0; i < NC; ++i)
        if (i < mine)
#pragma unroll
            for (int k = 0; k < EV; ++k) m[k] = MaxC<CT>::comb(m[k], Elem<T>::widen(get(i).v[k]));
    across(m, [](CT x, CT y) { return MaxC<CT>::comb(x, y); });
#pragma unroll
    for (int i = 0; i < NC; ++i) forget(i);
    // Types that are their own compute type (f32, f64) have nothing to widen: the softmax sweep overwrites
    // the raw value with its exponential, which is then taken once per element instead of twice (the
    // second exponential cost a quarter of the kernel's time on f32 [512, 512, 512] over axis 0 or 1).
    constexpr bool kKeepExp = std::is_same<T, CT>::value && !kLog;
#pragma unroll
    for (int i = 0; i < NC; ++i)
        if (i < mine)
#pragma unroll
            for (int k = 0; k < EV; ++k) {
                const CT e = exp_ct<T>(Elem<T>::widen(get(i).v[k]) - m[k]);
                s[k] += (ST)e;
                if constexpr (kKeepExp) raw[i].v[k] = Elem<T>::narrow(e);  // (f32 / f64 only: raw is the pack itself)
            }
    // (the thread's total is rounded to the compute type once; the thread rows then add up along a tree)
#pragma unroll
    for (int k = 0; k < EV; ++k) sf[k] = (CT)s[k];
    across(sf, [](CT x, CT y) { return x + y; });
#pragma unroll
    for (int i = 0; i < NC; ++i) forget(i);
    // (likewise the channel indices and the `i < mine` masks of the load sweep: carried to the store sweep
    // they cost a register per chunk; recomputing them is an instruction each)
    int ty_st = ty, mine_st = mine;
    asm volatile("" : "+v"(ty_st), "+v"(mine_st));
#pragma unroll
    for (int k = 0; k < EV; ++k) kk[k] = kLog ? log_ct<T>(sf[k]) : (CT)1 / sf[k];
#pragma unroll
    for (int i = 0; i < NC; ++i)
        if (i < mine_st) {
            Pack<T, EV> o;
#pragma unroll
            for (int k = 0; k < EV; ++k) {
                if constexpr (kKeepExp) {
                    o.v[k] = Elem<T>::narrow(Elem<T>::widen(get(i).v[k]) * kk[k]);
                } else {
                    const CT d = Elem<T>::widen(get(i).v[k]) - m[k];
                    o.v[k] = Elem<T>::narrow(kLog ? d - kk[k] : exp_ct<T>(d) * kk[k]);
                }
            }
            T* dst = out + (int64_t)(ty_st + (i << a.ty_log2)) * a.L;
            if constexpr (UA) {
                if (skip == 0) {
                    store_pack_unaligned<T, EV>(dst, o);
                } else {
#pragma unroll
                    for (int k = 0; k < EV; ++k)
                        if (k >= skip) dst[k] = o.v[k];
                }
            } else {
                store_pack_stream<T, EV>(dst, o);
            }
        }
}

// ---- the same, for a NARROW inner dim: the slab is walked as a flat array --------------------
// softmax over axis 0 of a contiguous [cols, L] slab with L = 3, 8, 33, 100: lanes along the inner
// dim would leave most of a wavefront idle. Thread t instead owns elements [t * VEC, t * VEC + VEC)
// of every period of Lp = threads * VEC elements, Lp a multiple of L: each vector slot stays on ONE
// inner index for the whole walk, all accesses are aligned 128-bit vectors, and the periods are
// dealt round-robin over the S workgroups of a slab. Statistics: per-slot running (max, rescaled
// sum), folded per inner index in LDS, one partial per workgroup in the layout of
// transposed_stats_kernel (stats[b][y][L]) so that transposed_finalize_kernel serves both. Apply:
// the same walk with the two per-index numbers of each slot in registers.
// UA: the batch slabs do not start on 16-byte boundaries; the same vectors, unaligned.
template <int KIND, class T, int VEC, bool UA = false>
__global__ void __launch_bounds__(1024) col_flat_stats_kernel(const TransposedArgs a, int threads) {
    static_assert(KIND != NORM_LAYERNORM, "a softmax pass");
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    using Part = SoftStat<CT, ST>;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Part* sm = (Part*)smem_raw;
    const int t = threadIdx.x;
    const int L = a.R;
    const int Lp = threads * VEC;
    const int p0 = t * VEC;
    const int64_t total = (int64_t)a.cols * L;
    CT m[VEC];
    ST s[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        m[k] = neg_inf<CT>();
        s[k] = 0;
    }
    auto fold = [&](const Pack<T, VEC>* v, auto cnt_tag) {
        constexpr int CNT = decltype(cnt_tag)::value;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            CT bm = neg_inf<CT>();
#pragma unroll
            for (int i = 0; i < CNT; ++i) bm = MaxC<CT>::comb(bm, Elem<T>::widen(v[i].v[k]));
            if (bm > m[k]) {
                s[k] = s[k] == (ST)0 ? (ST)0 : s[k] * (ST)exp_ct<T>(m[k] - bm);
                m[k] = bm;
            }
            if (m[k] > neg_inf<CT>()) {
#pragma unroll
                for (int i = 0; i < CNT; ++i) s[k] += (ST)exp_ct<T>(Elem<T>::widen(v[i].v[k]) - m[k]);
            }
        }
    };
    if (t < threads) {
        const T* base = (const T*)a.in + (int64_t)blockIdx.z * a.bi;
        const int64_t whole = total / Lp;
        const int S = a.S;
        int64_t it = blockIdx.x;
        for (; it + 3 * S < whole; it += 4 * S) {
            Pack<T, VEC> v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                v[u] = UA ? load_pack_unaligned<T, VEC>(base + (it + u * S) * Lp + p0) : load_pack<T, VEC>(base + (it + u * S) * Lp + p0);
            fold(v, std::integral_constant<int, 4>{});
        }
        for (; it < whole; it += S) {
            Pack<T, VEC> v = UA ? load_pack_unaligned<T, VEC>(base + it * Lp + p0) : load_pack<T, VEC>(base + it * Lp + p0);
            fold(&v, std::integral_constant<int, 1>{});
        }
        if (it == whole) {  // the last, partial period: element by element
            Pack<T, VEC> v;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const int64_t pos = whole * Lp + p0 + k;
                // (the index is clamped and the load unconditional: loads behind a test each wait for the one before)
                const T e = base[pos < total ? pos : total - 1];
                v.v[k] = pos < total ? e : Elem<T>::narrow(neg_inf<CT>());
            }
            fold(&v, std::integral_constant<int, 1>{});
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) sm[p0 + k] = Part{m[k], s[k]};
    }
    __syncthreads();
    // slot p holds inner index p % L: fold the Lp / L slot rows pairwise, upper half into lower half
    const int slot_rows = Lp / L;
    int top = 1;
    while (top < slot_rows) top <<= 1;
    for (int h = top >> 1; h >= 1; h >>= 1) {
        const int n = h * L;
        for (int i = t; i < n; i += blockDim.x)
            if (i + n < Lp) sm[i] = SoftStatOp<T, CT, ST>::comb(sm[i], sm[i + n]);
        __syncthreads();
    }
    Part* dst = (Part*)a.stats + ((int64_t)blockIdx.z * a.S + blockIdx.x) * L;
    for (int c = t; c < L; c += blockDim.x) dst[c] = sm[c];
}

template <int KIND, class T, int VEC, bool UA = false>
__global__ void __launch_bounds__(1024) col_flat_apply_kernel(const TransposedArgs a, int threads, int slices) {
    using CT = typename Elem<T>::Wide;
    constexpr bool kLog = KIND == NORM_LOGSOFTMAX;
    const int t = threadIdx.x;
    if (t >= threads) return;
    const int L = a.R;
    const int Lp = threads * VEC;
    const int p0 = t * VEC;
    const int64_t total = (int64_t)a.cols * L;
    const CT* pp = (const CT*)a.params + (int64_t)blockIdx.z * 3 * L;
    CT pm[VEC], pk[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        const int c = (p0 + k) % L;
        pm[k] = pp[c];
        pk[k] = pp[L + c];
    }
    const T* in = (const T*)a.in + (int64_t)blockIdx.z * a.bi;
    T* out = (T*)a.out + (int64_t)blockIdx.z * total;
    auto apply1 = [&](T x, int k) -> T {
        const CT d = Elem<T>::widen(x) - pm[k];
        return Elem<T>::narrow(kLog ? d - pk[k] : exp_ct<T>(d) * pk[k]);
    };
    const int64_t whole = total / Lp;
    int64_t it = blockIdx.x;
    for (; it + 3 * slices < whole; it += 4 * slices) {
        Pack<T, VEC> v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            v[u] = UA ? load_pack_unaligned<T, VEC>(in + (it + u * slices) * Lp + p0) : load_pack_stream<T, VEC>(in + (it + u * slices) * Lp + p0);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            Pack<T, VEC> o;
#pragma unroll
            for (int k = 0; k < VEC; ++k) o.v[k] = apply1(v[u].v[k], k);
            if constexpr (UA) store_pack_unaligned<T, VEC>(out + (it + u * slices) * Lp + p0, o);
            else store_pack_stream<T, VEC>(out + (it + u * slices) * Lp + p0, o);
        }
    }
    for (; it < whole; it += slices) {
        const Pack<T, VEC> v = UA ? load_pack_unaligned<T, VEC>(in + it * Lp + p0) : load_pack_stream<T, VEC>(in + it * Lp + p0);
        Pack<T, VEC> o;
#pragma unroll
        for (int k = 0; k < VEC; ++k) o.v[k] = apply1(v.v[k], k);
        if constexpr (UA) store_pack_unaligned<T, VEC>(out + it * Lp + p0, o);
        else store_pack_stream<T, VEC>(out + it * Lp + p0, o);
    }
    if (it == whole) {
        T e[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) {  // (clamped, unconditional loads: they go out together)
            const int64_t pos = whole * Lp + p0 + k;
            e[k] = in[pos < total ? pos : total - 1];
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const int64_t pos = whole * Lp + p0 + k;
            if (pos < total) out[pos] = apply1(e[k], k);
        }
    }
}

// ---- single pass: the whole row block lives in registers -------------------------
// When (16 * rgN bytes of consecutive rows) x (all columns) fits the register file of
// one compute unit (16 vectors per thread, up to 1024 threads), a workgroup loads its
// row block ONCE, takes the row statistics from registers (the reference's two-pass
// forms, no shifted sums needed), and stores the transposed result: one HBM read and
// one HBM write per element instead of two reads and one write.
//
// Lane (rg, cgl) of wavefront w: rg = lane % rgN picks VEC consecutive rows (one
// 128-bit vector along the rows); it holds 16 columns as H = 16 / VEC groups of VEC
// consecutive columns, group h starting at column w * 16 * CGW + h * VEC * CGW + cgl * VEC
// (CGW = 64 / rgN). A load instruction therefore reads 16 * rgN contiguous bytes per
// column; a store instruction writes, per row, VEC * CGW consecutive columns.
//
// With rgN = 4 (2) a 128-byte line of the input is shared by two (four) workgroups.
// Workgroups are handed to the eight XCDs (each with its own L2) round-robin, so the
// row blocks are renumbered to put the parts of a line on workgroups i, i + 8, (i + 16,
// i + 24): same XCD, dispatched together, and all but the first hit in L2.
struct TileArgs {
    const void* in;
    void* out;
    const void* gamma;
    const void* beta;
    int64_t sa;  // input stride along the normalised axis
    int64_t bi;  // input stride of the batch dim
    double eps, inv_cols;
    int R;       // rows per batch (contiguous in the input)
    int cols;
    int rg_log2; // log2(rgN), rgN = 2, 4, 8 or 16
    int share_log2;  // log2 of the workgroups that share a 128-byte line of the input (0, 1 or 2)
};

// All-reduce of VEC row values over every thread that holds a piece of the same rows:
// shuffles over the lanes of a wavefront that share rg, then LDS across wavefronts.
template <class Op, class A, int VEC>
__device__ __forceinline__ void tile_all_reduce(A (&v)[VEC], int rgN, int rg, int cgl, int w, int nw, A* part,
                                                A* res) {
    for (int m = rgN; m < 64; m <<= 1) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) v[k] = Op::comb(v[k], shfl_xor_any(v[k], m));
    }
    if (nw == 1) return;
    const int rows = rgN * VEC;
    __syncthreads();  // the slots may still be read from the previous use
    if (cgl == 0) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) part[w * rows + rg * VEC + k] = v[k];
    }
    __syncthreads();
    if ((int)threadIdx.x < rows) {
        A r = part[threadIdx.x];
        for (int o = 1; o < nw; ++o) r = Op::comb(r, part[o * rows + threadIdx.x]);
        res[threadIdx.x] = r;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < VEC; ++k) v[k] = res[rg * VEC + k];
}

// The four pairs of halves of a Pack<f16_t, 8>.
typedef f16_t half2_t __attribute__((ext_vector_type(2)));
struct alignas(16) HalfPairs {
    half2_t p[4];
};

// exp(x - m) of a tile element. f16: exp2(x * log2(e) - m * log2(e)) with the
// scaling folded into the one multiply-add that also widens x (`nml` = -m * log2(e));
// a row of -inf only still yields NaN (-inf + inf). Other types: as everywhere else.
template <class T>
__device__ __forceinline__ typename Elem<T>::Wide tile_exp(T x, typename Elem<T>::Wide m, typename Elem<T>::Wide nml) {
    using CT = typename Elem<T>::Wide;
    if constexpr (std::is_same<T, f16_t>::value) {
        return __builtin_amdgcn_exp2f(widen_fma(x, (CT)1.4426950408889634, nml));
    } else {
        return exp_ct<T>(Elem<T>::widen(x) - m);
    }
}

// Make the compiler forget what it knows about the tile's registers. Between two
// sweeps over a tile of 2-byte elements it would otherwise keep the widened (f32)
// copies of the first sweep alive for the second: twice the registers of the tile
// itself, i.e. spills to scratch memory. Widening again costs one conversion.
template <class T, int VEC> __device__ __forceinline__ void forget_values(Pack<T, VEC> (&v)[16]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int j = 0; j < 16; ++j) asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&v[j])));
    }
}

template <int KIND, class T>
__global__ void __launch_bounds__(1024) transposed_tile_kernel(const TileArgs a) {
    using CT = typename Elem<T>::Wide;
    using ST = typename StatType<T>::type;
    constexpr int VEC = 16 / sizeof(T);
    constexpr int H = 16 / VEC;
    constexpr bool kSoft = KIND != NORM_LAYERNORM;
    constexpr bool kKeepExp = kSoft && sizeof(T) == sizeof(CT);  // exp(x - max) fits back into the tile
    __shared__ __align__(8) unsigned char smem_raw[(16 * 128 + 128) * sizeof(double)];
    ST* part = reinterpret_cast<ST*>(smem_raw);
    ST* res = part + 16 * 128;

    const int rgN = 1 << a.rg_log2;
    const int cgw = 64 >> a.rg_log2;
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int rg = lane & (rgN - 1), cgl = lane >> a.rg_log2;

    int b = blockIdx.x;
    if (a.share_log2 && b < (int)(gridDim.x & ~((8u << a.share_log2) - 1))) {
        const int x = b & 7, q = b >> 3;
        b = ((x + 8 * (q >> a.share_log2)) << a.share_log2) | (q & ((1 << a.share_log2) - 1));
    }
    const int r0 = (b * rgN + rg) * VEC;
    const bool row_ok = r0 < a.R;
    const int gw = VEC * cgw;                       // columns a wavefront covers per group
    const int c_first = w * 16 * cgw + cgl * VEC;   // first column of group 0
    bool col_ok[H];
#pragma unroll
    for (int h = 0; h < H; ++h) col_ok[h] = c_first + h * gw < a.cols;

    const CT one = std::is_same<T, f16_t>::value ? (CT)opaque_one() : (CT)1;  // see widen_fma

    // Every thread loads 16 vectors, unconditionally: a thread whose rows or columns lie
    // outside the tensor reads row block 0 / column 0 instead (always there), and is
    // left out where it would count: its column groups are skipped when the per-thread
    // statistics are folded, and nothing of it is stored. No branch sits between the
    // loads, so all 16 are in flight at once and the first sweep below consumes them in
    // the order they return.
    Pack<T, VEC> v[16];
    {
        const T* base = (const T*)a.in + (int64_t)blockIdx.y * a.bi + (row_ok ? r0 : 0);
#pragma unroll
        for (int h = 0; h < H; ++h) {
            const T* p = base + (col_ok[h] ? (int64_t)(c_first + h * gw) * a.sa : (int64_t)0);
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[h * VEC + i] = load_pack<T, VEC>(p + i * a.sa);
        }
    }
    // gamma / beta of this thread's columns, fetched before anything is stored: a load
    // issued between the stores would have to wait for every store before it. (f64
    // holds too many registers for that and loads them group by group.)
    constexpr bool kHoistAffine = !kSoft && sizeof(T) <= 4;
    Pack<T, VEC> gam[kHoistAffine ? H : 1], bet[kHoistAffine ? H : 1];
    // (an absent gamma / beta still loads, from the start of the input, and the value is
    // then replaced: a load under a branch would make the compiler wait for it, and for
    // every load issued before it, at the end of the branch)
    auto load_affine = [&](int h, Pack<T, VEC>& gp, Pack<T, VEC>& bp) {
        const int c = col_ok[h] ? c_first + h * gw : 0;
        const T* gsrc = a.gamma ? (const T*)a.gamma + c : (const T*)a.in;
        const T* bsrc = a.beta ? (const T*)a.beta + c : (const T*)a.in;
        gp = load_pack<T, VEC>(gsrc);
        bp = load_pack<T, VEC>(bsrc);
        Pack<T, VEC> ones, zeros;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            ones.v[i] = Elem<T>::narrow((CT)1);
            zeros.v[i] = Elem<T>::narrow((CT)0);
        }
        // chosen per 32-bit word, not per element
        const u32x4 gw4 = __builtin_bit_cast(u32x4, gp), bw4 = __builtin_bit_cast(u32x4, bp);
        gp = __builtin_bit_cast(Pack<T, VEC>, a.gamma ? gw4 : __builtin_bit_cast(u32x4, ones));
        bp = __builtin_bit_cast(Pack<T, VEC>, a.beta ? bw4 : __builtin_bit_cast(u32x4, zeros));
    };
    if constexpr (kHoistAffine) {
#pragma unroll
        for (int h = 0; h < H; ++h) load_affine(h, gam[h], bet[h]);
    }

    // per row k: p0, p1 (and p2) are what the output pass needs
    CT p0[VEC], p1[VEC], p2[VEC];
    if constexpr (kSoft) {
        CT m[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) m[k] = neg_inf<CT>();
        if constexpr (std::is_same<T, f16_t>::value) {
            // a maximum is exact in any precision: take it on the packed halves, two rows
            // per instruction, and widen the VEC results once
            HalfPairs mp;
#pragma unroll
            for (int q = 0; q < 4; ++q) mp.p[q] = half2_t{(f16_t)-__builtin_huge_valf(), (f16_t)-__builtin_huge_valf()};
#pragma unroll
            for (int h = 0; h < H; ++h) {
                HalfPairs mh = __builtin_bit_cast(HalfPairs, v[h * VEC]);
#pragma unroll
                for (int i = 1; i < VEC; ++i) {
                    const HalfPairs x = __builtin_bit_cast(HalfPairs, v[h * VEC + i]);
#pragma unroll
                    for (int q = 0; q < 4; ++q) mh.p[q] = __builtin_elementwise_max(mh.p[q], x.p[q]);
                }
                if (col_ok[h]) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) mp.p[q] = __builtin_elementwise_max(mp.p[q], mh.p[q]);
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) m[k] = (CT)mp.p[k >> 1][k & 1];
        } else {
#pragma unroll
            for (int h = 0; h < H; ++h) {
                CT mh[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) mh[k] = neg_inf<CT>();
#pragma unroll
                for (int i = 0; i < VEC; ++i)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) mh[k] = MaxC<CT>::comb(mh[k], Elem<T>::widen(v[h * VEC + i].v[k]));
                if (col_ok[h]) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) m[k] = MaxC<CT>::comb(m[k], mh[k]);
                }
            }
        }
        forget_values(v);
        tile_all_reduce<MaxC<CT>, CT, VEC>(m, rgN, rg, cgl, w, nw, (CT*)part, (CT*)res);
        CT s[VEC], nml[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            s[k] = 0;
            nml[k] = -m[k] * (CT)1.4426950408889634;  // -max * log2(e), see tile_exp
        }
#pragma unroll
        for (int h = 0; h < H; ++h) {
            CT sh[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) sh[k] = 0;
#pragma unroll
            for (int i = 0; i < VEC; ++i)
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const CT e = tile_exp<T>(v[h * VEC + i].v[k], m[k], nml[k]);
                    sh[k] += e;
                    if constexpr (kKeepExp && KIND == NORM_SOFTMAX) v[h * VEC + i].v[k] = Elem<T>::narrow(e);
                }
            if (col_ok[h]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) s[k] += sh[k];
            }
        }
        forget_values(v);
        tile_all_reduce<SumC<CT>, CT, VEC>(s, rgN, rg, cgl, w, nw, (CT*)part, (CT*)res);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            p0[k] = m[k];
            p1[k] = KIND == NORM_SOFTMAX ? (CT)1 / s[k] : log_ct<T>(s[k]);
            p2[k] = nml[k];
        }
    } else {
        ST sum[VEC];
        if constexpr (sizeof(ST) > sizeof(CT)) {
            // (f32 rows: the lane's own sum in the wide type too, or a row whose spread is small against its
            // offset loses digits of the mean that matter: offset 1000, spread 1 came out 9e-6 off)
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum[k] = 0;
#pragma unroll
            for (int h = 0; h < H; ++h) {
                ST th[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) th[k] = 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) th[k] += (ST)Elem<T>::widen(v[h * VEC + i].v[k]);
                if (col_ok[h]) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) sum[k] += th[k];
                }
            }
        } else {
            CT t[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) t[k] = 0;
#pragma unroll
            for (int h = 0; h < H; ++h) {
                CT th[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) th[k] = 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) th[k] = widen_fma(v[h * VEC + i].v[k], one, th[k]);
                if (col_ok[h]) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) t[k] += th[k];
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum[k] = (ST)t[k];
        }
        forget_values(v);
        tile_all_reduce<SumC<ST>, ST, VEC>(sum, rgN, rg, cgl, w, nw, part, res);
        ST q[VEC];
        {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                // mean = sum / cols: reciprocal multiply plus one correction step
                const ST m0 = sum[k] * (ST)a.inv_cols;
                const ST mean = fma_ct(fma_ct(-m0, (ST)a.cols, sum[k]), (ST)a.inv_cols, m0);
                p0[k] = (CT)mean;
                if constexpr (sizeof(ST) > sizeof(CT)) p1[k] = (CT)(mean - (ST)p0[k]);
                else p1[k] = 0;
            }
            CT t[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) t[k] = 0;
#pragma unroll
            for (int h = 0; h < H; ++h) {
                CT th[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) th[k] = 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) {
                        CT d = widen_fma(v[h * VEC + i].v[k], one, -p0[k]);
                        if constexpr (sizeof(ST) > sizeof(CT)) d -= p1[k];
                        th[k] += d * d;
                    }
                if (col_ok[h]) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) t[k] += th[k];
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) q[k] = (ST)t[k];
        }
        forget_values(v);
        tile_all_reduce<SumC<ST>, ST, VEC>(q, rgN, rg, cgl, w, nw, part, res);
#pragma unroll
        for (int k = 0; k < VEC; ++k) p2[k] = rsqrt_ct((CT)(q[k] * (ST)a.inv_cols) + (CT)a.eps);
    }

    if (!row_ok) return;
    if constexpr (kHoistAffine) {
        // gamma / beta must have arrived before the first store is issued: loads and
        // stores share one counter, so waiting for them later would also wait for
        // every store issued in between
#pragma unroll
        for (int h = 0; h < H; ++h) {
            asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&gam[h])));
            asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&bet[h])));
        }
    }
    T* out = (T*)a.out + ((int64_t)blockIdx.y * a.R + r0) * a.cols + c_first;
#pragma unroll
    for (int h = 0; h < H; ++h) {
        if (!col_ok[h]) continue;
        CT g[VEC], bt[VEC];
        if constexpr (!kSoft) {
            Pack<T, VEC> gp, bp;
            if constexpr (kHoistAffine) {
                gp = gam[h];
                bp = bet[h];
            } else {
                load_affine(h, gp, bp);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                g[i] = Elem<T>::widen(gp.v[i]);
                bt[i] = Elem<T>::widen(bp.v[i]);
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            Pack<T, VEC> o;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                // x - p0 (max or mean) first, in one step
                const CT d = widen_fma(v[h * VEC + i].v[k], one, -p0[k]);
                CT y;
                if constexpr (KIND == NORM_LAYERNORM) {
                    y = d;
                    if constexpr (sizeof(ST) > sizeof(CT)) y -= p1[k];
                    y = y * p2[k] * g[i] + bt[i];
                } else if constexpr (KIND == NORM_SOFTMAX) {
                    if constexpr (kKeepExp) y = Elem<T>::widen(v[h * VEC + i].v[k]) * p1[k];
                    else y = tile_exp<T>(v[h * VEC + i].v[k], p0[k], p2[k]) * p1[k];
                } else {
                    y = d - p1[k];
                }
                o.v[i] = Elem<T>::narrow(y);
            }
            store_pack_stream<T, VEC>(out + (int64_t)k * a.cols + h * gw, o);
            // one output vector at a time: interleaving several only adds live registers
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

}  // namespace hpt
