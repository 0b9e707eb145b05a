// Host-side shape logic: axis normalisation, dimension coalescing and the
// choice of kernel family and launch shape for reductions and normalisations.
//
// The reference prepares a reduction by coalescing dims, grouping them by
// "reduced or kept" and permuting the reduced axes last
// (hpt/src/backends/cpu/utils/reduce/reduce_template.rs:165-253,
// hpt/src/backends/common/reduce.rs:44-96,
// hpt/src/backends/cpu/utils/reduce/reduce_utils.rs:23-56) and then splits on
// "does a reduced axis have stride 1" (hpt/src/backends/common/reduce.rs:24-33).
// The same preparation is done here, generalised to any strides: whichever
// group (kept or reduced) owns the smallest stride decides which way the lanes
// of a wavefront run, so that they always walk memory in address order.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "common.hpp"

namespace hpt {

void process_axes(const int64_t* axes, int naxes, int ndim, int64_t* out) {
    for (int i = 0; i < naxes; ++i) {
        int64_t a = axes[i];
        for (int j = 0; j < i; ++j)
            if (axes[j] == a) fail(HPT_ERR_PARAM, "Axis %lld is duplicated", (long long)a);
        int64_t v = a < 0 ? a + ndim : a;
        if (ndim > 0 && (v < 0 || v >= ndim))
            fail(HPT_ERR_SHAPE, "Dimension out of range: expected in 0..%d, got %lld", ndim,
                 (long long)v);
        out[i] = v;
    }
    // Two spellings of one axis (-1 and ndim-1) are the same axis.
    for (int i = 0; i < naxes; ++i)
        for (int j = 0; j < i; ++j)
            if (out[j] == out[i]) fail(HPT_ERR_PARAM, "Axis %lld is duplicated", (long long)axes[i]);
}

int reduce_out_dtype(int op, int in) {
    if (in < 0 || in >= HPT_DTYPE_COUNT) fail(HPT_ERR_DTYPE, "invalid dtype %d", in);
    switch (op) {
        case HPT_SUM: case HPT_PROD: case HPT_MAX: case HPT_MIN: case HPT_NANSUM:
        case HPT_NANPROD: case HPT_REDUCEL1: case HPT_SUM_SQUARE:
            return in;
        case HPT_ALL: case HPT_ANY:
            return HPT_BOOL;
        case HPT_MEAN: case HPT_REDUCEL2: case HPT_REDUCEL3: case HPT_LOGSUMEXP:
            // FloatBinaryType<T>: hpt-types/src/promotion/normal_promote/_*.rs
            switch (in) {
                case HPT_BOOL: case HPT_I8: case HPT_I16: case HPT_U8: case HPT_U16: case HPT_F16:
                    return HPT_F16;
                case HPT_I32: case HPT_U32: case HPT_F32: return HPT_F32;
                case HPT_BF16: return HPT_BF16;
                default: return HPT_F64;
            }
        default:
            fail(HPT_ERR_PARAM, "invalid reduce op %d", op);
    }
}

static int64_t iabs(int64_t v) { return v < 0 ? -v : v; }

static int64_t pow2_floor(int64_t v) {
    int64_t p = 1;
    while (p <= v / 2) p *= 2;
    return p;
}
static int64_t pow2_ceil(int64_t v) {
    int64_t p = 1;
    while (p < v && p < ((int64_t)1 << 62)) p *= 2;
    return p;
}

// Append (size, stride) to `d`, merging with the previous entry when the two
// are one dense run: prev.stride == stride * size.
static void push_merged(Dims& d, int64_t size, int64_t stride) {
    if (size == 1) return;
    if (d.n > 0 && d.stride[d.n - 1] == stride * size) {
        d.size[d.n - 1] *= size;
        d.stride[d.n - 1] = stride;
        return;
    }
    if (d.n == kMaxDims)
        fail(HPT_ERR_SHAPE, "view has more than %d non-mergeable dims in one group", kMaxDims);
    d.size[d.n] = size;
    d.stride[d.n] = stride;
    ++d.n;
}

// Largest power-of-two vector width (in elements, at most 16 bytes) that every
// access of the form data + sum(idx_i * stride_i) + inner*1 can use: the base
// address, every other stride and the inner length must be multiples of it.
// Kernels are built for two widths only: the full 16-byte vector or one element.
static int legal_vec(const void* data, size_t elem_size, int64_t inner_len, const Dims& a,
                     const Dims& b, int skip_a_last, int skip_b_last) {
    const int v = (int)(16 / elem_size);
    if (v <= 1) return 1;
    bool ok = ((uintptr_t)data % 16) == 0 && inner_len % v == 0;
    for (int i = 0; ok && i < a.n - skip_a_last; ++i) ok = a.stride[i] % v == 0;
    for (int i = 0; ok && i < b.n - skip_b_last; ++i) ok = b.stride[i] % v == 0;
    return ok ? v : 1;
}

// How many blocks of 256 threads keep an MI355X busy: 256 CUs, each able to
// hold 8 such blocks.
constexpr int64_t kBlocksToFill = 2048;
constexpr int64_t kComputeUnits = 256;  // MI355X

ReducePlan plan_reduce(const void* data, const int64_t* shape, const int64_t* strides, int ndim,
                       const int64_t* axes, int naxes, size_t elem_size, size_t acc_size, bool heavy) {
    ReducePlan p;
    bool is_red[kMaxRank] = {};
    for (int i = 0; i < naxes; ++i) is_red[axes[i]] = true;

    p.K = 1;
    p.R = 1;
    for (int i = 0; i < ndim; ++i) (is_red[i] ? p.R : p.K) *= shape[i];
    if (p.K == 0) {
        p.kind = ReduceKind::Empty;
        return p;
    }
    if (p.R == 0) {
        p.kind = ReduceKind::Identity;
        return p;
    }

    // kept dims keep their logical order (the output is contiguous in it)
    for (int i = 0; i < ndim; ++i)
        if (!is_red[i]) push_merged(p.kept, shape[i], strides[i]);
    // reduced dims may be visited in any order: sort by |stride| descending
    int order[kMaxRank], nr = 0;
    for (int i = 0; i < ndim; ++i)
        if (is_red[i] && shape[i] != 1) order[nr++] = i;
    std::stable_sort(order, order + nr,
                     [&](int a, int b) { return iabs(strides[a]) > iabs(strides[b]); });
    for (int i = 0; i < nr; ++i) push_merged(p.red, shape[order[i]], strides[order[i]]);

    int64_t sr = p.red.n ? iabs(p.red.stride[p.red.n - 1]) : INT64_MAX;
    int64_t sk = p.kept.n ? iabs(p.kept.stride[p.kept.n - 1]) : INT64_MAX;

    // the lean kernels index with 32-bit integers and form sums of two such values
    // (chunk starts plus chunk lengths, positions plus batch steps): stay below 2^30
    const int64_t kI32 = 1 << 30;
    if (p.red.n > 0 && (p.kept.n == 0 || sr <= sk)) {
        // ---- Row: lanes walk the reduced index space ---------------------
        p.kind = ReduceKind::Row;
        int64_t rin = p.red.size[p.red.n - 1];
        p.vec = 1;
        if (p.red.stride[p.red.n - 1] == 1)
            p.vec = legal_vec(data, elem_size, rin, p.kept, p.red, 0, 1);
        p.lean = p.red.n == 1 && p.kept.n <= 1 && p.K <= kI32 && rin <= kI32 &&
                 iabs(p.red.stride[0]) <= kI32;
        if (p.lean && p.red.stride[0] == 2 && elem_size <= 8 &&
            legal_vec(data, elem_size, rin * 2, p.kept, p.red, 0, 1) > 1) {
            // every second element along the row: full vectors, even positions kept
            p.vec = (int)(16 / elem_size);
            p.sstride = 2;
        }
        const int full = (int)(16 / elem_size);
        if (p.lean && p.kept.n == 1 && p.sstride == 1 && full > 1 && p.red.stride[0] == 1 && p.kept.stride[0] == rin &&
            (uintptr_t)data % 16 == 0 && rin * (int64_t)elem_size <= (rin % full == 0 ? 512 : 4096) && p.K * rin * (int64_t)elem_size >= (4ll << 20)) {
            // Short rows laid back to back ([N, 3], [N, 33], [N, 100]): a lane per row (or a few) reads
            // 4..12-byte pieces at a stride. Instead a workgroup brings 16 KiB of consecutive rows into
            // LDS with aligned 128-bit loads, whatever the row length, and the rows are summed from there.
            // Rows of whole vectors gain up to 512 bytes (f32 [N, 100]: 3.4 -> 5.9 TB/s; from 2 KiB on the
            // direct kernel is as fast or faster), other rows up to 4 KiB (f32 [N, 257]: 3.3 -> 5.5).
            const int64_t tile_bytes = 16 << 10;
            int64_t rows = tile_bytes / (rin * (int64_t)elem_size);
            rows -= rows % full;  // tiles start on 16-byte boundaries
            if (rows >= full) {
                p.row_tile = (int)rows;
                p.vec = full;
                p.tpr = (int)std::min<int64_t>(64, pow2_ceil((rin + 7) / 8));
                p.rpb = 256 / p.tpr;
                p.split = p.split_q = p.split_i = 1;
                return p;
            }
        }
        if (p.lean && p.vec == 1 && full > 1 && p.sstride == 1 && p.red.stride[0] == 1 && rin >= 64 * full &&
            (uintptr_t)data % elem_size == 0) {
            // Long contiguous rows whose length, pitch or base is off the 16-byte grid (the sum of a
            // whole array of odd length): the kernel peels each row's first elements up to a 16-byte
            // boundary and its last ones, and reads everything between as aligned vectors.
            p.ragged = true;
            p.vec = full;
        }
        if (p.vec == 1 && full > 1 && p.sstride == 1 && p.red.stride[p.red.n - 1] == 1 && rin >= full &&
            (uintptr_t)data % elem_size == 0) {
            // Shorter contiguous runs off the grid (the batch-norm sums of [N, C, 7, 7]: runs of 49):
            // unaligned 128-bit loads from the run's start on, the last one taken from the run's end.
            p.unaligned = true;
            p.vec = full;
        }
        int64_t nv = p.unaligned ? (p.R / rin) * ((rin + full - 1) / full) : p.R / (p.vec / p.sstride);  // vector loads per output
        // About 8 vector loads per lane; groups of one or two wavefronts per row
        // stream best (each wavefront walks its own long run of the row), and
        // only very long rows get a whole workgroup.
        p.tpr = (int)std::min<int64_t>(128, pow2_ceil((nv + 7) / 8));
        if (nv >= 128 * 64) p.tpr = nv >= 1024 * 32 ? 1024 : 256;
        // from four loads per thread on a whole workgroup per row streams a little better than half of
        // one (f16 [4096, 8192] rows: 12.2 -> 11.8 us); rows with peeled ends are better off with fewer
        // lanes idling through the ends
        else if (nv >= 256 * 4 && !p.ragged) p.tpr = 256;
        int block = std::max(256, p.tpr);
        p.rpb = block / p.tpr;
        int64_t blocks = (p.K + p.rpb - 1) / p.rpb;
        p.split = p.split_q = p.split_i = 1;
        if (blocks < kBlocksToFill / 4) {
            // Too few outputs to fill the chip: a whole workgroup per output when that leaves
            // each thread 8 loads or more, then several workgroups of 256 threads
            // per output, each with a long contiguous share (>= 16 loads per
            // thread, 8 when there are many outputs to amortise the second stage over); about
            // 512 workgroups in all is the measured sweet spot.
            if (p.tpr < 256 && nv >= 256 * 8) {
                p.tpr = 256;
                p.rpb = 1;
            }
            int64_t want = std::max<int64_t>(1, 512 / p.K);  // (never just over two rounds of the compute units)
            int64_t can = nv / (256 * (p.K >= 64 ? 8 : 16));
            int64_t split = std::min<int64_t>(std::min(want, can), 4096);
            if (split > 1) {
                p.tpr = 256;
                p.rpb = 1;
                int64_t rout = p.R / rin;
                int64_t sq = std::min(split, rout);
                int64_t si = std::max<int64_t>(1, split / sq);
                int64_t can_i = std::max<int64_t>(1, (rin / (p.vec / p.sstride)) / p.tpr);
                si = std::min(si, can_i);
                p.split_q = (int)sq;
                p.split_i = (int)si;
                p.split = (int)(sq * si);
            }
        }
    } else {
        // ---- Col: lanes walk the outputs -----------------------------------
        p.kind = ReduceKind::Col;
        const int nk = p.kept.n;
        // A reduction over the MIDDLE axis of a contiguous [B, C, L] whose inner dim divides the 16-byte vector (L = 2
        // or 4 four-byte elements; 2, 4 or 8 two-byte ones): the [C, L] slab is one ROW of C * L elements for the lean
        // row kernel, an element's place in its vector names its output, and a thread keeps L accumulators. Lanes
        // along L would idle, and the flat walk takes two launches.
        {
            const int64_t full = elem_size <= 16 ? (int64_t)(16 / elem_size) : 1;
            if (nk == 2 && p.red.n == 1 && full > 1 && p.kept.stride[1] == 1 && p.kept.size[1] > 1 && p.kept.size[1] <= 8 && full % p.kept.size[1] == 0 &&
                p.red.stride[0] == p.kept.size[1] && p.kept.stride[0] == p.R * p.kept.size[1] && p.R > 64 &&
                (p.R * p.kept.size[1]) % full == 0 && p.R * p.kept.size[1] * (int64_t)elem_size <= (128 << 10) &&
                p.kept.size[0] >= 256 && p.K * p.R * (int64_t)elem_size >= (4ll << 20) && ((uintptr_t)data & 15) == 0) {
                const int64_t L = p.kept.size[1];
                const int64_t shp[2] = {p.kept.size[0], p.R * L}, str[2] = {p.R * L, 1}, ax[1] = {1};
                ReducePlan q = plan_reduce(data, shp, str, 2, ax, 1, elem_size, acc_size, heavy);
                if (q.kind == ReduceKind::Row && q.lean && q.vec == full && !q.ragged && !q.unaligned && q.sstride == 1 &&
                    q.split == 1 && !q.row_tile) {
                    q.interleave = (int)L;
                    q.K = p.K;
                    q.R = p.R;
                    q.kept = p.kept;
                    q.red = p.red;
                    return q;
                }
            }
        }
        // Two kept dims of which the FIRST is the contiguous one (a reduction over the last axis of a
        // permuted view): the lanes must run along that one. List it last; the kernel then scatters
        // its (few) outputs instead of gathering its (many) inputs.
        if (nk == 2 && p.red.n <= 1 && iabs(p.kept.stride[0]) < iabs(p.kept.stride[1]) && p.kept.size[1] <= 65535 &&
            p.kept.size[0] <= kI32 && p.R <= kI32 && iabs(p.kept.stride[0]) <= kI32) {
            std::swap(p.kept.size[0], p.kept.size[1]);
            std::swap(p.kept.stride[0], p.kept.stride[1]);
            p.kept_swapped = true;
        }
        // The same slabs with an inner dim of 3, 5, 6 or 7 elements (points, colours): a row of the kernel whose
        // lanes, in multiples of L, keep an accumulator per vector place. Mid-sized slabs, many of them: groups up to
        // 2 KiB go through LDS tiles (f32 [30000, 100, 3] 9.1 us there against 13.5 here; above, against the flat walk,
        // [20000, 200, 3] 23.1 -> 12.4), few long ones through the flat walk.
        {
            const int64_t full = elem_size <= 8 ? (int64_t)(16 / elem_size) : 1;
            const int64_t L = nk == 2 ? p.kept.size[1] : 0;
            if (nk == 2 && !p.kept_swapped && p.red.n == 1 && full > 1 && p.kept.stride[1] == 1 && L >= 3 && L <= 7 && full % L != 0 &&
                p.red.stride[0] == L && p.kept.stride[0] == p.R * L && p.R * L * (int64_t)elem_size > 2048 &&
                p.R * L * (int64_t)elem_size <= (256 << 10) && p.kept.size[0] >= 512 &&
                p.K * p.R * (int64_t)elem_size >= (4ll << 20) && ((uintptr_t)data % elem_size) == 0) {
                p.kind = ReduceKind::Row;
                p.mod_rows = (int)L;
                p.vec = (int)full;
                p.tpr = p.R * L / full >= 1024 ? 256 : 64;
                p.rpb = 256 / p.tpr;
                return p;
            }
        }
        int64_t kin = nk ? p.kept.size[nk - 1] : 1;
        p.vec = 1;
        if (nk && p.kept.stride[nk - 1] == 1)
            p.vec = legal_vec(data, elem_size, kin, p.kept, p.red, 1, 0);
        const int64_t outer = nk > 1 ? p.kept.size[0] : 1;
        p.lean = p.red.n <= 1 && nk <= 2 && outer <= 65535 && kin <= kI32 && p.R <= kI32 &&
                 (nk == 0 || iabs(p.kept.stride[nk - 1]) <= kI32);
        if (p.kept_swapped && !p.lean) {  // the general kernel numbers its outputs in kept order: undo
            std::swap(p.kept.size[0], p.kept.size[1]);
            std::swap(p.kept.stride[0], p.kept.stride[1]);
            p.kept_swapped = false;
            kin = p.kept.size[nk - 1];
            p.vec = 1;
            if (p.kept.stride[nk - 1] == 1) p.vec = legal_vec(data, elem_size, kin, p.kept, p.red, 1, 0);
        }
        if (p.lean && nk && p.kept.stride[nk - 1] == 2 && elem_size <= 8 &&
            legal_vec(data, elem_size, kin * 2, p.kept, p.red, 1, 0) > 1) {
            // neighbouring outputs sit at every second position: full vectors, even positions kept
            p.vec = (int)(16 / elem_size);
            p.sstride = 2;
        }
        const int full = (int)(16 / elem_size);
        {
            // Small groups laid back to back ([outer, R, kin] with R * kin elements of at most 2 KiB and
            // rows of kin shorter than a wavefront of vectors): 16 KiB tiles of whole groups through LDS.
            const int64_t G = p.R * kin;
            if (nk == 2 && !p.kept_swapped && p.red.n == 1 && full > 1 && p.sstride == 1 && p.kept.stride[1] == 1 &&
                p.red.stride[0] == kin && p.kept.stride[0] == G && (uintptr_t)data % 16 == 0 &&
                G * (int64_t)elem_size <= 2048 && kin * (int64_t)elem_size < 1024 && p.R >= 2 && p.R <= 256 &&
                p.K * p.R * (int64_t)elem_size >= (4ll << 20) && p.kept.size[0] >= 1024) {
                int64_t groups = (16 << 10) / (G * (int64_t)elem_size);
                groups -= groups % full;  // tiles start on 16-byte boundaries
                if (groups >= full) {
                    p.group_tile = (int)groups;
                    p.vec = full;
                    p.lean = true;
                    p.split = 1;
                    p.bx = 256;
                    p.by = 1;
                    p.chunk = 0;
                    return p;
                }
            }
        }
        if (p.lean && nk && !p.kept_swapped && p.vec < full && p.sstride == 1 && full > 1 && p.kept.stride[nk - 1] == 1 &&
            p.red.n == 1 && p.red.stride[0] == kin && (uintptr_t)data % elem_size == 0 &&
            outer * kin * p.R * (int64_t)elem_size >= (8ll << 20)) {
            // (slabs that start off 16-byte boundaries take the same vectors unaligned)
            const bool slabs_aligned = (uintptr_t)data % 16 == 0 && (outer == 1 || p.kept.stride[0] % full == 0);
            // A contiguous [R, kin] slab whose rows are not whole vectors (kin = 3, 33, 257): walk it
            // as a FLAT array of aligned vectors. With a stride between a thread's visits that is a
            // multiple of kin, every vector slot of every thread stays on one column.
            int64_t g = kin, b = full;
            while (b) { int64_t t = g % b; g = b; b = t; }
            const int64_t kp = kin / g;  // threads per period: kp * full elements = full rows
            int64_t tmax = std::min<int64_t>(1024, (int64_t)((64u << 10) / ((size_t)full * acc_size)));
            // (each slab must be worth at least two periods of the walk: small slabs, of which there are
            // many, take fewer threads each)
            tmax = std::min(tmax, kin * p.R / (2 * full));
            if (kp <= tmax && tmax >= 64) {
                p.flat_t = (int)(kp * (tmax / kp));
                p.vec = full;
                p.unaligned = !slabs_aligned;
                const int64_t per_iter = (int64_t)p.flat_t * full;
                const int64_t iters = (kin * p.R + per_iter - 1) / per_iter;
                int64_t cap = std::max<int64_t>(1, (int64_t)((64ll << 20) / acc_size) / p.K);
                // one large workgroup per compute unit measured best (256: 4.4 TB/s, 512: 3.8, 128: 3.7)
                int64_t split = std::min<int64_t>(iters / 4, std::max<int64_t>(1, 256 / outer));
                p.split = (int)std::max<int64_t>(1, std::min(split, cap));
                p.bx = (p.flat_t + 63) / 64 * 64;
                p.by = 1;
                p.chunk = 0;
                return p;
            }
            // Wider rows (kin = 4097, 50257): a period of full / g rows spans several workgroups; every
            // vector slot is one (row phase, column) pair, so no fold inside the workgroup is needed and
            // the partials are [slice][phase][K].
            const int64_t phases = full / g;
            const int64_t xb = (kp + 1023) / 1024;
            if (slabs_aligned && kp > tmax && p.R >= 16 * phases && xb <= 65535 && kin * phases <= kI32) {
                p.flat_t = (int)(((kp + xb - 1) / xb + 63) / 64 * 64);
                p.flat_xb = (int)xb;
                p.flat_phases = (int)phases;
                p.vec = full;
                const int64_t periods = p.R / phases;
                int64_t cap = std::max<int64_t>(1, (int64_t)((64ll << 20) / acc_size) / (p.K * phases));
                int64_t slices = std::min<int64_t>(periods / 4, std::max<int64_t>(1, 256 / (outer * xb)));
                slices = std::max<int64_t>(1, std::min(slices, cap));
                p.split = (int)(slices * phases);
                p.bx = p.flat_t;
                p.by = 1;
                p.chunk = 0;
                return p;
            }
        }
        // Rows that are not whole, aligned vectors (an odd inner length, a base or pitch off 16 bytes):
        // a lane still takes `full` neighbouring outputs, with unaligned 128-bit loads (global memory
        // takes them; now and then one touches two lines) instead of one element at a time - eight
        // times the bytes in flight per lane for f16. The last lane of a row loads its few elements singly.
        // (Worth it when a row is a few wavefronts of such lanes and enough is reduced into each output
        // that the lane's outputs, which it then writes one by one, are a small part of the traffic.)
        if (p.lean && nk && p.vec == 1 && p.sstride == 1 && full > 1 && p.kept.stride[nk - 1] == 1 && kin >= 256 &&
            p.R >= 256 && (uintptr_t)data % elem_size == 0) {
            p.unaligned = true;
            p.vec = full;
        }
        int64_t kv = ((p.lean ? kin : p.K) + (p.unaligned ? full - 1 : 0)) / (p.vec / p.sstride);  // vector columns the lanes spread over
        p.bx = (int)std::min<int64_t>(64, pow2_ceil(kv));
        // A row of vector columns that is not a whole number of wavefronts (96: hidden size 768 in two-byte
        // elements) would leave the last wavefront of every row partly idle: narrower column blocks
        // (32 or 16 lanes, two or four reduced positions per wavefront) that divide it better.
        // Over axis 1, TB/s: f16 [128, 512, 1280] 4.7 -> 6.1, [512, 197, 768] 5.0 -> 5.7, f32 [256, 512, 320] 5.0 -> 6.2.
        if (kv > 64) {
            auto waste = [&](int64_t b) { return (kv + b - 1) / b * b - kv; };
            for (int b = 32; b >= 16; b >>= 1)
                if (waste(p.bx) * 8 > kv && waste(b) < waste(p.bx)) p.bx = b;
        }
        int64_t xblocks = (kv + p.bx - 1) / p.bx * (p.lean ? outer : 1);
        // One wavefront per 64 vector columns streams best when there are enough
        // columns (measured: 832 wavefronts with 128 loads each reach 5.9 TB/s);
        // with fewer, thread rows and then workgroups split the reduced range.
        const int base_by = 64 / p.bx;  // a workgroup is at least one wavefront
        const int64_t kWavesWanted = 768;
        const int uv = p.vec / p.sstride;
        p.by = base_by;
        p.split = 1;
        // r-partitions wanted so that about 768 wavefronts run, each with >= 16 loads
        const int64_t need = (kWavesWanted + xblocks - 1) / xblocks;
        const int64_t can = std::max<int64_t>(1, p.R / 16);
        const int64_t rp = std::min(need, can);
        if (rp > 1) {
            const int64_t bytes = p.K * p.R * (int64_t)elem_size;
            if (bytes >= (8ll << 20)) {
                // Large input: partition over WORKGROUPS first, so that the partitions land
                // on different CUs (48 workgroups of 1024 threads leave 208 CUs idle), and
                // fold the partials in a second launch.
                int64_t cap = std::max<int64_t>(1, (int64_t)((64ll << 20) / acc_size) / p.K);
                if (need > 64) {
                    // Very few column blocks (a narrow inner dim: [N, 3], [N, 33]): aim for ~2048
                    // wavefronts, eight per workgroup (measured best: [32768, 1024] f32 4.7 TB/s with sixteen, 5.3
                    // with eight), up to 256 workgroups per column block.
                    const int64_t slices = std::min((2048 + xblocks - 1) / xblocks, can);
                    int64_t by_waves = std::min<int64_t>(8, pow2_floor(slices));
                    while (by_waves > 1 && (size_t)64 * by_waves * uv * acc_size > (64u << 10)) by_waves /= 2;
                    p.split = (int)std::min<int64_t>(std::min<int64_t>((slices + by_waves - 1) / by_waves, 256), cap);
                    p.by = (int)by_waves * base_by;
                } else {
                    // A power of two of partitions (an even share of a power-of-two axis: whole batches
                    // of eight loads, nobody left with a short last batch), up to four of them as
                    // thread rows of one workgroup: a quarter of the partials, and with four or fewer
                    // no second launch at all. f16 [4096, 8192][:, ::2] over axis 0, 48 workgroup
                    // slices -> 16 of four thread rows: 17.9 -> 14.6 us; f32 [512, 65536] over axis 0,
                    // 3 slices -> one launch of four thread rows: 4.9 -> 6.1 TB/s.
                    // (An op that spends a dozen instructions per element - an exponential, f64 squares of f32
                    // data - needs a second wavefront per SIMD to run beside the loads: eight thread rows. f32
                    // [8192, 4096] over axis 0, us with 4 / 8 thread rows x 16 splits: sum 25.1 / 25.4,
                    // sum_square 27.7 / 25.8, logsumexp 34.7 / 28.4.)
                    const int64_t parts = std::min<int64_t>(pow2_ceil(rp), pow2_floor(can));
                    const int64_t by = std::min<int64_t>(parts, heavy ? 8 : 4);
                    p.split = (int)std::max<int64_t>(1, std::min<int64_t>(parts / by, cap));
                    p.by = (int)by * base_by;
                }
            } else {
                // Small input: one launch, thread rows meet in LDS
                int64_t by = std::min<int64_t>(pow2_ceil(rp), 1024 / p.bx / base_by) * base_by;
                while (by > base_by && (size_t)p.bx * by * uv * acc_size > (64u << 10)) by /= 2;
                p.by = (int)by;
            }
        }
        // Workgroups of several wavefronts each live as long as the launch does, one (or two ...) per
        // compute unit: a count just over a multiple of the 256 compute units leaves a few units with one
        // workgroup more than the rest, and everybody waits for those. f32 [6553, 5120] over axis 0, 20
        // column blocks x splits (workgroups): 12 (240) 24.9 us, 13 (260) 32.0, 16 (320) 29.0, 25 (500)
        // 25.2, 26 (520) 30.1; f32 [43690, 768], 3 column blocks: 85 (255) 26.7 us, 86 (258) 35.6.
        // So the split moves to the nearest count that fills whole rounds of compute units.
        if (p.split > 1 && p.by * p.bx >= 128) {
            const int64_t total = xblocks * p.split;
            const int64_t rounds = (total + kComputeUnits - 1) / kComputeUnits;
            if (total * 10 < rounds * kComputeUnits * 9) {  // less than 90 % of its rounds filled
                int64_t best = p.split, best_dist = -1;
                for (int64_t r = std::max<int64_t>(1, rounds - 1); r <= rounds; ++r) {
                    const int64_t cand = r * kComputeUnits / xblocks;
                    if (cand < 1 || cand > 256 || p.R / (cand * (p.by / base_by)) < 8) continue;
                    const int64_t dist = cand > p.split ? cand - p.split : p.split - cand;
                    if (best_dist < 0 || dist < best_dist) {
                        best = cand;
                        best_dist = dist;
                    }
                }
                const int64_t cap2 = std::max<int64_t>(1, (int64_t)((64ll << 20) / acc_size) / p.K);
                p.split = (int)std::min(best, cap2);
            }
        }
        p.chunk = (p.R + p.split - 1) / p.split;
    }
    return p;
}

static void describe_dims(std::string& s, const char* name, const Dims& d) {
    s += name;
    s += "=[";
    char buf[64];
    for (int i = 0; i < d.n; ++i) {
        snprintf(buf, sizeof buf, "%s%lld:%lld", i ? "," : "", (long long)d.size[i],
                 (long long)d.stride[i]);
        s += buf;
    }
    s += "]";
}

std::string describe(const ReducePlan& p) {
    char buf[256];
    std::string s;
    switch (p.kind) {
        case ReduceKind::Empty: return "empty";
        case ReduceKind::Identity: return "identity";
        case ReduceKind::Row:
            snprintf(buf, sizeof buf, "row%s%s vec=%d tpr=%d rpb=%d rows=%lld cols=%lld split=%d(%dx%d) ",
                     p.row_tile ? "-tile" : p.ragged ? "-ragged" : (p.lean || p.mod_rows) ? "" : "-general", p.sstride == 2 ? "-step2" : p.unaligned ? "-unaligned" : p.interleave > 1 ? "-interleaved" : p.mod_rows ? "-modular" : "", p.vec, p.tpr, p.rpb,
                     (long long)p.K, (long long)p.R, p.split, p.split_q, p.split_i);
            break;
        case ReduceKind::Col:
            snprintf(buf, sizeof buf, "col%s%s vec=%d bx=%d by=%d outs=%lld red=%lld split=%d ",
                     p.group_tile ? "-group-tile" : p.flat_xb ? "-flat-wide" : p.flat_t ? (p.unaligned ? "-flat-unaligned" : "-flat") : p.kept_swapped ? "-swapped" : p.unaligned ? "-unaligned" : p.lean ? "" : "-general",
                     p.sstride == 2 ? "-step2" : "", p.vec,
                     p.flat_t ? p.flat_t : p.bx, p.by,
                     (long long)p.K, (long long)p.R, p.split);
            break;
    }
    s = buf;
    describe_dims(s, "kept", p.kept);
    s += " ";
    describe_dims(s, "red", p.red);
    return s;
}

// ---- normalisation ---------------------------------------------------------

// Softmax rows held in registers and LDS (row_lds_kernel): the smallest of its three launch shapes whose
// slots hold the `nvec` vectors of a row's vector grid; false when none does. 24 + 8 vectors of a four-byte
// type (16 + 8 of a two-byte type) per thread, 256 or 512 threads; twice that per thread, 512 threads.
// Shifted four-byte rows keep four vectors fewer in registers (20 + 8, 44 + 16): the masks of the row ends
// beside 24 or 48 vectors spilled 30 registers, and the spills' traffic showed in the HBM counters (f32
// [640, 50257]: 1.22 times the algorithmic bytes; the aligned [640, 50304]: 1.00).
static bool lds_row_shape(NormPlan& p, int64_t nvec, size_t elem_size, bool shift) {
    const int per = elem_size == 4 ? (shift ? 28 : 32) : 24;
    const int big = elem_size == 4 ? (shift ? 60 : 64) : 48;
    if (nvec <= 256 * per) {
        p.tpr = 256;
        p.nchunk = per;
    } else if (nvec <= 512 * per) {
        p.tpr = 512;
        p.nchunk = per;
    } else if (nvec <= 1024 * per) {
        // one workgroup fills the compute unit either way; sixteen wavefronts of 128 registers keep more loads and
        // stores in flight than eight of 256 (f32 [1024, 128256] log_softmax 217 -> 208 us, f16 [2048, 151936] 262 -> 249,
        // f32 [1024, 100277] 183 -> 171, [2048, 69632] 237 -> 224)
        p.tpr = 1024;
        p.nchunk = per;
    } else if (nvec <= 512 * big) {
        p.tpr = 512;
        p.nchunk = big;
    } else {
        return false;
    }
    p.kind = NormKind::RowReg;
    p.lds_rows = 1;
    p.rpb = 1;
    return true;
}

NormPlan plan_normalize(const void* in_data, const void* out_data, const int64_t* shape,
                        const int64_t* strides, int ndim, int64_t axis, int n_norm_dims,
                        size_t elem_size, bool fused) {
    NormPlan p;
    int64_t total = 1;
    for (int i = 0; i < ndim; ++i) total *= shape[i];
    if (total == 0 || ndim == 0) {
        p.kind = NormKind::Empty;
        return p;
    }
    // contiguous output strides
    int64_t ostr[kMaxRank];
    {
        int64_t s = 1;
        for (int i = ndim - 1; i >= 0; --i) {
            ostr[i] = s;
            s *= shape[i];
        }
    }
    bool is_norm[kMaxRank] = {};
    if (n_norm_dims > 0)
        for (int i = ndim - n_norm_dims; i < ndim; ++i) is_norm[i] = true;
    else
        is_norm[axis] = true;

    // Row dims: merged only where input AND output are both one dense run.
    p.rows = 1;
    for (int i = 0; i < ndim; ++i) {
        if (is_norm[i]) continue;
        p.rows *= shape[i];
        if (shape[i] == 1) continue;
        int n = p.kept_in.n;
        if (n > 0 && p.kept_in.stride[n - 1] == strides[i] * shape[i] &&
            p.kept_out.stride[n - 1] == ostr[i] * shape[i]) {
            p.kept_in.size[n - 1] *= shape[i];
            p.kept_in.stride[n - 1] = strides[i];
            p.kept_out.size[n - 1] *= shape[i];
            p.kept_out.stride[n - 1] = ostr[i];
        } else {
            if (n == kMaxDims)
                fail(HPT_ERR_SHAPE, "view has more than %d non-mergeable row dims", kMaxDims);
            p.kept_in.size[n] = p.kept_out.size[n] = shape[i];
            p.kept_in.stride[n] = strides[i];
            p.kept_out.stride[n] = ostr[i];
            p.kept_in.n = p.kept_out.n = n + 1;
        }
    }
    // Normalised dims keep their logical order (gamma/beta and the output index by it).
    p.cols = 1;
    for (int i = 0; i < ndim; ++i) {
        if (!is_norm[i]) continue;
        p.cols *= shape[i];
        push_merged(p.norm_in, shape[i], strides[i]);
    }
    // Output stride along the (flattened) normalised index.
    p.out_axis_stride = 1;
    if (n_norm_dims <= 0) p.out_axis_stride = ostr[axis];
    if (p.cols == 1) {
        // one element per row: still a legal call. The axis has no extent, so neither of its strides
        // matters: say 1 and the row plans (one lane per "row") take it, whatever the axis was.
        p.norm_in.n = 1;
        p.norm_in.size[0] = 1;
        p.norm_in.stride[0] = 1;
        p.out_axis_stride = 1;
    }

    const int64_t sa = p.norm_in.n == 1 ? p.norm_in.stride[0] : 0;  // input stride along the row
    const int max_vec = (int)(16 / elem_size);

    // default: one group of lanes per row, striding along the row
    p.kind = NormKind::Generic;
    p.vec = 1;
    p.tpr = (int)std::min<int64_t>(1024, pow2_ceil((p.cols + 3) / 4));
    if (p.tpr > 64 && p.tpr < 256) p.tpr = 256;
    p.rpb = std::max(1, 256 / p.tpr);

    if (p.norm_in.n == 1 && p.out_axis_stride == 1) {
        // rows are contiguous in the output
        // input contiguous along the rows, output along the axis (a transposed view):
        // statistics pass + register-tile transpose, when 128-bit access is legal both ways
        const int nk = p.kept_in.n;
        const int v = max_vec;
        bool transposed = sa > 1 && nk >= 1 && nk <= 2 && p.kept_in.stride[nk - 1] == 1 && v > 1 &&
                          p.kept_in.size[nk - 1] % v == 0 && p.cols % v == 0 && sa % v == 0 &&
                          (nk == 1 || (p.kept_in.stride[0] % v == 0 && p.kept_in.size[0] <= 65535)) &&
                          ((uintptr_t)in_data % 16) == 0 && ((uintptr_t)out_data % 16) == 0 &&
                          p.kept_in.size[nk - 1] <= (1 << 30) && p.cols <= (1 << 30) &&  // 32-bit positions
                          p.kept_in.size[nk - 1] >= 8 * v && p.cols >= 8 * v;
        if (transposed) {
            p.vec = v;
            {
                // Single pass when 16 vectors per thread hold (16 * rgN bytes of rows) x (all
                // columns): rgN lanes along the rows, 1024 / rgN thread columns of 16 columns
                // each. Prefer long row segments, but keep at least ~one workgroup per
                // compute unit; below 64-byte segments the three-pass form is used.
                const int64_t R = p.kept_in.size[nk - 1];
                const int64_t batch = nk > 1 ? p.kept_in.size[0] : 1;
                const int64_t cgroups = (p.cols + 15) / 16;
                int rgN = 16;
                while (rgN >= 4 && cgroups * rgN > 1024) rgN >>= 1;
                while (rgN > 8 && (R + rgN * v - 1) / (rgN * v) * batch < 256) rgN >>= 1;
                const int64_t blocks = rgN >= 4 ? (R + rgN * v - 1) / (rgN * v) * batch : 0;
                if (rgN >= 4 && blocks >= 128) {
                    p.kind = NormKind::TransposedTile;
                    p.tpr = rgN;
                    const int64_t cols_per_wave = 16 * (64 / rgN);
                    p.rpb = (int)((p.cols + cols_per_wave - 1) / cols_per_wave);
                    return p;
                }
            }
            p.kind = NormKind::Transposed;
            // statistics pass: a wavefront covers 64*v rows; enough column splits for
            // about 2048 wavefronts, each keeping at least 32 columns
            const int64_t R = p.kept_in.size[nk - 1];
            const int64_t batch = nk > 1 ? p.kept_in.size[0] : 1;
            const int64_t groups = (R + 64 * v - 1) / (64 * v) * batch;
            int64_t S = std::max<int64_t>(1, std::min<int64_t>(512 / groups, p.cols / 128));
            p.tsplit = (int)std::min<int64_t>(S, 64);
            p.tpr = 4;  // wavefronts per workgroup of the statistics pass
            p.scratch_bytes = (size_t)p.rows * p.tsplit * 16 + (size_t)p.rows * 3 * 8;
            return p;
        }
        if (sa >= 1 && sa <= 4) {
            // vector width: input and output must both allow it
            int v = 1;
            if (sa == 1) {
                Dims none;
                int vi = legal_vec(in_data, elem_size, p.cols, p.kept_in, none, 0, 0);
                int vo = legal_vec(out_data, elem_size, p.cols, p.kept_out, none, 0, 0);
                v = std::min(std::min(vi, vo), max_vec);
            } else if (sa == 2 && max_vec >= 2) {
                // every second element: load full vectors, keep the even positions
                Dims none;
                const int uv = max_vec / 2;
                int vi = legal_vec(in_data, elem_size, p.cols * 2, p.kept_in, none, 0, 0);
                bool out_ok = ((uintptr_t)out_data % (uv * elem_size)) == 0 && p.cols % uv == 0;
                if (vi == max_vec && out_ok) {
                    v = max_vec;
                    p.sstride = 2;
                }
            }
            p.vec = v;
            // Rows that start off 16-byte boundaries (odd row lengths): the row kernels can still move
            // aligned vectors and mask the two ends of a row, provided input and output rows are
            // misaligned by the same amount: equal bases and row pitches modulo 16 bytes.
            // (few, very long rows are shared among workgroups below, element by element). Measured: the
            // register kernel gains from this between about 16 and 2048 vectors per row (f32 [130561, 257]
            // softmax 3.5 -> 4.9 TB/s, [8190, 4097] 3.1 -> 4.1); shorter rows are mostly row ends and stay
            // element-wise, longer ones stream (two sweeps) at the same speed.
            if (sa == 1 && v == 1 && max_vec > 1 && p.cols >= 16 * max_vec && !(p.rows <= 128 && p.cols >= 16384)) {
                bool same = (((uintptr_t)in_data ^ (uintptr_t)out_data) & 15) == 0 && ((uintptr_t)in_data % elem_size) == 0;
                for (int i = 0; i < p.kept_in.n; ++i)
                    if (((p.kept_in.stride[i] - p.kept_out.stride[i]) * (int64_t)elem_size) % 16 != 0) same = false;
                const int64_t nvs = (p.cols + 2 * (max_vec - 1)) / max_vec;
                // (two-byte layernorm keeps two vectors per thread, so its rows stay in registers up to 1024
                // vectors, 512 threads; f16 [8190, 4097] 1.9 -> 2.2 TB/s, [5461, 6145] 1.9 -> 2.8 against streaming)
                // Softmax rows beyond the register kernel's 2048 shifted vectors stay on chip in registers and
                // LDS (row_lds_kernel, whose vector grid starts on the 128-byte line that holds the row's first
                // element) up to 122846 four-byte or 196545 two-byte elements; they streamed before (two reads).
                // Measured (TB/s): f32 [4096, 30522] 3.5 -> 5.55, [2048, 50257] 4.45 -> 5.3, [1024, 100277] 3.7 -> 4.55;
                // f16 [8192, 32001] 4.0 -> 5.55, [4096, 50257] 4.35 -> 5.2, [2048, 98001] 4.2 -> 4.9.
                if (same && n_norm_dims <= 0 && nvs > 2048 && (elem_size == 2 || elem_size == 4) &&
                    lds_row_shape(p, (p.cols + 128 / (int64_t)elem_size + max_vec - 2) / max_vec, elem_size, true)) {
                    p.vec = max_vec;
                    p.shift = 1;
                    return p;
                }
                if (same && nvs > ((n_norm_dims > 0 && elem_size == 2) ? 1024 : 2048)) {
                    p.kind = NormKind::RowStream;
                    p.vec = max_vec;
                    p.shift = 1;
                    p.tpr = p.cols >= 4096 * max_vec ? 1024 : 256;
                    p.rpb = 1;
                    return p;
                }
                if (same) {
                    v = max_vec;
                    p.vec = v;
                    p.shift = 1;
                }
            }
            // vector loads per row (shifted rows: one more than the row's own length needs)
            int64_t nv = p.shift ? (p.cols + 2 * (v - 1)) / v : p.cols / (v / p.sstride);
            // Few, very long contiguous rows: share each row among workgroups. (One workgroup per
            // row would leave a chip of 256 compute units mostly idle.)
            if (sa == 1 && !p.shift && p.rows <= 128 && p.cols >= 16384 && p.cols % v == 0) {
                if (v == 1 && max_vec > 1 && ((uintptr_t)in_data % elem_size) == 0 && ((uintptr_t)out_data % elem_size) == 0) {
                    // rows off the 16-byte grid: unaligned vectors, the last one from the row's end backwards
                    v = max_vec;
                    p.vec = v;
                    p.shift = 1;
                }
                const int64_t nvec = (p.cols + v - 1) / v;
                int64_t S = std::min<int64_t>(512, std::max<int64_t>(1, 1024 / p.rows));
                S = std::min<int64_t>(S, std::max<int64_t>(1, nvec / 1024));  // at least 4 vectors per thread
                if (S >= 2) {
                    p.kind = NormKind::RowSplit;
                    p.tsplit = (int)S;
                    p.scratch_bytes = (size_t)p.rows * S * 16;
                    return p;
                }
                if (p.shift) {  // not worth splitting: back to element-wise rows
                    p.shift = 0;
                    p.vec = v = 1;
                }
            }
            // A row fits the registers of a workgroup up to 8 vectors per thread; layernorm also keeps
            // gamma and beta there (the eight-vector form spills), so it stops at four and streams
            // longer rows (two sweeps; gamma / beta as vectors).
            // Two-byte types hold eight elements per vector: with gamma and beta beside the row, sixteen
            // elements per thread is what fits 128 registers, i.e. two vectors (four of a stride-2 row).
            bool ln_half = n_norm_dims > 0 && v > 1 && elem_size == 2;
            // Two-byte layernorm rows of 640 ... 16384 elements: gamma / beta go to LDS (at most 64 KiB)
            // and the row takes three or four vectors per thread like any other. Measured, f16 (TB/s): [6553, 5120]
            // 3.5 -> 4.6, [4096, 8192] 4.7 -> 5.0, [2730, 12288] 3.2 -> 4.6, [2048, 16384] 3.8 -> 4.6; [65536, 1024]
            // 5.0 -> 5.4, [32768, 2048] 4.6 -> 5.3, [74898, 896] 4.5 -> 5.2, [104857, 640] 4.5 -> 4.9 (shorter rows lose:
            // [131072, 512] 4.9 -> 4.5).
            if (ln_half && p.sstride == 1 && !p.shift && nv * v >= 640 && nv * v <= 16384) {
                p.gb_lds = 1;
                ln_half = false;
            }
            const int64_t per = ln_half ? 2 * p.sstride : 4;
            const int64_t reg_limit = ln_half ? 1024 * per : (n_norm_dims > 0 && v > 1) ? 4096 : 8192;
            // Softmax rows beyond eight vectors per thread of a four-byte type (four of a two-byte type) stay on
            // chip in registers and LDS, one read instead of the streaming kernel's two: row_lds_kernel, up to
            // 131072 four-byte or 196608 two-byte elements. Two-byte rows of 98305 ... 131072 elements keep the
            // raw row in the registers of 1024 threads (sixteen vectors each), which measured faster there.
            // (Layernorm in such a kernel, with gamma / beta from L2 in the last sweep, spilled 60 to 130
            // registers and ran at 1.6-3.3 TB/s: such rows stream, at 3.0-3.4.)
            // Measured (TB/s; before: 1024 threads with 8 + 8 vectors staged through registers, the raw-row
            // kernel, or streaming): f32 [640, 50304] 4.35 -> 5.05, [2048, 50304] 5.05 -> 5.35, [2048, 40960]
            // 4.9 -> 5.35, [1024, 128256] 3.75 -> 4.7; f16 [4096, 50304] 4.75 -> 5.55, [4096, 65536] 5.0 -> 5.6,
            // [2048, 98304] 4.45 -> 5.1, [2048, 151936] 4.25 -> 4.55.
            if (n_norm_dims <= 0 && v == max_vec && p.sstride == 1 && !p.shift) {
                const bool raw16 = elem_size == 2 && nv > 12288 && nv <= 16384;
                if (raw16) {
                    p.kind = NormKind::RowReg;
                    p.raw_rows = 1;
                    p.tpr = 1024;
                    p.rpb = 1;
                    p.nchunk = 16;
                    return p;
                }
                // (the causal softmax has no such kernel: its rows stay with the register kernel while they fit)
                if ((elem_size == 4 ? nv > 8192 : elem_size == 2 && nv > 4096) && !(fused && nv <= reg_limit) &&
                    lds_row_shape(p, nv, elem_size, false))
                    return p;
            }
            // Layernorm rows beyond that (up to 32768 four-byte, 49152 two-byte or 16384 eight-byte elements) still fit
            // the registers of 512 or 1024 threads when gamma / beta do not sit beside them: those are read again for
            // every row, vector by vector in the last sweep, from L2. One read of the row instead of the streaming
            // kernel's two. Measured (% of the HBM peak, streaming -> this): f32 [1771, 18944] 39 -> 60, [1310, 25600]
            // 37 -> 57, [1024, 32768] 43 -> 62; f16 [1771, 18944] 27 -> 55, [1310, 25600] 28 -> 43, [1024, 32768] 33 -> 50.
            // (Two-byte rows of seven or eight vectors per thread spill. Where the forms above exist they are as fast
            // or faster: f32 [4096, 8192] 67.5 against 68, [2730, 12288] 68 against 65; f16 [4096, 8192] 59 against 53.)
            if (n_norm_dims > 0 && v == max_vec && v > 1 && p.sstride == 1 && !p.shift && !p.gb_lds && nv > reg_limit) {
                int t = 1024;
                if (elem_size == 2 && nv <= 512 * 5) t = 512;  // f16 [1771, 18944]: 512 x 5 55 %, 1024 x 3 45 %
                const int64_t c = (nv + t - 1) / t;
                // (layernorm(x + residual) holds the residual's vectors beside the row's: fewer fit before it spills)
                if (c <= (fused ? (elem_size == 2 ? 4 : 6) : (elem_size == 2 ? 6 : 8))) {
                    p.kind = NormKind::RowReg;
                    p.gb_lds = 2;
                    p.tpr = t;
                    p.nchunk = (int)c;
                    p.rpb = 1;
                    return p;
                }
            }
            if (nv <= reg_limit) {
                p.kind = NormKind::RowReg;
                // Short rows laid back to back: the plain kinds move whole 16 KiB tiles through LDS
                // (aligned vectors both ways whatever the row length); the fused kinds keep the
                // register plan made below.
                // Measured (TB/s, registers -> tile): f32 softmax [N, 8] 4.0 -> 5.9, [N, 33] 3.5 -> 5.5,
                // [N, 100] 4.0 -> 5.7, [N, 197] 4.5 -> 5.4; f32 layernorm [N, 33] 3.3 -> 5.1, [N, 100]
                // 3.3 -> 5.4; f16 softmax [N, 33] 2.1 -> 4.0, [N, 64] 2.1 -> 4.8. Rows of whole vectors
                // from 512 bytes on (and two-byte layernorm rows of whole vectors) are as fast or faster
                // from registers.
                const int64_t row_bytes = p.cols * (int64_t)elem_size;
                const bool whole = p.cols % max_vec == 0;
                const bool gains = whole ? (row_bytes >= 32 && row_bytes < 512 && !(elem_size == 2 && n_norm_dims > 0)) : true;
                if (sa == 1 && max_vec > 1 && gains && p.kept_in.n == 1 && p.kept_in.stride[0] == p.cols &&
                    (((uintptr_t)in_data | (uintptr_t)out_data) & 15) == 0 && p.cols <= 512 &&
                    p.rows * row_bytes >= (4ll << 20)) {
                    int64_t rows = (16 << 10) / (p.cols * (int64_t)elem_size);
                    rows -= rows % max_vec;
                    if (rows >= max_vec) p.tile_rows = (int)rows;
                }
                // about four 128-bit vectors per thread; rows that only allow single elements
                // take eight per thread (fewer, busier threads: a 257-element row stays in one
                // wavefront instead of four that meet in LDS)
                p.tpr = (int)std::min<int64_t>(1024, v > 1 ? pow2_ceil((nv + per - 1) / per) : pow2_ceil((nv + 7) / 8));
                if (p.tpr > 64 && p.tpr < 256 && !(ln_half && p.tpr == 128)) p.tpr = 256;
                // A row just over a power of two (4097: 1026 vectors) would take twice the threads with half of
                // them idle: softmax (no gamma / beta beside the row) of 4-byte types takes half the threads and five
                // vectors each. Measured (TB/s): f32 [8190, 4097] 4.6 -> 5.1, [8192, 4100] 4.6 -> 5.7, [4096, 8200]
                // 4.1 -> 4.9, [4000, 10000] 4.7 -> 5.1; f16 [8192, 8200] loses (4.7 -> 3.0: eight widened vectors spill).
                if (n_norm_dims <= 0 && v > 1 && elem_size >= 4 && p.tpr >= 512 && nv <= (p.tpr / 2) * 5) p.tpr /= 2;
                int64_t nc = (nv + p.tpr - 1) / p.tpr;
                p.nchunk = (int)std::max<int64_t>(1, pow2_ceil(nc));
                // Threads per row and vectors per thread are powers of two so far, which leaves a quarter
                // to a third of the lanes idle on rows of 3, 5, 6 or 7 times a power of two - the hidden
                // sizes 768, 1536, 2560, 3072, 5120, 6144, 12288. Aligned rows of whole vectors may take 3
                // (any type) or 5, 6, 7 (4- and 8-byte softmax; layernorm up to 6) vectors per thread: the
                // fewest slots win; among equals, rows of up to 256 threads (layernorm: 512) with the fewest
                // vectors per thread, else the fewest threads. Measured, TB/s: f32 softmax [21845, 1536]
                // 256 x 2 4.7 -> 128 x 3 6.0, [5461, 6144] 512 x 4 4.8 -> 256 x 6 5.8, [2730, 12288] 4.3 -> 5.2;
                // f32 layernorm [13107, 2560] 256 x 4 4.5 -> 128 x 5 5.5, [6553, 5120] 4.7 -> 5.6 (256 x 5),
                // [10922, 3072] 4.9 -> 5.7 (256 x 3); f16 softmax [21845, 3072] 256 x 2 4.5 -> 128 x 3 5.9,
                // [13107, 5120] 4.7 -> 5.8 (256 x 3); f16 layernorm [87381, 768] 4.1 -> 5.0 (32 x 3), [43690, 1536]
                // 3.9 -> 4.9 (64 x 3). (Two-byte rows of five vectors or more per thread lose: layernorm spills.)
                // (gamma / beta in LDS: three or four vectors per thread. Five lose to three with twice the threads, idle
                // lanes and all - f16, % of the HBM peak: [29127, 1152] 58 -> 66.5, [13107, 2560] 58 -> 64, [6553, 5120]
                // 56 -> 62, [3640, 9216] 53 -> 58, [3276, 10240] 39 -> 61)
                // (Rows of odd length, covered by aligned vectors: softmax alike - f16 [116306, 577] 3.6 -> 4.1,
                // [44739, 1500] 4.2 -> 4.9, f32 [8190, 4097] 4.4 -> 5.3, [16000, 2051] 4.3 -> 5.5; layernorm, which
                // carries the masks and the unaligned gamma / beta besides, only up to what it had: more spills.)
                if (v == max_vec && v > 1 && p.sstride == 1 && !p.tile_rows) {
                    const int maxc = n_norm_dims > 0 && p.shift ? (elem_size == 2 ? 2 : 4)
                                                                : elem_size == 2 ? (ln_half ? 3 : 4)
                                                                : (n_norm_dims > 0 ? (fused ? 4 : 6) : 8);
                    // (layernorm(x + residual) holds the residual's vectors beside the row's: with five or six
                    // per thread it spills - f32 [2730, 12288] 3.1 TB/s)
                    const int pref_tpr = n_norm_dims > 0 ? 512 : 256;
                    // (gamma / beta in LDS: the form exists for three to five vectors per thread only)
                    int64_t best = p.gb_lds ? INT64_MAX : (int64_t)p.tpr * p.nchunk;
                    int bt = p.gb_lds ? 0 : p.tpr, bc = p.nchunk;
                    bool base_stands = !p.gb_lds;  // the shape chosen above is still the best one
                    for (int t = p.gb_lds ? 32 : 16; t <= 1024; t <<= 1) {
                        const int64_t c = std::max<int64_t>((nv + t - 1) / t, p.gb_lds ? 3 : 1);
                        if (c > maxc) continue;
                        const int64_t slots = t * c;
                        bool take = slots < best;
                        if (!take && bt && slots == best && t != bt) {
                            // equal: a row inside the preferred width beats one outside it; inside, the wider row
                            // (fewer vectors per thread) wins, outside, the narrower one (f32 softmax [4096, 8192]
                            // 512 x 4 5.3 -> 256 x 8 5.7 TB/s, [2048, 16384] 1024 x 4 4.8 -> 512 x 8 5.2). The shape
                            // chosen above only gives way when it lies outside the preferred width.
                            const bool in_t = t <= pref_tpr, in_b = bt <= pref_tpr;
                            take = in_t != in_b ? in_t : (in_t ? t > bt : t < bt);
                            if (base_stands && in_b) take = false;
                        }
                        if (take) {
                            best = slots;
                            bt = t;
                            bc = (int)c;
                            base_stands = false;
                        }
                    }
                    if (bt) {
                        p.tpr = bt;
                        p.nchunk = bc;
                    }
                    // Softmax rows beyond 2048 vectors that still leave a sixteenth of those slots idle (threads
                    // come in powers of two): row_lds_kernel's 256 threads take slots in steps of 256 vectors.
                    // Measured (TB/s): f32 [4096, 16388] 4.8 -> 5.15; f16 [8192, 16392] 4.2 -> 5.45. (Full rows
                    // gain nothing: f32 [4096, 32768] 5.55 -> 5.55, f16 [8192, 32768] 5.75 -> 5.35.)
                    if (n_norm_dims <= 0 && !fused && !p.shift && nv > (elem_size == 2 ? 1024 : 2048) && (elem_size == 2 || elem_size == 4) &&
                        (int64_t)p.tpr * p.nchunk - nv >= nv / 16 && lds_row_shape(p, nv, elem_size, false))
                        return p;
                }
                int block = std::max(256, p.tpr);
                p.rpb = block / p.tpr;
                // Layernorm workgroups walk the rows; how many of them is best depends on how many a compute unit
                // can hold. f32 rows of four vectors per thread (gamma and beta beside them: ~100 registers, four
                // workgroups of 256 threads per compute unit) do best with THREE per compute unit, rows of two vectors
                // with six. Measured, us (768 / 1024 / 1536 workgroups): [8192, 4096] 45.7 / 47.6 / 47.5, [32768, 1024]
                // 45.1 / 46.2 / 47.1, [65536, 512] 45.0 / 46.4 / 47.4; [16384, 2048] 52.9 / 47.5 / 46.3, [8192, 2048]
                // 29.1 / 26.2 / 25.2, [8192, 1536] 26.9 / 23.1 / 20.3. Two-byte rows prefetch their next row and stay at 1024.
                // Two-byte rows with gamma / beta in LDS, up to four vectors per thread: three times as many workgroups
                // as a compute unit holds at once, so that one that ends early is replaced (with 1024 a workgroup walks
                // 10 or 11 row pairs and the last step runs two thirds empty). Measured, us (1024 / 1536 / 3072 / all rows):
                // f16 [21845, 3072] 52.1 / 50.5 / 48.6 / 51.0, [16384, 4096] 50.7 / 54.3 / 48.6 / 51.3, [65536, 1024]
                // 49.0 / 49.9 / 47.3 / 46.4; rows of five vectors per thread do best with 1024 ([13107, 5120] 53.2 / 61.9 / 59.2 / 64.2).
                if (n_norm_dims > 0 && p.gb_lds && p.nchunk <= 4 && p.tpr < 512) p.max_blocks = 3072;
                if (n_norm_dims > 0 && elem_size == 4 && v > 1 && p.tpr <= 256) {
                    // (Few rows: with 1024 every workgroup of [1024, 4096] has one row instead of one or two -
                    // 9.7 -> 8.3 us; [1536, 4096] 13.1 -> 11.6, [3072, 4096] 20.9 -> 20.5, from 4096 rows on no difference.)
                    if (p.nchunk >= 4) p.max_blocks = (p.rows + p.rpb - 1) / p.rpb > 3072 ? 768 : 1024;
                    else if (p.nchunk == 2) p.max_blocks = 1536;
                }
            } else {
                p.kind = NormKind::RowStream;
                p.tpr = 1024;
                p.rpb = 1;
                if (p.sstride == 2) {  // the streaming kernel gathers stride-2 rows element by element
                    p.vec = 1;
                    p.sstride = 1;
                }
            }
            return p;
        }
    }
    if (p.norm_in.n == 1 && p.out_axis_stride > 1 && n_norm_dims <= 0) {
        // Softmax over an axis that is not the last: the inner kept dim is contiguous in the output.
        // When it is in the input too, three passes spread over the whole chip: partial statistics
        // (lanes along the inner dim, the axis dealt over wavefronts and workgroups), finalize, apply.
        const int nk = p.kept_in.n;
        // Small groups laid back to back (a contiguous [batch, cols, L] tensor with cols * L elements of at
        // most 2 KiB: softmax over 4 heads of 64, over the 2 of [N, 2, 3]): lanes along L would idle and a
        // lane per (batch, inner) pair reads single elements at a stride. A workgroup stages 16 KiB of whole
        // groups in LDS with aligned vectors, one lane per pair normalises its column there, and the
        // tile leaves as it came.
        if (nk == 2 && max_vec > 1 && p.cols >= 2 && sa == p.kept_in.size[1] && p.kept_in.stride[1] == 1 &&
            p.kept_out.stride[1] == 1 && p.kept_in.size[1] == p.out_axis_stride &&
            p.kept_in.stride[0] == p.cols * sa && p.kept_out.stride[0] == p.cols * sa &&
            p.cols * sa * (int64_t)elem_size <= 2048 && sa * (int64_t)elem_size < 512 && p.kept_in.size[0] >= 1024 &&
            p.rows * p.cols * (int64_t)elem_size >= (4ll << 20) && (((uintptr_t)in_data | (uintptr_t)out_data) & 15) == 0) {
            int64_t groups = (16 << 10) / (p.cols * sa * (int64_t)elem_size);
            groups -= groups % max_vec;  // tiles start on 16-byte boundaries
            if (groups >= max_vec) {
                p.kind = NormKind::Col;
                p.inner = p.out_axis_stride;
                p.group_tile = (int)groups;
                p.vec = max_vec;
                return p;
            }
        }
        // Slabs whose inner dim divides the vector (2 or 4 four-byte elements; 2, 4 or 8 two-byte ones; 2 of eight bytes):
        // the slab is a ROW of cols * L elements for the register row kernel, which keeps one maximum and one sum per
        // place in the vector - one read and one write, no round trip through LDS.
        // An inner dim of two vectors (8 four-byte heads, 16 two-byte ones) likewise, where the axis is too long for the
        // register columns (which are faster up to 1024: f32 [2048, 512, 16] 22.1 against 28.3 us; beyond, against the
        // slab and the flat walk, f32 [1000, 2048, 8] 60.0 -> 31.1): a thread's vectors all hold the same places, and
        // only threads two apart are folded together.
        if (nk == 2 && max_vec > 1 && p.cols > 64 && sa > 1 && sa == p.kept_in.size[1] &&
            (max_vec % sa == 0 || (sa == 2 * max_vec && p.cols > 1024) || ((sa == 3 || sa == 5 || sa == 6 || sa == 7) && max_vec % sa != 0)) &&
            p.kept_in.stride[1] == 1 && p.kept_out.stride[1] == 1 && p.kept_in.size[1] == p.out_axis_stride &&
            p.kept_in.stride[0] == p.cols * sa && p.kept_out.stride[0] == p.cols * sa && (p.cols * sa) % max_vec == 0 &&
            p.cols * sa * (int64_t)elem_size <= (128 << 10) && p.kept_in.size[0] >= 256 &&
            p.rows * p.cols * (int64_t)elem_size >= (4ll << 20) && (((uintptr_t)in_data | (uintptr_t)out_data) & 15) == 0) {
            const int64_t shp[2] = {p.kept_in.size[0], p.cols * sa}, str[2] = {p.cols * sa, 1};
            NormPlan q = plan_normalize(in_data, out_data, shp, str, 2, 1, 0, elem_size, fused);
            if (q.kind == NormKind::RowReg && q.vec == max_vec && q.sstride == 1 && !q.shift && !q.tile_rows && !q.gb_lds &&
                !q.lds_rows && !q.raw_rows && q.tpr * max_vec >= sa) {
                if (max_vec % sa == 0 || sa == 2 * max_vec) {
                    q.interleave = (int)sa;
                    return q;
                }
                // An inner dim of 3, 5, 6 or 7: the largest multiple of it of a row's lanes take part, so that all of a
                // lane's vectors start at the same place modulo the inner dim; the lane keeps a (max, sum) per vector
                // place and the places are rotated into softmaxes, folded, and rotated back.
                const int64_t act = q.tpr / sa * sa, nvr = p.cols * sa / max_vec;
                const int64_t nc = (nvr + act - 1) / act;
                if (nc <= 8) {
                    q.interleave = -(int)sa;
                    q.nchunk = (int)nc;
                    return q;
                }
            }
        }
        // Mid-sized slabs with a very narrow inner dim ([B, 1000, 3], [B, 2048, 5]): one workgroup per slab through LDS.
        // (From 16 bytes of inner dim on the register kernel, which serves axes up to 1024, is as fast or faster:
        // f32 [2048, 1024, 8] 4.0 against 2.6 TB/s; beyond 1024 the alternative is the three-pass flat walk.
        // Four-byte inner dims of 5 ... 11 elements that are not whole vectors are the exception - the register kernel
        // loads them one or two elements at a time: f32, % of the HBM peak, registers -> slab: [4000, 512, 5] 29.5 -> 45.7,
        // [4000, 512, 7] 31.6 -> 46.8, [4000, 300, 10] 37.1 -> 45.3, [4000, 300, 11] 34.0 -> 43.9, [8000, 100, 6] 23.3 -> 33.1.
        // Two-byte inner dims of 7 ... 20 elements go either way by a few points and stay; f64 gains nothing.)
        if (nk == 2 && max_vec > 1 && p.cols > 64 && sa == p.kept_in.size[1] && p.kept_in.stride[1] == 1 &&
            p.kept_out.stride[1] == 1 && p.kept_in.size[1] == p.out_axis_stride &&
            p.kept_in.stride[0] == p.cols * sa && p.kept_out.stride[0] == p.cols * sa &&
            p.cols * sa * (int64_t)elem_size <= (64 << 10) && sa * (int64_t)elem_size <= ((p.cols > 1024 || (elem_size == 4 && sa % max_vec != 0)) ? (elem_size == 4 && sa % max_vec != 0 ? 48 : 32) : 12) &&
            p.kept_in.size[0] >= 256 &&
            p.rows * p.cols * (int64_t)elem_size >= (4ll << 20) && ((uintptr_t)in_data % elem_size) == 0 &&
            ((uintptr_t)out_data % elem_size) == 0) {
            p.kind = NormKind::Col;
            p.inner = p.out_axis_stride;
            // lanes per column: as many as 256 threads leave for each of the L columns, a wavefront at most
            int64_t tpc = 64;
            while (tpc > 1 && tpc * sa > 256) tpc >>= 1;
            p.slab_tile = (int)tpc;
            p.vec = max_vec;
            return p;
        }
        if (nk >= 1 && nk <= 2 && p.kept_in.stride[nk - 1] == 1 && p.kept_out.stride[nk - 1] == 1 &&
            p.kept_in.size[nk - 1] == p.out_axis_stride && p.kept_in.size[nk - 1] <= (1 << 30) && p.cols <= (1 << 30) &&
            (nk == 1 || p.kept_in.size[0] <= 65535)) {
            const int64_t L = p.kept_in.size[nk - 1];
            const int64_t batch = nk > 1 ? p.kept_in.size[0] : 1;
            // A SHORT axis (softmax over the channels of [B, 21, H, W]): a thread keeps the whole axis of
            // its inner positions in registers, up to 64 registers of raw values: one read, one write.
            // The widest vector that the axis length leaves room for and the layout allows is taken.
            if (p.cols <= 1024 && p.cols > 1) {
                // (two-byte types: vectors of at least 8 bytes, or the loads are too many and too small)
                // (... unless the axis is so short that one thread holds it anyway)
                // (... or the inner dim so narrow that the alternative, lanes along it, would leave most idle:
                // f16 [4097, 12, 96, 5] over axis 2, 0.4 -> 1.3 TB/s)
                for (int ev = max_vec; ev >= ((elem_size == 2 && p.cols > 16 && L >= 64) ? 4 : 1); ev /= 2) {
                    const int64_t regs = std::max<int64_t>(1, ev * (int64_t)elem_size / 4);
                    int64_t nc_max = std::min<int64_t>(64, 64 / regs);
                    const size_t vb = (size_t)ev * elem_size;
                    // thread rows that share an inner position when the axis is longer than one thread holds
                    int64_t ty = pow2_ceil((p.cols + nc_max - 1) / nc_max);
                    // A four-byte axis of 257 ... 512 elements fits sixteen thread rows only as 8-byte pieces, i.e.
                    // 128-byte segments of each inner row per workgroup, fetched by sixteen workgroups on eight XCDs at
                    // different moments. With 128 registers of raw values per thread instead of 64 the pieces are whole
                    // vectors and the segments 256 bytes (f32 [512, 512, 512] over axis 0 or 1: 4.8 TB/s before).
                    if (ty > 16 && elem_size == 4 && ev == 4 && p.cols <= 512 && L % 64 == 0) {
                        nc_max = 32;
                        ty = 16;
                    }
                    // Likewise 129 ... 256 elements: eight thread rows of 128 registers read 512-byte segments where sixteen
                    // of 64 read 256-byte ones. f32 [256, 256, 256] over axis 0 / 1, five processes each, us: 26.3-29.1 /
                    // 23.6-28.9 (which end depends on where the allocator put the buffers) -> 25.2-25.7 / 25.2-26.9.
                    // (65 ... 128 elements the same way, four thread rows, lose: C3 [64, 128, 56, 56] over the channels 41.3 -> 44.6 us)
                    if (ty == 16 && nc_max == 16 && elem_size == 4 && ev == 4 && p.cols > 128 && L % 128 == 0) {
                        nc_max = 32;
                        ty = 8;
                    }
                    // enough threads to fill the chip: inner positions x thread rows
                    if (!(ty <= 16 && p.rows / ev * ty >= 8 * 1024)) continue;
                    // (a long axis of two-byte elements that only fits with sixteen thread rows of 4-byte pieces: the
                    // three-pass flat walk is faster, f16 [512, 768, 60] 1.3 -> 2.1 TB/s, [768, 1024, 33] 1.0 -> 2.3;
                    // f32 single elements are not: [2048, 1024, 8] 4.0 against 2.3)
                    if (ty == 16 && elem_size == 2 && ev <= 2 && sa == L && L <= 1024 * max_vec &&
                        batch * p.cols * L * (int64_t)elem_size >= (8ll << 20))
                        continue;
                    if (L % ev == 0 && sa % ev == 0 && (nk == 1 || p.kept_in.stride[0] % ev == 0) &&
                        (p.cols * L) % ev == 0 && ((uintptr_t)in_data % vb) == 0 && ((uintptr_t)out_data % vb) == 0) {
                        p.kind = NormKind::ColReg;
                        p.vec = ev;
                        p.nchunk = (int)nc_max;
                        p.tpr = (int)ty;
                        return p;
                    }
                    // an inner dim that is not whole, aligned vectors of this width (odd L, odd strides): the
                    // same vectors unaligned beat narrower aligned ones
                    if (ev > 1 && L >= 8 * ev && ((uintptr_t)in_data % elem_size) == 0 && ((uintptr_t)out_data % elem_size) == 0) {
                        p.kind = NormKind::ColReg;
                        p.vec = ev;
                        p.shift = 1;
                        p.nchunk = (int)nc_max;
                        p.tpr = (int)ty;
                        return p;
                    }
                }
            }
            int v = max_vec;
            const bool vec_ok = v > 1 && L % v == 0 && sa % v == 0 && (nk == 1 || p.kept_in.stride[0] % v == 0) &&
                                ((uintptr_t)in_data % 16) == 0 && ((uintptr_t)out_data % 16) == 0;
            if (!vec_ok) v = 1;
            p.kind = NormKind::ColSplit;
            p.vec = v;
            // A narrow inner dim (or one that is not whole vectors) leaves most lanes idle: walk the
            // contiguous [cols, L] slab as a flat array of aligned vectors instead.
            if (max_vec > 1 && (!vec_ok || L <= 1024 * max_vec) && sa == L && ((uintptr_t)in_data % elem_size) == 0 &&
                ((uintptr_t)out_data % elem_size) == 0 && batch * p.cols * L * (int64_t)elem_size >= (8ll << 20)) {
                // (slabs that start off 16-byte boundaries take the same vectors unaligned: `shift`)
                const bool aligned = ((uintptr_t)in_data % 16) == 0 && ((uintptr_t)out_data % 16) == 0 &&
                                     (batch == 1 || (p.kept_in.stride[0] % max_vec == 0 && (p.cols * L) % max_vec == 0));
                int64_t g = L, b = max_vec;
                while (b) { int64_t t = g % b; g = b; b = t; }
                const int64_t lp = L / g;  // threads per period
                int64_t tmax = std::min<int64_t>(1024, (64 << 10) / (max_vec * (elem_size >= 4 ? 16 : 8)));
                // (each batch slab must be worth at least two periods of the walk: small slabs, of which there
                // are many, take fewer threads each)
                tmax = std::min(tmax, p.cols * L / (2 * max_vec));
                if (lp <= tmax && tmax >= 64) {
                    p.flat_t = (int)(lp * (tmax / lp));
                    p.vec = max_vec;
                    p.shift = aligned ? 0 : 1;
                    const int64_t periods = p.cols * L / ((int64_t)p.flat_t * max_vec);
                    p.tsplit = (int)std::max<int64_t>(1, std::min<int64_t>(periods / 4, std::max<int64_t>(1, 256 / batch)));
                    p.scratch_bytes = (size_t)p.rows * p.tsplit * 16 + (size_t)p.rows * 3 * 8;
                    return p;
                }
            }
            // Inner rows that are not whole, aligned vectors and too wide for the flat walk (an odd inner length of
            // thousands): a lane still takes a vector's worth of neighbouring inner positions, unaligned, instead of one
            // element (a wavefront then reads 1 KiB per axis position, not 128 or 256 bytes). Below a wavefront of vectors
            // the single elements already cover the inner row in one step.
            if (!vec_ok && max_vec > 1 && L >= 64 * max_vec && ((uintptr_t)in_data % elem_size) == 0 &&
                ((uintptr_t)out_data % elem_size) == 0) {
                v = max_vec;
                p.vec = v;
                p.shift = 1;
            }
            const int64_t groups = (L + 64 * v - 1) / (64 * v) * batch;
            int64_t S = std::max<int64_t>(1, std::min<int64_t>(512 / groups, p.cols / 32));
            p.tsplit = (int)std::min<int64_t>(S, 64);
            p.tpr = 4;  // wavefronts per workgroup of the statistics pass
            p.scratch_bytes = (size_t)p.rows * p.tsplit * 16 + (size_t)p.rows * 3 * 8;
            return p;
        }
        p.kind = NormKind::Col;
        p.inner = p.out_axis_stride;
        if (p.rows >= 1024) {
            // every lane owns one row; neighbouring lanes are neighbours in memory
            p.tpr = 1;
            p.rpb = 256;
        }
        return p;
    }
    return p;
}

void demote_to_generic(NormPlan& p) {
    p.kind = NormKind::Generic;
    p.raw_rows = 0;
    p.lds_rows = 0;
    p.group_tile = 0;
    p.slab_tile = 0;
    p.gb_lds = 0;
    p.tile_rows = 0;
    p.flat_t = 0;
    p.vec = 1;
    p.shift = 0;
    p.sstride = 1;
    p.nchunk = 1;
    p.scratch_bytes = 0;
    p.tpr = (int)std::min<int64_t>(1024, pow2_ceil((p.cols + 3) / 4));
    if (p.tpr > 64 && p.tpr < 256) p.tpr = 256;
    p.rpb = std::max(1, 256 / p.tpr);
}

void restrict_to_row_stream(NormPlan& p) {
    if (p.kind == NormKind::Empty) return;
    const bool rows_on_grid = (p.kind == NormKind::RowReg || p.kind == NormKind::RowStream) && p.vec > 1 &&
                              p.sstride == 1 && !p.shift && p.norm_in.n == 1 && p.norm_in.stride[0] == 1 &&
                              p.out_axis_stride == 1;
    const int vec = rows_on_grid ? p.vec : 1;
    demote_to_generic(p);
    if (!rows_on_grid) return;
    p.kind = NormKind::RowStream;
    p.vec = vec;
    p.tpr = (int)std::min<int64_t>(1024, pow2_ceil((p.cols / vec + 3) / 4));
    if (p.tpr > 64 && p.tpr < 256) p.tpr = 256;
    p.rpb = std::max(1, 256 / p.tpr);
}

std::string describe(const NormPlan& p) {
    static const char* names[] = {"empty", "rowreg", "rowstream", "rowsplit", "col", "col-split", "transposed", "transposed-tile", "col-reg", "generic"};
    char buf[256];
    snprintf(buf, sizeof buf, "%s%s%s rows=%lld cols=%lld vec=%d tpr=%d rpb=%d nchunk=%d ostride=%lld ",
             names[(int)p.kind], p.sstride == 2 ? "-step2" : (p.flat_t ? (p.shift ? "-flat-unaligned" : "-flat") : (p.shift ? ((p.kind == NormKind::RowSplit || p.kind == NormKind::ColReg || p.kind == NormKind::ColSplit) ? "-unaligned" : (p.lds_rows ? "-lds-shift" : "-shift")) : (p.gb_lds == 2 ? "-l2gb" : p.gb_lds ? "-ldsgb" : (p.raw_rows ? "-raw" : (p.lds_rows ? "-lds" : ""))))), p.tile_rows ? "+tile" : (p.interleave > 1 ? "-interleaved" : p.interleave < 0 ? "-modular" : p.group_tile ? "-group-tile" : (p.slab_tile ? "-slab" : "")), (long long)p.rows, (long long)p.cols, p.vec, p.tpr, p.rpb,
             p.nchunk, (long long)p.out_axis_stride);
    std::string s = buf;
    if (p.kind == NormKind::RowReg) s += "max_blocks=" + std::to_string(p.max_blocks) + " ";  // (layernorm walks its rows)
    describe_dims(s, "rows_in", p.kept_in);
    s += " ";
    describe_dims(s, "norm_in", p.norm_in);
    return s;
}

// ---- elementwise ------------------------------------------------------------------

EwPlan plan_elementwise(const void* out_data, const int64_t* shape, int ndim, int nin, const void* const* in_data,
                        const int64_t* const* in_strides, size_t elem_size, bool allow_transpose) {
    EwPlan p;
    p.nin = nin;
    p.total = 1;
    for (int i = 0; i < ndim; ++i) p.total *= shape[i];
    if (p.total == 0) return p;
    // coalesce: drop size-1 dims; merge dim i into i+1 when every operand (and the
    // contiguous output, which always can) steps over dim i+1 exactly once per step of i
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] == 1) continue;
        bool merge = p.n > 0;
        if (merge) {
            for (int k = 0; k < nin; ++k)
                if (p.stride[k][p.n - 1] != in_strides[k][i] * shape[i]) merge = false;
        }
        if (merge) {
            p.size[p.n - 1] *= shape[i];
            for (int k = 0; k < nin; ++k) p.stride[k][p.n - 1] = in_strides[k][i];
        } else {
            if (p.n == kMaxDims)
                fail(HPT_ERR_SHAPE, "elementwise: the view does not coalesce to %d dims or fewer", kMaxDims);
            p.size[p.n] = shape[i];
            for (int k = 0; k < nin; ++k) p.stride[k][p.n] = in_strides[k][i];
            ++p.n;
        }
    }
    if (p.n == 0) {  // a single element
        p.n = 1;
        p.size[0] = 1;
        for (int k = 0; k < nin; ++k) p.stride[k][0] = 1;
    }
    p.kind = EwKind::Inner;
    const int full = (int)(16 / elem_size);
    const int last = p.n - 1;
    auto aligned = [&](const void* ptr) { return ((uintptr_t)ptr % 16) == 0; };
    // vectors along the innermost dim: every operand is either contiguous there (stride 1,
    // with 16-byte aligned base and outer strides) or broadcast there (stride 0)
    bool vec_ok = full > 1 && p.size[last] % full == 0 && aligned(out_data);
    for (int k = 0; k < nin && vec_ok; ++k) {
        const int64_t s = p.stride[k][last];
        if (s == 1) {
            if (!aligned(in_data[k])) vec_ok = false;
            for (int i = 0; i < last; ++i)
                if (p.stride[k][i] % full != 0) vec_ok = false;
        } else if (s != 0) {
            vec_ok = false;
        }
    }
    if (vec_ok) {
        p.vec = full;
        return p;
    }
    // copy of a view whose innermost stride is 2: full vectors in, the even positions kept
    if (nin == 1 && full > 1 && p.stride[0][last] == 2 && p.size[last] % full == 0 && aligned(out_data) &&
        aligned(in_data[0])) {
        bool ok = true;
        for (int i = 0; i < last; ++i)
            if (p.stride[0][i] % full != 0) ok = false;
        if (ok) {
            p.vec = full;
            p.sstride = 2;
            return p;
        }
    }
    // copy of a view whose contiguous dim is not the innermost one: transpose in registers
    if (allow_transpose && nin == 1 && full > 1 && p.stride[0][last] != 1 && p.stride[0][last] != 0) {
        int t = -1;
        for (int i = 0; i < last; ++i)
            if (p.stride[0][i] == 1) t = i;
        if (t >= 0 && p.n <= 6) {
            bool ok = aligned(out_data) && aligned(in_data[0]) && p.size[last] % full == 0 && p.size[t] % full == 0 &&
                      p.size[last] >= 2 * full && p.size[t] >= 2 * full && p.size[last] <= (1 << 30) &&
                      p.size[t] <= (1 << 30);
            for (int i = 0; i < p.n; ++i)
                if (i != t && p.stride[0][i] % full != 0) ok = false;
            // the remaining dims ride on blockIdx.z
            int64_t others = 1;
            for (int i = 0; i < p.n; ++i)
                if (i != t && i != last) others *= p.size[i];
            if (ok && others <= 65535) {
                p.kind = EwKind::Transpose;
                p.vec = full;
                p.tdim = t;
                p.tmask = 1;
                p.tile_lds = p.size[last] >= 16 * full && p.size[t] >= 16 * full;
            }
        }
    }
    // binary op with an operand (or both) whose contiguous dim is not the innermost one (a + b.t()): whole
    // tiles of those operands are transposed through LDS; an operand in the output's own layout (or
    // broadcast along the innermost dim) is read as the result is written
    if (allow_transpose && nin == 2 && full > 1 && full <= 8 && p.n <= 6) {
        int mask = 0;
        for (int k = 0; k < 2; ++k)
            if (p.stride[k][last] != 1 && p.stride[k][last] != 0) mask |= 1 << k;
        int t = -1;
        for (int i = 0; i < last && mask; ++i) {
            bool all = true;
            for (int k = 0; k < 2; ++k)
                if ((mask >> k & 1) && p.stride[k][i] != 1) all = false;
            if (all) t = i;
        }
        if (t >= 0) {
            bool ok = aligned(out_data) && p.size[last] % full == 0 && p.size[t] % full == 0 && p.size[last] >= 16 * full &&
                      p.size[t] >= 16 * full && p.size[last] <= (1 << 30) && p.size[t] <= (1 << 30);
            for (int k = 0; k < 2 && ok; ++k) {
                const bool transposed = mask >> k & 1;
                if (!transposed && p.stride[k][last] == 0) continue;  // single elements, splat
                if (!aligned(in_data[k])) ok = false;
                for (int i = 0; i < p.n; ++i)
                    if (i != (transposed ? t : last) && p.stride[k][i] % full != 0) ok = false;
            }
            int64_t others = 1;
            for (int i = 0; i < p.n; ++i)
                if (i != t && i != last) others *= p.size[i];
            if (ok && others <= 65535) {
                p.kind = EwKind::Transpose;
                p.vec = full;
                p.tdim = t;
                p.tmask = mask;
                p.tile_lds = true;
            }
        }
    }
    return p;
}

std::string describe(const EwPlan& p) {
    static const char* names[] = {"empty", "inner", "transpose"};
    char buf[128];
    snprintf(buf, sizeof buf, "%s%s vec=%d total=%lld dims=[", names[(int)p.kind], p.sstride == 2 ? "-step2" : "", p.vec,
             (long long)p.total);
    std::string s = buf;
    for (int i = 0; i < p.n; ++i) {
        snprintf(buf, sizeof buf, "%s%lld:", i ? "," : "", (long long)p.size[i]);
        s += buf;
        for (int k = 0; k < p.nin; ++k) {
            snprintf(buf, sizeof buf, "%s%lld", k ? "/" : "", (long long)p.stride[k][i]);
            s += buf;
        }
    }
    s += "]";
    if (p.kind == EwKind::Transpose) {
        snprintf(buf, sizeof buf, " tdim=%d%s%s", p.tdim, p.nin == 2 ? (p.tmask == 3 ? " both" : p.tmask == 1 ? " lhs" : " rhs") : "",
                 p.tile_lds ? " lds" : "");
        s += buf;
    }
    return s;
}

}  // namespace hpt
