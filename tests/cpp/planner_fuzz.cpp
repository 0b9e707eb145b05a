// Host-only fuzz of the launch planners (layout.cpp), meant to be built with
// -fsanitize=address,undefined: random views (permuted, sliced, reversed, broadcast,
// offset by a few bytes) go through plan_reduce / plan_normalize / plan_elementwise and
// describe(); the plan that comes back must keep the element counts of the view and
// a launch shape the kernels can take. No GPU call is made.
//
// usage: planner_fuzz <iterations> <seed>
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "common.hpp"

using namespace hpt;

static std::mt19937_64 rng;
static int64_t uni(int64_t lo, int64_t hi) { return std::uniform_int_distribution<int64_t>(lo, hi)(rng); }

static const int64_t kSizes[] = {0, 1, 1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127,
                                 128, 255, 256, 257, 511, 512, 768, 1000, 1024, 1536, 2048, 2560, 3072,
                                 4096, 4097, 5120, 8192, 10000, 12288, 16384, 32768, 50257, 65536, 131072,
                                 1 << 20, (1 << 20) + 3, 1 << 24, (int64_t)1 << 31, ((int64_t)1 << 32) + 5};
static constexpr int kNSizes = sizeof kSizes / sizeof kSizes[0];

struct View {
    std::vector<int64_t> shape, strides;
    uintptr_t base = 0;
    int64_t total() const {
        int64_t t = 1;
        for (int64_t s : shape) t *= s;
        return t;
    }
};

// A view of at most `budget` elements: a contiguous parent, then permuted, sliced with
// steps of either sign, broadcast along some dims, the base moved off the 16-byte grid.
static View random_view(size_t elem, int64_t budget, bool allow_zero, bool allow_broadcast) {
    View v;
    const int ndim = (int)uni(1, uni(0, 3) ? 4 : 7);
    int64_t left = budget;
    for (int i = 0; i < ndim; ++i) {
        int64_t s;
        do s = kSizes[uni(allow_zero && uni(0, 30) == 0 ? 0 : 1, kNSizes - 1)];
        while (s > left);
        v.shape.push_back(s);
        if (s > 1) left /= s;
    }
    // parent sizes: slices keep every step-th element of a larger dim
    std::vector<int64_t> step(ndim, 1), psize(ndim);
    for (int i = 0; i < ndim; ++i) {
        if (uni(0, 4) == 0) step[i] = uni(0, 1) ? 2 : uni(-3, 5);
        if (step[i] == 0) step[i] = allow_broadcast ? 0 : 1;
        const int64_t a = step[i] < 0 ? -step[i] : step[i];
        psize[i] = a == 0 ? 1 : v.shape[i] * a + (uni(0, 3) == 0 ? uni(0, 9) : 0);
        if (psize[i] == 0) psize[i] = 1;
    }
    std::vector<int> perm(ndim);
    for (int i = 0; i < ndim; ++i) perm[i] = i;
    if (uni(0, 2) == 0)
        for (int i = ndim - 1; i > 0; --i) std::swap(perm[i], perm[uni(0, i)]);
    // perm[k] = the view dim stored k-th outermost in memory
    std::vector<int64_t> pstride(ndim);
    int64_t run = 1;
    for (int k = ndim - 1; k >= 0; --k) {
        pstride[perm[k]] = run;
        run *= psize[perm[k]];
    }
    v.strides.resize(ndim);
    for (int i = 0; i < ndim; ++i) v.strides[i] = pstride[i] * step[i];
    static const int offs[] = {0, 0, 0, 0, 16, 8, 4, 2, 1, 6, 12, 3};
    int64_t off = offs[uni(0, 11)];
    off -= off % (int64_t)elem;
    v.base = 0x7f0000000000ull + (uintptr_t)uni(0, 1 << 20) * 256 + (uintptr_t)off;
    return v;
}

static int failures = 0;
static long seen_transposed_binary = 0, seen_lds_rows = 0;
#define CHECK(cond, ...)                       \
    do {                                       \
        if (!(cond)) {                         \
            ++failures;                        \
            std::fprintf(stderr, "FAIL %s: ", #cond); \
            std::fprintf(stderr, __VA_ARGS__); \
            std::fprintf(stderr, "\n");        \
        }                                      \
    } while (0)

static bool pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

static std::string show(const View& v) {
    std::string s = "shape=[";
    for (int64_t x : v.shape) s += std::to_string(x) + ",";
    s += "] strides=[";
    for (int64_t x : v.strides) s += std::to_string(x) + ",";
    s += "] base%16=" + std::to_string(v.base % 16);
    return s;
}

static void fuzz_reduce() {
    static const size_t elems[] = {1, 2, 4, 8};
    const size_t elem = elems[uni(0, 3)];
    const size_t acc = uni(0, 3) == 0 ? 16 : (elem < 4 ? (uni(0, 1) ? 4 : 8) : (elem == 4 && uni(0, 1) ? 4 : 8));
    View v = random_view(elem, (int64_t)1 << 34, true, false);
    const int ndim = (int)v.shape.size();
    std::vector<int64_t> axes;
    for (int i = 0; i < ndim; ++i)
        if (uni(0, 1)) axes.push_back(i);
    if (axes.empty() && uni(0, 3)) axes.push_back(uni(0, ndim - 1));
    for (int i = (int)axes.size() - 1; i > 0; --i) std::swap(axes[i], axes[uni(0, i)]);
    try {
        ReducePlan p = plan_reduce((const void*)v.base, v.shape.data(), v.strides.data(), ndim, axes.data(),
                                   (int)axes.size(), elem, acc);
        const std::string d = describe(p);
        int64_t K = 1, R = 1;
        for (int i = 0; i < ndim; ++i) {
            bool red = false;
            for (int64_t a : axes) red |= a == i;
            (red ? R : K) *= v.shape[i];
        }
        if (p.kind == ReduceKind::Empty) {
            CHECK(K == 0, "%s", show(v).c_str());
            return;
        }
        CHECK(p.K == K, "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.kind == ReduceKind::Identity) {
            CHECK(R == 0, "%s", show(v).c_str());
            return;
        }
        CHECK(p.R == R, "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(p.kept.count() == K && p.red.count() == R, "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(pow2(p.vec) && (size_t)p.vec * elem <= 16, "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(p.split >= 1 && p.split_q >= 1 && p.split_i >= 1, "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(p.interleave >= 1, "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.interleave > 1)  // rows that are [R, interleave] slabs: whole aligned vectors, one workgroup per row
            CHECK(p.kind == ReduceKind::Row && p.lean && p.split == 1 && (size_t)p.vec * elem == 16 && p.vec % p.interleave == 0 &&
                      p.interleave <= 8 && p.K % p.interleave == 0 && (p.R * p.interleave) % p.vec == 0 && !p.ragged && !p.unaligned &&
                      p.sstride == 1 && !p.row_tile && p.kept.n == 2 && p.kept.size[1] == p.interleave && p.kept.stride[1] == 1 &&
                      p.kept.stride[0] == p.R * p.interleave && v.base % 16 == 0,
                  "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.mod_rows > 0)  // rows that are [R, L] slabs, L = 3, 5, 6, 7: 256-thread workgroups of whole rows
            CHECK(p.kind == ReduceKind::Row && p.split == 1 && (size_t)p.vec * elem == 16 && p.vec % p.mod_rows != 0 && p.mod_rows >= 3 &&
                      p.mod_rows <= 7 && p.K % p.mod_rows == 0 && p.tpr * p.rpb == 256 && p.tpr >= 64 && p.kept.n == 2 &&
                      p.kept.size[1] == p.mod_rows && p.kept.stride[1] == 1 && p.kept.stride[0] == p.R * p.mod_rows &&
                      p.red.n == 1 && p.red.stride[0] == p.mod_rows && p.R * p.mod_rows < (1ll << 30) && p.interleave == 1,
                  "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.kind == ReduceKind::Row) {
            CHECK(pow2(p.tpr) && p.rpb >= 1 && (int64_t)p.tpr * p.rpb <= 1024, "%s plan=%s", show(v).c_str(),
                  d.c_str());
            CHECK(p.split == p.split_q * p.split_i, "%s plan=%s", show(v).c_str(), d.c_str());
        } else {
            CHECK(p.bx >= 1 && p.by >= 1 && (int64_t)p.bx * p.by <= 1024, "%s plan=%s", show(v).c_str(), d.c_str());
            if (!p.flat_t && !p.group_tile && p.split > 1)
                CHECK(p.chunk >= 1 && (p.chunk * p.split >= R || p.flat_xb), "%s plan=%s", show(v).c_str(),
                      d.c_str());
        }
    } catch (const Error&) {
        // a view the planner refuses (too many dims after coalescing) is reported to the caller
    }
}

static void fuzz_normalize() {
    static const size_t elems[] = {2, 2, 4, 4, 8};
    const size_t elem = elems[uni(0, 4)];
    View v = random_view(elem, (int64_t)1 << 33, true, false);
    const int ndim = (int)v.shape.size();
    const bool layernorm = uni(0, 1);
    const int64_t axis = layernorm ? -1 : uni(0, ndim - 1);
    const int nd = layernorm ? (int)uni(1, ndim) : 0;
    // the output is a fresh contiguous tensor, now and then the input itself (in place)
    const uintptr_t out = uni(0, 5) == 0 ? v.base : 0x7e0000000000ull + (uintptr_t)uni(0, 1 << 20) * 256;
    try {
        NormPlan p = plan_normalize((const void*)v.base, (const void*)out, v.shape.data(), v.strides.data(), ndim,
                                    axis, nd, elem, layernorm && uni(0, 3) == 0);
        std::string d = describe(p);
        int64_t cols = 1;
        if (layernorm)
            for (int i = ndim - nd; i < ndim; ++i) cols *= v.shape[i];
        else
            cols = v.shape[axis];
        const int64_t total = v.total();
        if (p.kind == NormKind::Empty) {
            CHECK(total == 0, "%s", show(v).c_str());
            return;
        }
        // (interleaved rows: a row is a whole [axis, inner] slab, the inner dim a divisor of the full vector)
        const int64_t il = p.interleave < 0 ? -p.interleave : p.interleave;
        CHECK(il >= 1 && p.cols == cols * il && p.rows * p.cols == total, "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.interleave < 0)  // an inner dim of 3, 5, 6, 7: lanes in multiples of it hold the row
            CHECK(p.kind == hpt::NormKind::RowReg && (size_t)p.vec * elem == 16 && il >= 3 && il <= 7 && p.vec % il != 0 && !p.shift &&
                      p.sstride == 1 && !p.tile_rows && !p.gb_lds && !layernorm && p.cols % p.vec == 0 &&
                      p.cols / p.vec <= (int64_t)(p.tpr / il * il) * p.nchunk && p.nchunk <= 8,
                  "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.interleave > 1)
            CHECK(p.kind == hpt::NormKind::RowReg && (size_t)p.vec * elem == 16 && (p.vec % p.interleave == 0 || (p.interleave == 2 * p.vec && p.tpr >= 2)) && !p.shift && p.sstride == 1 &&
                      !p.tile_rows && !p.gb_lds && !layernorm && p.cols % p.vec == 0 && p.cols / p.vec <= (int64_t)p.tpr * p.nchunk && p.nchunk <= 8,
                  "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(pow2(p.vec) && (size_t)p.vec * elem <= 16, "%s plan=%s", show(v).c_str(), d.c_str());
        CHECK(p.tpr >= 1 && p.rpb >= 1 && p.nchunk >= 1 && p.max_blocks >= 1, "%s plan=%s", show(v).c_str(),
              d.c_str());
        if (p.kind == NormKind::RowReg && !p.lds_rows && !p.raw_rows) CHECK(p.nchunk <= 8, "%s plan=%s", show(v).c_str(), d.c_str());
        if (p.kind == NormKind::RowReg && !p.tile_rows && !p.lds_rows && !p.raw_rows) {
            CHECK(pow2(p.tpr) && (int64_t)p.tpr * p.rpb <= 1024, "%s plan=%s", show(v).c_str(), d.c_str());
            // the registers of a row's threads hold the whole row
            const int64_t slots = (int64_t)p.tpr * p.nchunk * p.vec;
            CHECK(slots >= cols * p.sstride || p.shift, "%s plan=%s", show(v).c_str(), d.c_str());
        }
        if (p.kind == NormKind::RowReg && p.lds_rows) {
            ++seen_lds_rows;
            // the register + LDS kernel's vector grid may start up to a 128-byte line before the row
            const int64_t line = 128 / (int64_t)elem;
            const int64_t grid = (cols + (p.shift ? line - 1 : 0) + p.vec - 1) / p.vec;
            CHECK((p.tpr == 256 || p.tpr == 512 || p.tpr == 1024) && p.rpb == 1 && grid <= (int64_t)p.tpr * p.nchunk && (size_t)p.vec * elem == 16,
                  "%s plan=%s", show(v).c_str(), d.c_str());
        }
        NormPlan g = p;
        demote_to_generic(g);
        d = describe(g);
        CHECK(g.rows == p.rows && g.cols == p.cols, "%s plan=%s", show(v).c_str(), d.c_str());
        NormPlan s = p;
        restrict_to_row_stream(s);
        d = describe(s);
        CHECK(s.rows == p.rows && s.cols == p.cols, "%s plan=%s", show(v).c_str(), d.c_str());
    } catch (const Error&) {
    }
}

static void fuzz_elementwise() {
    static const size_t elems[] = {1, 2, 4, 8};
    const size_t elem = elems[uni(0, 3)];
    const int nin = (int)uni(0, 2);
    View a = random_view(elem, (int64_t)1 << 33, true, true);
    const int ndim = (int)a.shape.size();
    View b = a;
    if (nin == 2) {
        // the second operand: contiguous over the same shape, with some dims broadcast
        int64_t run = 1;
        for (int i = ndim - 1; i >= 0; --i) {
            if (uni(0, 2) == 0 || a.shape[i] == 1) b.strides[i] = 0;
            else {
                b.strides[i] = run;
                run *= a.shape[i];
            }
        }
        b.base = 0x7d0000000000ull + (uintptr_t)uni(0, 64) * elem;
        if (uni(0, 2) == 0 && ndim >= 2) {  // the second operand contiguous along another dim than the last
            const int t = (int)uni(0, ndim - 2);
            int64_t run = a.shape[t];
            b.strides[t] = 1;
            for (int i = ndim - 1; i >= 0; --i) {
                if (i == t) continue;
                b.strides[i] = run;
                run *= a.shape[i];
            }
            if (uni(0, 1)) b.base -= b.base % 16;
        }
    }
    const void* in_data[2] = {(const void*)a.base, (const void*)b.base};
    const int64_t* in_strides[2] = {a.strides.data(), b.strides.data()};
    const uintptr_t out = 0x7c0000000000ull + (uintptr_t)uni(0, 1 << 20) * 256;
    try {
        EwPlan p = plan_elementwise((const void*)out, a.shape.data(), ndim, nin, in_data, in_strides, elem,
                                    nin >= 1 && uni(0, 3) != 0);
        const std::string d = describe(p);
        const int64_t total = a.total();
        if (p.kind == EwKind::Empty) {
            CHECK(total == 0, "%s", show(a).c_str());
            return;
        }
        int64_t t = 1;
        for (int i = 0; i < p.n; ++i) t *= p.size[i];
        CHECK(p.total == total && t == total, "%s plan=%s", show(a).c_str(), d.c_str());
        CHECK(p.n >= 1 && p.n <= kMaxDims && p.nin == nin, "%s plan=%s", show(a).c_str(), d.c_str());
        CHECK(pow2(p.vec) && (size_t)p.vec * elem <= 16, "%s plan=%s", show(a).c_str(), d.c_str());
        if (p.kind == EwKind::Transpose) {
            seen_transposed_binary += nin == 2;
            CHECK(p.tdim >= 0 && p.tdim < p.n - 1 && p.tmask >= 1 && p.tmask < (1 << nin), "%s plan=%s", show(a).c_str(),
                  d.c_str());
            for (int k = 0; k < nin; ++k) {
                // an operand is contiguous along the transposed dim, or along the innermost one (or broadcast there)
                const int64_t s_last = p.stride[k][p.n - 1];
                CHECK((p.tmask >> k & 1) ? p.stride[k][p.tdim] == 1 : (s_last == 1 || s_last == 0), "%s plan=%s",
                      show(a).c_str(), d.c_str());
            }
            CHECK(p.size[p.n - 1] % p.vec == 0 && p.size[p.tdim] % p.vec == 0, "%s plan=%s", show(a).c_str(), d.c_str());
        }
        if (p.kind == EwKind::Inner && p.vec > 1)
            CHECK(p.size[p.n - 1] % p.vec == 0, "%s plan=%s", show(a).c_str(), d.c_str());
    } catch (const Error&) {
    }
}

int main(int argc, char** argv) {
    const long iters = argc > 1 ? std::atol(argv[1]) : 20000;
    rng.seed(argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 1);
    for (long i = 0; i < iters; ++i) {
        fuzz_reduce();
        fuzz_normalize();
        fuzz_elementwise();
        if (failures > 20) break;
    }
    std::printf("planner_fuzz: %ld iterations, %d failures (%ld transposing binary plans, %ld register + LDS row plans)\n", iters,
                failures, seen_transposed_binary, seen_lds_rows);
    return failures ? 1 : 0;
}
