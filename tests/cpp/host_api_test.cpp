// Parity tests of the C++ host side (include/hpt_hip.hpp) on a device, written the way the
// reference writes its own: the documented examples of the reduce / normalisation traits
// (hpt-traits/src/ops/reduce.rs:21-39, 58-62, 146-149, 166-168, 294-297, 328-331, 347-350), views
// against a plain host loop over the same strides (hpt-tests/src/hpt/cpu/reduce.rs:63-291), closed
// forms for softmax / layernorm, and the error texts of hpt-common/src/axis/axis.rs:38-73.
// Prints one line per failure; exit status 0 when all pass.
#include <dlfcn.h>

#include <cmath>
#include <cstdio>
#include <functional>
#include <random>

#include "hpt_hip.hpp"

using hpt::Tensor;
static int failures = 0, checks = 0;

#define EXPECT(cond, ...)                                  \
    do {                                                   \
        ++checks;                                          \
        if (!(cond)) {                                     \
            ++failures;                                    \
            printf("FAIL %s:%d: ", __FILE__, __LINE__);    \
            printf(__VA_ARGS__);                           \
            printf("\n");                                  \
        }                                                  \
    } while (0)

static bool close(double got, double want, double rtol = 1e-5, double atol = 1e-6) {
    return std::fabs(got - want) <= atol + rtol * std::fabs(want);
}

template <class F> static void expect_error(hpt::ErrorKind kind, const char* text, F f, const char* what) {
    ++checks;
    try {
        f();
    } catch (const hpt::TensorError& e) {
        if (e.kind != kind || (text && std::string(e.what()).find(text) == std::string::npos)) {
            ++failures;
            printf("FAIL %s: wrong error: kind %d, text '%s'\n", what, (int)e.kind, e.what());
        }
        return;
    }
    ++failures;
    printf("FAIL %s: no error raised\n", what);
}

// host gather of a strided view: out[i] for row-major index i
template <class T>
static std::vector<T> gather(const std::vector<T>& base, int64_t offset, const hpt::Shape& shape, const hpt::Shape& strides) {
    int64_t n = 1;
    for (auto d : shape) n *= d;
    std::vector<T> out((size_t)n);
    std::vector<int64_t> idx(shape.size(), 0);
    for (int64_t i = 0; i < n; ++i) {
        int64_t off = offset;
        for (size_t d = 0; d < shape.size(); ++d) off += idx[d] * strides[d];
        out[(size_t)i] = base[(size_t)off];
        for (int d = (int)shape.size() - 1; d >= 0; --d) {
            if (++idx[d] < shape[d]) break;
            idx[d] = 0;
        }
    }
    return out;
}

static void documented_examples() {
    auto a = Tensor<float>::from_host({1, 2, 3, 4}, {2, 2});
    EXPECT(a.sum({0, 1}).to_host()[0] == 10.0f, "sum([[1,2],[3,4]], [0,1]) != 10");
    EXPECT(a.sum({0, 1}).shape() == hpt::Shape({1}), "full reduction has shape [1]");
    EXPECT(a.sum({0, 1}, true).shape() == hpt::Shape({1, 1}), "keep_dims shape");
    EXPECT(a.mean({0, 1}).to_host()[0] == 2.5f, "mean != 2.5");
    EXPECT(a.sum_square({0, 1}).to_host()[0] == 30.0f, "sum_square != 30");
    EXPECT(a.reducel1({0, 1}).to_host()[0] == 10.0f, "reducel1 != 10");
    EXPECT(close(a.reducel2({0, 1}).to_host()[0], std::sqrt(30.0)), "reducel2");
    EXPECT(close(a.reducel3({0, 1}).to_host()[0], std::cbrt(100.0)), "reducel3");
    EXPECT(close(a.logsumexp({0, 1}).to_host()[0], 4.4401898), "logsumexp");
    EXPECT(a.prod({1}).to_host() == std::vector<float>({2, 12}), "prod over axis 1");
    EXPECT(a.max({0}).to_host() == std::vector<float>({3, 4}) && a.min({-1}).to_host() == std::vector<float>({1, 3}), "max / min");
    auto v = Tensor<float>::from_host({10, 3, 2}, {3});
    EXPECT(v.argmax(0).to_host()[0] == 0 && v.argmin(0).to_host()[0] == 2, "argmax([10,3,2]) = 0, argmin = 2");
    auto ties = Tensor<int32_t>::from_host({5, 9, 9, 1, 1, 7}, {2, 3});
    EXPECT(ties.argmax(1).to_host() == std::vector<int64_t>({1, 2}), "ties resolve to the first index");
    EXPECT(ties.argmin(-1, true).shape() == hpt::Shape({2, 1}), "argmin keep_dims");
    // integers wrap; bool all / any; nansum
    auto w = Tensor<int8_t>::from_host({100, 100, 100, -128}, {4});
    EXPECT(w.sum({0}).to_host()[0] == (int8_t)(172), "i8 sum wraps");
    auto b = Tensor<bool>::from_host({1, 0, 1, 1}, {2, 2});
    EXPECT(b.all({1}).to_host() == std::vector<uint8_t>({0, 1}) && b.any({0}).to_host() == std::vector<uint8_t>({1, 1}), "all / any");
    auto nn = Tensor<float>::from_host({1, NAN, 3, 4}, {2, 2});
    EXPECT(nn.nansum({1}).to_host() == std::vector<float>({1, 7}), "nansum");
    // i32 mean -> f32 (FloatBinaryType)
    auto im = Tensor<int32_t>::from_host({1, 2, 3, 5}, {2, 2});
    static_assert(std::is_same<decltype(im.mean({0}))::Elem, float>::value, "mean of i32 is f32");
    EXPECT(im.mean({1}).to_host() == std::vector<float>({1.5f, 4.0f}), "mean of i32");
    // sum_ accumulates into out
    auto acc = Tensor<float>::full(100.0f, {2});
    a.sum_({1}, false, false, acc);
    EXPECT(acc.to_host() == std::vector<float>({103, 107}), "sum_ with init_out = false accumulates");
}

static void views_against_host_loops() {
    std::mt19937 rng(7);
    std::normal_distribution<float> nd(0.f, 1.f);
    const hpt::Shape shape = {6, 10, 14};
    std::vector<float> base(6 * 10 * 14);
    for (auto& x : base) x = nd(rng);
    auto t = Tensor<float>::from_host(base, shape);
    struct Case { const char* name; Tensor<float> view; };
    std::vector<Case> cases = {
        {"contiguous", t},
        {"permuted", t.permute({2, 0, 1})},
        {"sliced", t.slice({{1, 5, 1}, {2, 9, 1}, {0, 14, 1}})},
        {"stepped", t.slice({{0, 6, 2}, {1, 10, 3}, {0, 14, 2}})},
        {"permuted + stepped", t.permute({1, 2, 0}).slice({{0, 10, 2}, {3, 14, 1}})},
    };
    for (auto& c : cases) {
        const auto& v = c.view;
        // offset of the view inside the base buffer = difference of the data pointers
        const int64_t off = ((const float*)v.view().data - (const float*)t.view().data);
        auto host = gather(base, off, v.shape(), v.strides());
        EXPECT(v.to_host() == host, "%s: to_host differs from the host gather", c.name);
        EXPECT(v.contiguous().to_host() == host, "%s: contiguous()", c.name);
        const hpt::Shape sh = v.shape();
        for (int axis = 0; axis < 3; ++axis) {
            // reduce one axis on the host in double
            int64_t outer = 1, n = sh[axis], inner = 1;
            for (int d = 0; d < axis; ++d) outer *= sh[d];
            for (int d = axis + 1; d < 3; ++d) inner *= sh[d];
            auto got_sum = v.sum({axis}).to_host();
            auto got_max = v.max({axis}).to_host();
            auto got_arg = v.argmax(axis).to_host();
            bool ok = true;
            for (int64_t o = 0; o < outer && ok; ++o)
                for (int64_t i = 0; i < inner && ok; ++i) {
                    double s = 0;
                    float m = -INFINITY;
                    int64_t am = 0;
                    for (int64_t k = 0; k < n; ++k) {
                        const float x = host[(size_t)((o * n + k) * inner + i)];
                        s += x;
                        if (x > m) { m = x; am = k; }
                    }
                    const size_t oi = (size_t)(o * inner + i);
                    ok = close(got_sum[oi], s) && got_max[oi] == m && got_arg[oi] == am;
                }
            EXPECT(ok, "%s: sum / max / argmax over axis %d", c.name, axis);
        }
        // softmax over the last axis: rows sum to one and follow exp(x - max) / sum
        auto sm = v.softmax(-1).to_host();
        const int64_t rows = sh[0] * sh[1], cols = sh[2];
        bool ok = true;
        for (int64_t r = 0; r < rows && ok; ++r) {
            double m = -INFINITY, s = 0;
            for (int64_t k = 0; k < cols; ++k) m = std::max<double>(m, host[(size_t)(r * cols + k)]);
            for (int64_t k = 0; k < cols; ++k) s += std::exp(host[(size_t)(r * cols + k)] - m);
            for (int64_t k = 0; k < cols && ok; ++k) ok = close(sm[(size_t)(r * cols + k)], std::exp(host[(size_t)(r * cols + k)] - m) / s);
        }
        EXPECT(ok, "%s: softmax(-1)", c.name);
    }
}

static void normalisation_closed_forms() {
    auto a = Tensor<float>::from_host({1, 2, 3, 4}, {2, 2});
    auto s = a.softmax(1).to_host();
    EXPECT(close(s[0], 0.2689414213699951) && close(s[1], 0.7310585786300049) && close(s[2], s[0]), "softmax [[1,2],[3,4]]");
    auto ls = a.log_softmax(0).to_host();
    EXPECT(close(ls[0], -2.1269280110429727) && close(ls[2], -0.1269280110429727), "log_softmax over axis 0");
    // constant rows -> beta; 2-element rows -> +-1/sqrt(1 + eps/var)
    std::vector<float> c(3 * 64, 7.25f), g(64), b(64);
    for (int i = 0; i < 64; ++i) { g[i] = 0.5f + i / 64.f; b[i] = -1.f + i / 32.f; }
    auto tc = Tensor<float>::from_host(c, {3, 64});
    auto tg = Tensor<float>::from_host(g, {64}), tb = Tensor<float>::from_host(b, {64});
    auto out = tc.layernorm({64}, &tg, &tb, 1e-5).to_host();
    bool ok = true;
    for (int r = 0; r < 3; ++r)
        for (int i = 0; i < 64; ++i) ok = ok && out[r * 64 + i] == b[i];
    EXPECT(ok, "layernorm of constant rows is beta");
    auto two = Tensor<float>::from_host({1, 3, -2, 6}, {2, 2}).layernorm({2}, nullptr, nullptr, 1e-5).to_host();
    EXPECT(close(two[0], -1 / std::sqrt(1 + 1e-5 / 1.0), 1e-6, 1e-7) && close(two[3], 1 / std::sqrt(1 + 1e-5 / 16.0), 1e-6, 1e-7),
           "layernorm of 2-element rows");
    // integer input: Output = Tensor<FloatBinaryType<T>>
    auto is = Tensor<int32_t>::from_host({1, 2, 3, 4}, {2, 2}).softmax(1);
    static_assert(std::is_same<decltype(is)::Elem, float>::value, "softmax of i32 is f32");
    EXPECT(close(is.to_host()[1], 0.7310585786300049), "softmax of an i32 tensor");
    // in-place affine steps equal the fused layernorm
    auto x = Tensor<float>::from_host({0.5f, -1.f, 2.f, 4.f, 1.f, 1.5f, -3.f, 0.f}, {2, 4});
    auto g4 = Tensor<float>::from_host({1, 2, 3, 4}, {4}), b4 = Tensor<float>::from_host({0.1f, 0.2f, 0.3f, 0.4f}, {4});
    auto fused = x.layernorm({4}, &g4, &b4, 1e-5).to_host();
    auto steps = x.layernorm({4}, nullptr, nullptr, 1e-5);
    steps.mul_(g4, steps);
    steps.add_(b4, steps);
    auto sh = steps.to_host();
    ok = true;
    for (size_t i = 0; i < fused.size(); ++i) ok = ok && close(sh[i], fused[i], 2e-6, 2e-7);
    EXPECT(ok, "normalise, mul_(gamma), add_(beta) equals the fused layernorm");
}

static void error_behaviour() {
    auto a = Tensor<float>::from_host({1, 2, 3, 4}, {2, 2});
    expect_error(hpt::ErrorKind::Shape, "Dimension out of range: expected in 0..2, got 2", [&] { a.sum({2}); }, "axis out of range");
    expect_error(hpt::ErrorKind::Shape, "Dimension out of range", [&] { a.sum({-3}); }, "negative axis out of range");
    expect_error(hpt::ErrorKind::Param, "Axis 1 is duplicated", [&] { a.sum({1, 1}); }, "duplicated axis");
    // the same axis named twice in different forms is refused too (the reference compares the raw values only)
    expect_error(hpt::ErrorKind::Param, "Axis -1 is duplicated", [&] { a.sum({1, -1}); }, "duplicated axis, mixed signs");
    expect_error(hpt::ErrorKind::Shape, "normalized dims must match last dims", [&] { a.layernorm({3}, nullptr, nullptr, 1e-5); },
                 "layernorm shape");
    expect_error(hpt::ErrorKind::Shape, nullptr, [&] { a + Tensor<float>::from_host({1, 2, 3}, {3}); }, "broadcast failure");
    expect_error(hpt::ErrorKind::DType, nullptr, [&] { Tensor<int32_t>::from_host({1, 2}, {2}) / Tensor<int32_t>::from_host({1, 2}, {2}); },
                 "integer division is not provided");
    EXPECT(a.sum({-1}).to_host() == std::vector<float>({3, 7}), "negative axis wraps");
}

// Tensor::forget / from_raw / allclose (hpt/src/backends/cuda/tensor_impls.rs:259-306,
// hpt/src/backends/cpu/tensor_impls.rs:123-147, 218-248): a block given up by the library becomes
// the caller's raw device memory; tensors adopted over it - at an address that is only
// element-aligned - compute like any other and free nothing when they go.
static void foreign_memory() {
    uint64_t live0 = 0, live1 = 0, live2 = 0;
    std::vector<float> data(1000);
    std::mt19937 rng(5);
    std::normal_distribution<float> nd(0.f, 2.f);
    for (auto& x : data) x = nd(rng);
    auto t = Tensor<float>::from_host(data, {1000});
    hpt_hip_alloc_stats(0, &live0, nullptr, nullptr);
    expect_error(hpt::ErrorKind::Param, "tensor is a view", [&] { auto v = t.slice({{1, 1000, 1}}); v.forget(); }, "forget of a view");
    {
        auto shared = t.reshape({1000});  // a second owner of the block
        (void)shared;
    }
    {
        Tensor<float> second = t;
        expect_error(hpt::ErrorKind::Param, "ref_count: 2", [&] { t.forget(); }, "forget of a shared block");
    }
    const auto f = t.forget();
    hpt_hip_alloc_stats(0, &live1, nullptr, nullptr);
    EXPECT(live1 + 1 == live0, "forget: live blocks %llu -> %llu", (unsigned long long)live0, (unsigned long long)live1);
    EXPECT(f.bytes == 4000 && f.align == 64 && t.size() == 0, "forget: layout (%zu, %zu)", f.bytes, f.align);
    EXPECT(hpt_hip_free(0, f.ptr, f.bytes, f.align) == HPT_ERR_MEMORY, "the allocator must not know a forgotten block");
    {
        // 999 floats from the second element on: 4 bytes past a 64-byte boundary
        auto raw = Tensor<float>::from_raw((float*)f.ptr + 1, {37, 27});
        auto sums = raw.sum({1}).to_host();
        bool ok = true;
        for (int r = 0; r < 37; ++r) {
            double want = 0;
            for (int c = 0; c < 27; ++c) want += data[1 + r * 27 + c];
            ok = ok && close(sums[r], want, 1e-5, 1e-5);
        }
        EXPECT(ok, "sum over rows of a raw, odd-aligned tensor");
        auto am = raw.argmax(1).to_host();
        ok = true;
        for (int r = 0; r < 37; ++r) {
            int best = 0;
            for (int c = 1; c < 27; ++c)
                if (data[1 + r * 27 + c] > data[1 + r * 27 + best]) best = c;
            ok = ok && am[r] == best;
        }
        EXPECT(ok, "argmax of a raw tensor");
        auto sm = raw.softmax(1);
        auto rows = sm.sum({1}).to_host();
        ok = true;
        for (float v : rows) ok = ok && close(v, 1.0, 1e-5, 1e-6);
        EXPECT(ok, "softmax rows of a raw tensor sum to one");
        auto ln = raw.layernorm({27}, nullptr, nullptr, 1e-5);
        auto means = ln.mean({1}).to_host();
        ok = true;
        for (float v : means) ok = ok && std::fabs(v) < 1e-5;
        EXPECT(ok, "layernorm rows of a raw tensor have mean zero");
        // a strided view of the raw memory: every second column, and the same numbers gathered on the host
        auto stepped = Tensor<float>::from_raw((float*)f.ptr + 1, {37, 14}, {27, 2});
        std::vector<float> gathered;
        for (int r = 0; r < 37; ++r)
            for (int c = 0; c < 27; c += 2) gathered.push_back(data[1 + r * 27 + c]);
        auto copy = Tensor<float>::from_host(gathered, {37, 14});
        EXPECT(stepped.allclose(copy, 0.0, 0.0), "allclose: a raw stepped view against its gathered copy");
        EXPECT(!stepped.allclose(copy.reshape({14, 37}), 1.0, 1.0), "allclose: shapes differ");
        auto shifted = copy + Tensor<float>::full(1e-3f, {1});
        EXPECT(!stepped.allclose(shifted, 0.0, 1e-4) && stepped.allclose(shifted, 0.0, 2e-3), "allclose: absolute tolerance");
        auto nan1 = Tensor<float>::from_host({NAN, INFINITY, 1.f}, {3}), nan2 = Tensor<float>::from_host({NAN, INFINITY, 1.f}, {3});
        auto inf2 = Tensor<float>::from_host({NAN, -INFINITY, 1.f}, {3});
        EXPECT(nan1.allclose(nan2, 0.0, 0.0) && !nan1.allclose(inf2, 1.0, 1.0), "allclose: NaN equals NaN, infinities by sign");
    }
    hpt::synchronize();
    hpt_hip_alloc_stats(0, &live2, nullptr, nullptr);
    EXPECT(live2 == live1, "tensors over raw memory changed the live block count: %llu -> %llu", (unsigned long long)live1,
           (unsigned long long)live2);
    // the memory is the caller's now: release it with the runtime's own free
    using hipFree_t = int (*)(void*);
    auto hip_free = (hipFree_t)dlsym(RTLD_DEFAULT, "hipFree");
    EXPECT(hip_free != nullptr && hip_free(f.ptr) == 0, "hipFree of the forgotten block");
    expect_error(hpt::ErrorKind::Param, "data is null", [&] { Tensor<float>::from_raw(nullptr, {4}); }, "from_raw(null)");
}

int main() {
    if (hpt::device_count() < 1) {
        printf("no HIP device\n");
        return 2;
    }
    documented_examples();
    views_against_host_loops();
    normalisation_closed_forms();
    error_behaviour();
    foreign_memory();
    hpt::synchronize();
    printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
