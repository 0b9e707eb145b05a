// hpt_hip.hpp — the host side of the Hip backend in C++ (header only), above the C ABI of
// libhpt_hip.so (hpt_hip.h). It mirrors, for the reduction / softmax / layernorm path, the
// interface Hpt's tensors have in Rust: the same method names, argument meaning, output types
// and error behaviour, so that code and tests written against the reference read the same.
//
//   hpt::Tensor<T>                      Tensor<T, Hip, DEVICE_ID>   (hpt/src/tensor.rs:31-37)
//   Tensor::from_host / to_host         Tensor::new(..).to_cuda() / to_cpu()
//                                       (hpt/src/backends/cpu/tensor_impls.rs:295-313,
//                                        hpt/src/backends/cuda/tensor_impls.rs:142-169)
//   Tensor::from_raw / forget / allclose
//                                       (hpt/src/backends/cpu/tensor_impls.rs:123-147, 218-248;
//                                        hpt/src/backends/cuda/tensor_impls.rs:259-306)
//   permute / transpose / t / slice / expand
//                                       ShapeManipulate, Slice (hpt/src/backends/common/
//                                       shape_manipulate.rs:19-52, hpt-common/src/slice.rs:20-95)
//   sum prod min max reducel1 sum_square sum_     NormalReduce  (hpt-traits/src/ops/reduce.rs:45-176)
//   nansum nanprod all any                        NormalEvalReduce / EvalReduce (:180-278)
//   mean reducel2 reducel3 logsumexp              FloatReduce   (:280-358)
//   argmax argmin                                 IndexReduce   (:6-42)
//   softmax log_softmax layernorm                 NormalizationOps (hpt-traits/src/ops/normalization.rs:6-64)
//   contiguous astype add_ sub_ mul_ div_         Contiguous, astype, NormalBinOps
//
// Errors are thrown as hpt::TensorError, whose `kind` is the TensorError variant the Rust shim
// would return (hpt-common/src/error/base.rs:8-45) and whose text is the library's.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <numeric>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "hpt_hip.h"

namespace hpt {

// ---- errors ------------------------------------------------------------------------------
enum class ErrorKind { Param = 1, Shape = 2, DType = 3, Memory = 4, Kernel = 5, Device = 6 };

struct TensorError : std::runtime_error {
    ErrorKind kind;
    TensorError(ErrorKind k, const std::string& m) : std::runtime_error(m), kind(k) {}
};

inline void check(int32_t status) {
    if (status == HPT_OK) return;
    const char* m = hpt_hip_last_error();
    throw TensorError(static_cast<ErrorKind>(status), m ? m : "unknown error");
}

// ---- element types -------------------------------------------------------------------------
struct f16 { uint16_t bits; };   // IEEE binary16 bit pattern (`half::f16`)
struct bf16 { uint16_t bits; };  // bfloat16 bit pattern (`half::bf16`)

inline float to_float(bf16 h) {
    uint32_t u = (uint32_t)h.bits << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
inline bf16 bf16_from_float(float f) {  // round to nearest even
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return bf16{(uint16_t)((u >> 16) | 0x40)};
    u += 0x7fffu + ((u >> 16) & 1u);
    return bf16{(uint16_t)(u >> 16)};
}
inline float to_float(f16 h) {
    const uint32_t s = (uint32_t)(h.bits & 0x8000) << 16, e = (h.bits >> 10) & 0x1f, m = h.bits & 0x3ff;
    uint32_t u;
    if (e == 0) {
        if (m == 0) {
            u = s;
        } else {  // subnormal: normalise
            int sh = 0;
            uint32_t mm = m;
            while (!(mm & 0x400)) { mm <<= 1; ++sh; }
            u = s | ((uint32_t)(113 - sh) << 23) | ((mm & 0x3ff) << 13);
        }
    } else if (e == 31) {
        u = s | 0x7f800000u | (m << 13);
    } else {
        u = s | ((e + 112) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

template <class T> struct dtype_of;
#define HPT_DTYPE_OF(T, D) template <> struct dtype_of<T> { static constexpr hpt_dtype value = D; };
HPT_DTYPE_OF(bool, HPT_BOOL) HPT_DTYPE_OF(int8_t, HPT_I8) HPT_DTYPE_OF(int16_t, HPT_I16) HPT_DTYPE_OF(int32_t, HPT_I32)
HPT_DTYPE_OF(int64_t, HPT_I64) HPT_DTYPE_OF(uint8_t, HPT_U8) HPT_DTYPE_OF(uint16_t, HPT_U16) HPT_DTYPE_OF(uint32_t, HPT_U32)
HPT_DTYPE_OF(uint64_t, HPT_U64) HPT_DTYPE_OF(f16, HPT_F16) HPT_DTYPE_OF(bf16, HPT_BF16) HPT_DTYPE_OF(float, HPT_F32)
HPT_DTYPE_OF(double, HPT_F64)
#undef HPT_DTYPE_OF

// FloatBinaryType<T> (hpt-types/src/type_promote.rs; normal_promote tables): the output element
// type of mean / reducel2 / logsumexp / softmax / layernorm.
template <class T> struct float_binary_type { using type = f16; };  // bool, i8, i16, u8, u16, f16
template <> struct float_binary_type<int32_t> { using type = float; };
template <> struct float_binary_type<uint32_t> { using type = float; };
template <> struct float_binary_type<float> { using type = float; };
template <> struct float_binary_type<bf16> { using type = bf16; };
template <> struct float_binary_type<int64_t> { using type = double; };
template <> struct float_binary_type<uint64_t> { using type = double; };
template <> struct float_binary_type<double> { using type = double; };
template <class T> using FloatBinaryType = typename float_binary_type<T>::type;

// host-side element type (std::vector<bool> is bit-packed: bool tensors travel as bytes)
template <class T> struct host_elem { using type = T; };
template <> struct host_elem<bool> { using type = uint8_t; };
template <class T> using HostElem = typename host_elem<T>::type;

using Shape = std::vector<int64_t>;
using Axes = std::vector<int64_t>;
constexpr size_t kAlign = 64;  // the alignment Hpt's allocators use (hpt-allocator/src/lib.rs ALIGN)

// ---- device storage: freed back to the library's LRU cache when the last tensor drops it -------
struct DeviceBlock {
    int device;
    void* ptr = nullptr;
    size_t bytes;
    DeviceBlock(int dev, size_t n) : device(dev), bytes(n ? n : 1) { check(hpt_hip_alloc(dev, bytes, kAlign, 0, &ptr)); }
    ~DeviceBlock() {
        if (ptr) hpt_hip_free(device, ptr, bytes, kAlign);
    }
    DeviceBlock(const DeviceBlock&) = delete;
    DeviceBlock& operator=(const DeviceBlock&) = delete;
};

inline Shape contiguous_strides(const Shape& shape) {
    Shape st(shape.size());
    int64_t acc = 1;
    for (int i = (int)shape.size() - 1; i >= 0; --i) {
        st[i] = acc;
        acc *= shape[i];
    }
    return st;
}

template <class T> class Tensor {
  public:
    using Elem = T;

    // ---- creation / transfer ------------------------------------------------------------
    static Tensor empty(const Shape& shape, int device = 0) {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        Tensor t;
        t.block_ = std::make_shared<DeviceBlock>(device, (size_t)n * sizeof(T));
        t.data_ = (T*)t.block_->ptr;
        t.shape_ = shape;
        t.strides_ = contiguous_strides(shape);
        t.device_ = device;
        return t;
    }
    // Tensor::new(data).to_cuda(): one synchronous host-to-device copy
    static Tensor from_host(const std::vector<HostElem<T>>& data, const Shape& shape, int device = 0) {
        Tensor t = empty(shape, device);
        if ((int64_t)data.size() != t.size())
            throw TensorError(ErrorKind::Shape, "from_host: data has " + std::to_string(data.size()) + " elements, shape needs " +
                                                    std::to_string(t.size()));
        if (!data.empty()) check(hpt_hip_memcpy_h2d_sync(device, t.data_, data.data(), data.size() * sizeof(T)));
        return t;
    }
    // Tensor::from_raw: a tensor over device memory the caller owns; dropping it frees nothing. The
    // reference takes a contiguous shape and asserts 64-byte alignment; here any element-aligned
    // pointer is taken (the kernels read unaligned rows) and `strides` may describe any view.
    static Tensor from_raw(T* data, const Shape& shape, int device = 0) { return from_raw(data, shape, contiguous_strides(shape), device); }
    static Tensor from_raw(T* data, const Shape& shape, const Shape& strides, int device = 0) {
        if (!data) throw TensorError(ErrorKind::Param, "data is null");
        if ((uintptr_t)data % sizeof(T)) throw TensorError(ErrorKind::Param, "data is not aligned to its element size");
        if (shape.size() != strides.size()) throw TensorError(ErrorKind::Shape, "from_raw: shape and strides differ in length");
        Tensor t;
        t.data_ = data;
        t.shape_ = shape;
        t.strides_ = strides;
        t.device_ = device;
        return t;
    }
    // Tensor::forget: give the allocation up. The allocator stops tracking the block and the caller
    // releases it (hipFree). Fails for a view and while another tensor shares the storage.
    struct Forgotten { void* ptr; size_t bytes, align; };
    Forgotten forget() {
        if (is_view_) throw TensorError(ErrorKind::Param, "Can't forget tensor: tensor is a view, cannot forget");
        if (block_ && block_.use_count() > 1)
            throw TensorError(ErrorKind::Param, "Can't forget tensor: ref_count: " + std::to_string(block_.use_count()));
        Forgotten f{(void*)data_, block_ ? block_->bytes : (size_t)size() * sizeof(T), kAlign};
        if (block_) {
            check(hpt_hip_stream_synchronize(device_, nullptr));
            check(hpt_hip_forget(device_, block_->ptr));
            block_->ptr = nullptr;
            block_.reset();
        }
        data_ = nullptr;
        shape_ = {0};
        strides_ = {1};
        return f;
    }
    // allclose: both sides go to the host; shapes must match, NaN equals NaN, infinities by sign,
    // else |a - b| <= atol + rtol * |b|.
    bool allclose(const Tensor& other, double rtol, double atol) const {
        if (shape_ != other.shape_) return false;
        const auto a = to_host(), b = other.to_host();
        auto val = [](HostElem<T> v) -> double {
            if constexpr (std::is_same<T, f16>::value || std::is_same<T, bf16>::value) return (double)to_float(v);
            else return (double)v;
        };
        for (size_t i = 0; i < a.size(); ++i) {
            const double x = val(a[i]), y = val(b[i]);
            if (std::isnan(x) && std::isnan(y)) continue;
            if (std::isinf(x) && std::isinf(y)) {
                if ((x > 0) != (y > 0)) return false;
                continue;
            }
            if (!(std::fabs(x - y) <= atol + rtol * std::fabs(y))) return false;
        }
        return true;
    }
    static Tensor full(T value, const Shape& shape, int device = 0) {
        Tensor t = empty(shape, device);
        hpt_view v = t.view();
        check(hpt_hip_fill(device, nullptr, &v, &value));
        return t;
    }
    // to_cpu: a view is made contiguous on the device first, then copied back synchronously
    std::vector<HostElem<T>> to_host() const {
        const Tensor src = (is_contiguous() && !is_view_) ? *this : contiguous();
        std::vector<HostElem<T>> out((size_t)size());
        check(hpt_hip_stream_synchronize(device_, nullptr));
        if (!out.empty()) check(hpt_hip_memcpy_d2h_sync(device_, out.data(), src.data_, out.size() * sizeof(T)));
        return out;
    }

    // ---- layout --------------------------------------------------------------------------------
    const Shape& shape() const { return shape_; }
    const Shape& strides() const { return strides_; }
    int ndim() const { return (int)shape_.size(); }
    int64_t size() const {
        int64_t n = 1;
        for (int64_t d : shape_) n *= d;
        return n;
    }
    int device() const { return device_; }
    bool is_contiguous() const {
        int64_t expect = 1;
        for (int i = ndim() - 1; i >= 0; --i) {
            if (shape_[i] == 0) return true;
            if (shape_[i] != 1 && strides_[i] != expect) return false;
            expect *= shape_[i];
        }
        return true;
    }
    hpt_view view() const { return hpt_view{(void*)data_, shape_.data(), strides_.data(), (int32_t)shape_.size(), dtype_of<T>::value}; }

    // ---- views (share the storage) ---------------------------------------------------------------
    Tensor permute(const Axes& axes) const {
        Axes norm(axes.size());
        if ((int)axes.size() != ndim())
            throw TensorError(ErrorKind::Shape, "permute: expected " + std::to_string(ndim()) + " axes");
        check(hpt_hip_process_axes(axes.data(), (int32_t)axes.size(), ndim(), norm.data()));
        Tensor t = alias();
        for (int i = 0; i < ndim(); ++i) {
            t.shape_[i] = shape_[norm[i]];
            t.strides_[i] = strides_[norm[i]];
        }
        return t;
    }
    Tensor transpose(int64_t a, int64_t b) const {
        Axes ax(ndim());
        std::iota(ax.begin(), ax.end(), 0);
        Axes two = {a, b}, norm(2);
        check(hpt_hip_process_axes(two.data(), 2, ndim(), norm.data()));
        std::swap(ax[norm[0]], ax[norm[1]]);
        return permute(ax);
    }
    Tensor t() const {
        Axes ax(ndim());
        for (int i = 0; i < ndim(); ++i) ax[i] = ndim() - 1 - i;
        return permute(ax);
    }
    // (start, end, step) per leading dim, end exclusive, negative indices count from the back; step > 0
    struct Range { int64_t start, end, step; };
    Tensor slice(const std::vector<Range>& ranges) const {
        if ((int)ranges.size() > ndim()) throw TensorError(ErrorKind::Shape, "slice: more ranges than dims");
        Tensor t = alias();
        for (size_t i = 0; i < ranges.size(); ++i) {
            const int64_t n = shape_[i];
            int64_t s = ranges[i].start, e = ranges[i].end, st = ranges[i].step;
            if (st <= 0) throw TensorError(ErrorKind::Param, "slice: this mirror takes positive steps only");
            if (s < 0) s += n;
            if (e < 0) e += n;
            s = s < 0 ? 0 : (s > n ? n : s);
            e = e < 0 ? 0 : (e > n ? n : e);
            const int64_t len = e > s ? (e - s + st - 1) / st : 0;
            t.data_ += s * strides_[i];
            t.shape_[i] = len;
            t.strides_[i] = strides_[i] * st;
        }
        return t;
    }
    Tensor expand(const Shape& shape) const {
        if ((int)shape.size() < ndim()) throw TensorError(ErrorKind::Shape, "expand: fewer dims than the tensor has");
        Tensor t = alias();
        const int pad = (int)shape.size() - ndim();
        t.shape_ = shape;
        t.strides_.assign(shape.size(), 0);
        for (int i = pad; i < (int)shape.size(); ++i) {
            const int64_t old = shape_[i - pad];
            if (old == shape[i]) t.strides_[i] = strides_[i - pad];
            else if (old != 1) throw TensorError(ErrorKind::Shape, "expand: cannot broadcast dim " + std::to_string(i - pad));
        }
        return t;
    }

    // ---- NormalReduce ---------------------------------------------------------------------------
    Tensor sum(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_SUM, axes, keep_dims); }
    Tensor prod(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_PROD, axes, keep_dims); }
    Tensor min(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_MIN, axes, keep_dims); }
    Tensor max(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_MAX, axes, keep_dims); }
    Tensor reducel1(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_REDUCEL1, axes, keep_dims); }
    Tensor sum_square(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_SUM_SQUARE, axes, keep_dims); }
    // sum_: the result goes to `out`; init_out = false accumulates into what `out` holds
    Tensor sum_(const Axes& axes, bool keep_dims, bool init_out, Tensor out) const {
        return reduce_into(HPT_SUM, axes, keep_dims, init_out, out);
    }
    // ---- NormalEvalReduce / EvalReduce ----------------------------------------------------------
    Tensor nansum(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_NANSUM, axes, keep_dims); }
    Tensor nanprod(const Axes& axes, bool keep_dims = false) const { return reduce<T>(HPT_NANPROD, axes, keep_dims); }
    Tensor nansum_(const Axes& axes, bool keep_dims, bool init_out, Tensor out) const {
        return reduce_into(HPT_NANSUM, axes, keep_dims, init_out, out);
    }
    Tensor<bool> all(const Axes& axes, bool keep_dims = false) const { return reduce<bool>(HPT_ALL, axes, keep_dims); }
    Tensor<bool> any(const Axes& axes, bool keep_dims = false) const { return reduce<bool>(HPT_ANY, axes, keep_dims); }
    // ---- FloatReduce ------------------------------------------------------------------------------
    using FloatOut = Tensor<FloatBinaryType<T>>;
    FloatOut mean(const Axes& axes, bool keep_dims = false) const { return reduce<FloatBinaryType<T>>(HPT_MEAN, axes, keep_dims); }
    FloatOut reducel2(const Axes& axes, bool keep_dims = false) const { return reduce<FloatBinaryType<T>>(HPT_REDUCEL2, axes, keep_dims); }
    FloatOut reducel3(const Axes& axes, bool keep_dims = false) const { return reduce<FloatBinaryType<T>>(HPT_REDUCEL3, axes, keep_dims); }
    FloatOut logsumexp(const Axes& axes, bool keep_dims = false) const { return reduce<FloatBinaryType<T>>(HPT_LOGSUMEXP, axes, keep_dims); }
    // ---- IndexReduce --------------------------------------------------------------------------------
    Tensor<int64_t> argmax(int64_t axis, bool keep_dims = false) const { return argreduce(true, axis, keep_dims); }
    Tensor<int64_t> argmin(int64_t axis, bool keep_dims = false) const { return argreduce(false, axis, keep_dims); }

    // ---- NormalizationOps (Output = Tensor<FloatBinaryType<T>>) -----------------------------------
    FloatOut softmax(int64_t axis) const { return softmax_impl(false, axis); }
    FloatOut log_softmax(int64_t axis) const { return softmax_impl(true, axis); }
    FloatOut layernorm(const Shape& normalized_shape, const FloatOut* gamma, const FloatOut* beta, double eps) const {
        // same check (and text) as hpt/src/backends/cpu/tensor_internal/normalization.rs:61-72
        bool ok = !normalized_shape.empty() && (int)normalized_shape.size() <= ndim();
        for (size_t i = 0; ok && i < normalized_shape.size(); ++i)
            ok = shape_[ndim() - normalized_shape.size() + i] == normalized_shape[i];
        if (!ok) throw TensorError(ErrorKind::Shape, "normalized dims must match last dims of input tensor");
        // a non-float input is promoted to FloatBinaryType<T> inside the kernel: one call, no copy
        FloatOut res = FloatOut::empty(shape_, device_);
        hpt_view vin = view(), vout = res.view(), vg{}, vb{};
        if (gamma) vg = gamma->view();
        if (beta) vb = beta->view();
        check(hpt_hip_layernorm(device_, nullptr, &vin, (int32_t)normalized_shape.size(), gamma ? &vg : nullptr,
                                beta ? &vb : nullptr, eps, &vout));
        return res;
    }

    // ---- the steps either side ---------------------------------------------------------------------
    Tensor contiguous() const {
        Tensor res = empty(shape_, device_);
        hpt_view vin = view(), vout = res.view();
        check(hpt_hip_contiguous(device_, nullptr, &vin, &vout));
        return res;
    }
    template <class U> Tensor<U> astype() const {
        Tensor<U> res = Tensor<U>::empty(shape_, device_);
        hpt_view vin = view(), vout = res.view();
        check(hpt_hip_cast(device_, nullptr, &vin, &vout));
        return res;
    }
    Tensor add_(const Tensor& rhs, Tensor out) const { return binary(HPT_BIN_ADD, rhs, &out); }
    Tensor sub_(const Tensor& rhs, Tensor out) const { return binary(HPT_BIN_SUB, rhs, &out); }
    Tensor mul_(const Tensor& rhs, Tensor out) const { return binary(HPT_BIN_MUL, rhs, &out); }
    Tensor div_(const Tensor& rhs, Tensor out) const { return binary(HPT_BIN_DIV, rhs, &out); }
    Tensor operator+(const Tensor& rhs) const { return binary(HPT_BIN_ADD, rhs, nullptr); }
    Tensor operator-(const Tensor& rhs) const { return binary(HPT_BIN_SUB, rhs, nullptr); }
    Tensor operator*(const Tensor& rhs) const { return binary(HPT_BIN_MUL, rhs, nullptr); }
    Tensor operator/(const Tensor& rhs) const { return binary(HPT_BIN_DIV, rhs, nullptr); }

    // reshape of a contiguous tensor (what keep_dims amounts to, reduce_template.rs:252)
    Tensor reshape(const Shape& shape) const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        if (n != size() || !is_contiguous()) throw TensorError(ErrorKind::Shape, "reshape: needs a contiguous tensor of the same size");
        Tensor t = alias();
        t.shape_ = shape;
        t.strides_ = contiguous_strides(shape);
        return t;
    }

  private:
    template <class U> friend class Tensor;
    std::shared_ptr<DeviceBlock> block_;
    T* data_ = nullptr;
    Shape shape_, strides_;
    int device_ = 0;
    bool is_view_ = false;  // Hpt's `parent.is_some()`

    Tensor alias() const {
        Tensor t = *this;
        t.is_view_ = true;
        return t;
    }
    Shape reduced_shape(const Axes& axes, bool keep_dims) const {
        Shape out(ndim() > 0 ? ndim() : 1);
        int32_t n = 0;
        check(hpt_hip_reduce_shape(shape_.data(), ndim(), axes.data(), (int32_t)axes.size(), keep_dims, out.data(), &n));
        out.resize(n);
        return out;
    }
    template <class O> Tensor<O> reduce(int op, const Axes& axes, bool keep_dims) const {
        Tensor<O> res = Tensor<O>::empty(reduced_shape(axes, false), device_);
        hpt_view vin = view(), vout = res.view();
        check(hpt_hip_reduce(device_, nullptr, op, &vin, axes.data(), (int32_t)axes.size(), 1, &vout));
        return keep_dims ? res.reshape(reduced_shape(axes, true)) : res;
    }
    Tensor reduce_into(int op, const Axes& axes, bool keep_dims, bool init_out, Tensor out) const {
        Tensor flat = out.reshape(reduced_shape(axes, false));  // also checks the size
        hpt_view vin = view(), vout = flat.view();
        check(hpt_hip_reduce(device_, nullptr, op, &vin, axes.data(), (int32_t)axes.size(), init_out ? 1 : 0, &vout));
        return keep_dims ? flat.reshape(reduced_shape(axes, true)) : flat;
    }
    Tensor<int64_t> argreduce(bool is_max, int64_t axis, bool keep_dims) const {
        Axes ax = {axis};
        Tensor<int64_t> res = Tensor<int64_t>::empty(reduced_shape(ax, false), device_);
        hpt_view vin = view(), vout = res.view();
        check(hpt_hip_argreduce(device_, nullptr, is_max ? 1 : 0, &vin, axis, &vout));
        return keep_dims ? res.reshape(reduced_shape(ax, true)) : res;
    }
    // (a non-float input is promoted to FloatBinaryType<T>, the entries' Output type, inside the kernel)
    FloatOut softmax_impl(bool log, int64_t axis) const {
        FloatOut res = FloatOut::empty(shape_, device_);
        hpt_view vin = view(), vout = res.view();
        check(hpt_hip_softmax(device_, nullptr, log ? 1 : 0, &vin, axis, &vout));
        return res;
    }
    Tensor binary(int op, const Tensor& rhs, Tensor* out) const {
        // predict_broadcast_shape (hpt-common/src/shape/shape_utils.rs): numpy's rule
        const int nd = std::max(ndim(), rhs.ndim());
        Shape shape(nd);
        for (int i = 0; i < nd; ++i) {
            const int64_t x = i < nd - ndim() ? 1 : shape_[i - (nd - ndim())];
            const int64_t y = i < nd - rhs.ndim() ? 1 : rhs.shape_[i - (nd - rhs.ndim())];
            if (x != y && x != 1 && y != 1) throw TensorError(ErrorKind::Shape, "broadcast failed at dim " + std::to_string(i));
            shape[i] = x == 1 ? y : x;
        }
        const Tensor a = expand(shape), b = rhs.expand(shape);
        Tensor res = out ? *out : empty(shape, device_);
        hpt_view va = a.view(), vb = b.view(), vo = res.view();
        check(hpt_hip_binary(device_, nullptr, op, &va, &vb, &vo));
        return res;
    }
};

inline int device_count() {
    int32_t n = 0;
    check(hpt_hip_device_count(&n));
    return n;
}
inline void synchronize(int device = 0) { check(hpt_hip_stream_synchronize(device, nullptr)); }

}  // namespace hpt
