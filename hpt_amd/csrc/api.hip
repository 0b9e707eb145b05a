// C ABI of libhpt_hip (see include/hpt_hip.h): argument validation, the device
// caching allocator, per-stream scratch, and dispatch into the kernel tables.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <memory>
#include <list>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.hpp"
#include "elementwise_entry.hpp"
#include "norm_entry.hpp"
#include "reduce_entry.hpp"

namespace hpt {

// ---- error transport ---------------------------------------------------------

static thread_local std::string g_last_error;

template <class F> static int32_t guarded(F&& f) {
    try {
        f();
        return HPT_OK;
    } catch (const Error& e) {
        g_last_error = e.msg;
        return e.code;
    } catch (const std::bad_alloc&) {
        g_last_error = "host allocation failed";
        return HPT_ERR_MEMORY;
    } catch (...) {
        g_last_error = "unknown error";
        return HPT_ERR_KERNEL;
    }
}

static void hip_check(hipError_t e, int code, const char* what) {
    if (e != hipSuccess) fail(code, "%s: %s", what, hipGetErrorString(e));
}

// Make `dev` the calling thread's device. The device count is asked for once per process and
// hipSetDevice is skipped when the thread is already there (hipGetDevice reads a thread-local of the
// runtime): on launch-bound calls the two runtime calls this saves are a measurable part of the
// host time.
static void use_device(int dev) {
    static std::atomic<int> count{-1};
    int n = count.load(std::memory_order_relaxed);
    if (n < 0) {
        hip_check(hipGetDeviceCount(&n), HPT_ERR_DEVICE, "hipGetDeviceCount");
        count.store(n, std::memory_order_relaxed);
    }
    if (dev < 0 || dev >= n) fail(HPT_ERR_DEVICE, "device %d does not exist (%d visible)", dev, n);
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != dev)
        hip_check(hipSetDevice(dev), HPT_ERR_DEVICE, "hipSetDevice");
}

// ---- device caching allocator ------------------------------------------------
// Same policy as the reference's CudaAllocator
// (hpt-allocator/src/allocators/cuda.rs:41-322, utils/allocate.rs:15-130,
// utils/deallocate.rs:11-32): blocks are keyed by their exact (size, align)
// layout; a freed block is kept in an LRU cache of layouts; evicting a layout
// releases all of its blocks; when the device is out of memory, layouts are
// evicted least-recently-used first and the allocation is retried.

struct LayoutKey {
    size_t bytes, align;
    bool operator<(const LayoutKey& o) const {
        return bytes != o.bytes ? bytes < o.bytes : align < o.align;
    }
};

struct DeviceAllocator {
    std::mutex mu;
    size_t capacity = 100;  // cached layouts; the CPU allocator's default (allocators/cpu.rs:22)
    std::list<LayoutKey> lru;  // front = most recently used
    std::map<LayoutKey, std::pair<std::list<LayoutKey>::iterator, std::vector<void*>>> cache;
    std::unordered_map<void*, LayoutKey> live;
    uint64_t device_mallocs = 0;
    size_t internal_blocks = 0;  // live blocks the library itself holds (scratch), not a caller

    size_t cached_blocks() const {
        size_t n = 0;
        for (auto& kv : cache) n += kv.second.second.size();
        return n;
    }
    void evict_one() {  // requires a non-empty cache
        LayoutKey k = lru.back();
        auto it = cache.find(k);
        for (void* p : it->second.second) (void)hipFree(p);
        cache.erase(it);
        lru.pop_back();
    }
    void* allocate(size_t bytes, size_t align) {
        LayoutKey k{bytes, align};
        auto it = cache.find(k);
        if (it != cache.end() && !it->second.second.empty()) {
            void* p = it->second.second.back();
            it->second.second.pop_back();
            lru.splice(lru.begin(), lru, it->second.first);
            if (it->second.second.empty()) {
                lru.erase(it->second.first);
                cache.erase(it);
            }
            live[p] = k;
            return p;
        }
        void* p = nullptr;
        for (;;) {
            hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
            if (e == hipSuccess) break;
            (void)hipGetLastError();  // clear the sticky error before retrying
            if (cache.empty())
                fail(HPT_ERR_MEMORY, "Failed to allocate %zu bytes on device: %s", bytes,
                     hipGetErrorString(e));
            evict_one();
        }
        ++device_mallocs;
        if (align > 1 && ((uintptr_t)p % align) != 0) {
            (void)hipFree(p);
            fail(HPT_ERR_MEMORY, "device allocation cannot satisfy alignment %zu", align);
        }
        live[p] = k;
        return p;
    }
    void deallocate(void* p, size_t bytes, size_t align) {
        auto it = live.find(p);
        if (it == live.end()) fail(HPT_ERR_MEMORY, "pointer %p was not allocated by hpt_hip_alloc", p);
        if (it->second.bytes != bytes || it->second.align != align)
            fail(HPT_ERR_MEMORY, "layout mismatch on free: allocated (%zu, %zu), freed as (%zu, %zu)",
                 it->second.bytes, it->second.align, bytes, align);
        LayoutKey k = it->second;
        live.erase(it);
        if (capacity == 0) {
            (void)hipFree(p);
            return;
        }
        auto c = cache.find(k);
        if (c == cache.end()) {
            lru.push_front(k);
            cache[k] = {lru.begin(), {p}};
            while (cache.size() > capacity) evict_one();
        } else {
            c->second.second.push_back(p);
            lru.splice(lru.begin(), lru, c->second.first);
        }
    }
    // The caller takes the block over: it leaves the table of live blocks and is not cached.
    bool forget(void* p) { return live.erase(p) != 0; }
    void clear() {
        while (!cache.empty()) evict_one();
    }
};

static std::mutex g_alloc_table_mu;
static std::map<int, DeviceAllocator*> g_allocators;

static DeviceAllocator& allocator_of(int dev) {
    std::lock_guard<std::mutex> g(g_alloc_table_mu);
    auto it = g_allocators.find(dev);
    if (it == g_allocators.end()) it = g_allocators.emplace(dev, new DeviceAllocator()).first;
    return *it->second;
}

// ---- scratch of the multi-workgroup reductions -----------------------------------
// One buffer per (device, stream), taken from the device's caching allocator (so that
// hpt_hip_cache_clear and the evict-and-retry path see it) and guarded by a lock of its own:
// calls on different streams do not wait for each other. It grows geometrically; the buffer it
// outgrows is not handed back while work that uses it may still be queued, but parked until
// hpt_hip_cache_clear, which waits for the device first. No call on the hot path frees device
// memory.

constexpr size_t kScratchAlign = 256;

struct StreamScratch {
    std::mutex mu;  // held from lookup to launch by the call that uses the buffer
    void* base = nullptr;
    size_t bytes = 0;
    std::vector<std::pair<void*, size_t>> retired;
};

static std::mutex g_scratch_table_mu;  // guards the map only
static std::map<std::pair<int, hipStream_t>, std::unique_ptr<StreamScratch>> g_scratch;

static StreamScratch& scratch_entry(int dev, hipStream_t st) {
    std::lock_guard<std::mutex> g(g_scratch_table_mu);
    auto& e = g_scratch[{dev, st}];
    if (!e) e.reset(new StreamScratch());
    return *e;
}

// Requires s.mu. Returns a buffer of at least `bytes`. Nothing in it has to start from a known
// value: every kernel that reads a scratch slot runs after the kernel that wrote it, on this stream.
static void* scratch_reserve(int dev, StreamScratch& s, size_t bytes) {
    if (!s.base || bytes > s.bytes) {
        const size_t want = std::max<size_t>({bytes, s.bytes * 2, (size_t)1 << 20});
        DeviceAllocator& a = allocator_of(dev);
        void* p;
        {
            std::lock_guard<std::mutex> g(a.mu);
            p = a.allocate(want, kScratchAlign);
            ++a.internal_blocks;
        }
        if (s.base) s.retired.emplace_back(s.base, s.bytes);
        s.base = p;
        s.bytes = want;
    }
    return s.base;
}

// Give every scratch buffer of `dev` back to its allocator. The table and every buffer of the device are
// locked BEFORE the device is waited for and stay locked until the buffers are back: a call on another thread
// that needs scratch either got its buffer earlier (its kernels are then queued, and waited for here) or
// blocks until this is over and allocates afresh. (Locks are taken table -> buffer -> allocator everywhere.)
static void scratch_release_all(int dev) {
    std::lock_guard<std::mutex> gt(g_scratch_table_mu);
    std::vector<std::unique_lock<std::mutex>> held;
    for (auto& kv : g_scratch)
        if (kv.first.first == dev) held.emplace_back(kv.second->mu);
    hip_check(hipDeviceSynchronize(), HPT_ERR_KERNEL, "hipDeviceSynchronize");
    DeviceAllocator& a = allocator_of(dev);
    for (auto& kv : g_scratch) {
        if (kv.first.first != dev) continue;
        StreamScratch& s = *kv.second;
        std::lock_guard<std::mutex> ga(a.mu);
        if (s.base) s.retired.emplace_back(s.base, s.bytes);
        for (auto& r : s.retired) {
            a.deallocate(r.first, r.second, kScratchAlign);
            --a.internal_blocks;
        }
        s.retired.clear();
        s.base = nullptr;
        s.bytes = 0;
    }
}

size_t scratch_need(const ReducePlan& p, size_t acc_size) {
    return p.split > 1 ? (size_t)p.K * p.split * acc_size : 0;
}

// ---- scratch that is never allocated (hpt_hip_reduce_static) ------------------------
// Part of the library's image on every device it runs on. In host code the array's name
// is only a handle for hipGetSymbolAddress: the device address is looked up once per
// device, with that device current, and only that address is ever handed to a kernel.
constexpr size_t kStaticScratchBytes = HPT_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static std::mutex g_static_scratch_mu;
static std::map<int, void*> g_static_scratch_ptr;

// Requires `dev` to be the current device.
static void* static_scratch_of(int dev) {
    std::lock_guard<std::mutex> g(g_static_scratch_mu);
    auto it = g_static_scratch_ptr.find(dev);
    if (it != g_static_scratch_ptr.end()) return it->second;
    void* ptr = nullptr;
    hip_check(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)), HPT_ERR_DEVICE,
              "hipGetSymbolAddress(scratch)");
    if (!ptr) fail(HPT_ERR_DEVICE, "hipGetSymbolAddress(scratch) returned a null address");
    g_static_scratch_ptr.emplace(dev, ptr);
    return ptr;
}

// ---- dispatch tables -----------------------------------------------------------

const ReduceEntry& reduce_entry_for(int e) {
    switch (e) {
        case 0: return reduce_entry<0>();
        case 1: return reduce_entry<1>();
        case 2: return reduce_entry<2>();
        case 3: return reduce_entry<3>();
        case 4: return reduce_entry<4>();
        case 5: return reduce_entry<5>();
        case 6: return reduce_entry<6>();
        case 7: return reduce_entry<7>();
        case 8: return reduce_entry<8>();
        case 9: return reduce_entry<9>();
        case 10: return reduce_entry<10>();
        case 11: return reduce_entry<11>();
        case 12: return reduce_entry<12>();
        case 13: return reduce_entry<13>();
        case 14: return reduce_entry<14>();
        case 15: return reduce_entry<15>();
        default: fail(HPT_ERR_PARAM, "invalid reduce op %d", e);
    }
}

NormLaunchFn norm_launcher_for(int kind, int dtype) {
    switch (kind) {
        case NORM_SOFTMAX: return norm_launcher<NORM_SOFTMAX>(dtype);
        case NORM_LOGSOFTMAX: return norm_launcher<NORM_LOGSOFTMAX>(dtype);
        case NORM_LAYERNORM: return norm_launcher<NORM_LAYERNORM>(dtype);
        case NORM_ADD_LAYERNORM: return norm_launcher<NORM_ADD_LAYERNORM>(dtype);
        case NORM_SOFTMAX_CAUSAL: return norm_launcher<NORM_SOFTMAX_CAUSAL>(dtype);
        case NORM_LOGSOFTMAX_CAUSAL: return norm_launcher<NORM_LOGSOFTMAX_CAUSAL>(dtype);
        default: return nullptr;
    }
}

NormLaunchFn norm_promoting_launcher_for(int kind, int in_dtype) {
    switch (kind) {
        case NORM_SOFTMAX: return norm_promoting_launcher<NORM_SOFTMAX>(in_dtype);
        case NORM_LOGSOFTMAX: return norm_promoting_launcher<NORM_LOGSOFTMAX>(in_dtype);
        case NORM_LAYERNORM: return norm_promoting_launcher<NORM_LAYERNORM>(in_dtype);
        default: return nullptr;  // the fused kinds take float inputs only
    }
}

// ---- view validation -------------------------------------------------------------

static void check_view(const hpt_view* v, const char* name, bool need_data) {
    if (!v) fail(HPT_ERR_PARAM, "%s: view is null", name);
    if (v->dtype < 0 || v->dtype >= HPT_DTYPE_COUNT)
        fail(HPT_ERR_DTYPE, "%s: invalid dtype %d", name, v->dtype);
    if (v->ndim < 0 || v->ndim > kMaxRank)
        fail(HPT_ERR_SHAPE, "%s: ndim %d outside 0..%d", name, v->ndim, kMaxRank);
    if (v->ndim > 0 && (!v->shape || !v->strides))
        fail(HPT_ERR_PARAM, "%s: shape/strides are null", name);
    int64_t n = 1;
    for (int i = 0; i < v->ndim; ++i) {
        if (v->shape[i] < 0) fail(HPT_ERR_SHAPE, "%s: negative dim %lld", name, (long long)v->shape[i]);
        n *= v->shape[i];
    }
    if (need_data && n > 0 && !v->data) fail(HPT_ERR_PARAM, "%s: data pointer is null", name);
}

static int64_t view_size(const hpt_view* v) {
    int64_t n = 1;
    for (int i = 0; i < v->ndim; ++i) n *= v->shape[i];
    return n;
}

// Layout::is_contiguous (hpt-common/src/layout/layout_utils.rs:363-375), with
// size-1 dims allowed any stride.
static bool view_contiguous(const hpt_view* v) {
    int64_t expect = 1;
    for (int i = v->ndim - 1; i >= 0; --i) {
        if (v->shape[i] == 0) return true;
        if (v->shape[i] == 1) continue;
        if (v->strides[i] != expect) return false;
        expect *= v->shape[i];
    }
    return true;
}

static void check_out(const hpt_view* out, int dtype, int64_t count, const char* name) {
    check_view(out, name, true);
    if (out->dtype != dtype)
        fail(HPT_ERR_DTYPE, "%s: dtype is %s, expected %s", name, dtype_name(out->dtype),
             dtype_name(dtype));
    if (!view_contiguous(out)) fail(HPT_ERR_SHAPE, "%s: output tensor must be contiguous", name);
    if (view_size(out) != count)
        fail(HPT_ERR_SHAPE, "%s: Size mismatch: expected %lld, got %lld", name, (long long)count,
             (long long)view_size(out));
}

// The bytes a view can touch: [lo, hi) around its data pointer.
static void view_extent(const hpt_view* v, const char** lo, const char** hi) {
    const int64_t es = (int64_t)dtype_size(v->dtype);
    int64_t below = 0, above = 0;
    for (int i = 0; i < v->ndim; ++i) {
        const int64_t span = (v->shape[i] - 1) * v->strides[i];
        if (span < 0) below += span;
        else above += span;
    }
    *lo = (const char*)v->data + below * es;
    *hi = (const char*)v->data + (above + 1) * es;
}

// `out` must not share memory with `in`. With allow_same, `out` may be `in` itself: the same
// pointer, dtype and contiguous layout, where every element is read before it is written by the
// thread that writes it. Anything else (a permuted, sliced, stepped or shifted view of out's
// buffer) would be read and written in different orders by different workgroups.
static void check_alias(const hpt_view* in, const hpt_view* out, bool allow_same, const char* what,
                        const char* in_name) {
    if (!in || !in->data || !out->data) return;
    if (view_size(in) == 0 || view_size(out) == 0) return;
    const char *ilo, *ihi, *olo, *ohi;
    view_extent(in, &ilo, &ihi);
    view_extent(out, &olo, &ohi);
    if (!(ilo < ohi && olo < ihi)) return;
    bool same = allow_same && in->data == out->data && in->dtype == out->dtype && in->ndim == out->ndim &&
                view_contiguous(in);
    for (int i = 0; same && i < in->ndim; ++i) same = in->shape[i] == out->shape[i];
    if (!same)
        fail(HPT_ERR_PARAM, "%s: out overlaps %s%s", what, in_name,
             allow_same ? " without being that very tensor (same pointer and contiguous layout)" : "");
}

static void check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) fail(HPT_ERR_KERNEL, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
}

struct ReduceCall {
    ReducePlan plan;
    const ReduceEntry* entry;
    int out_dtype;
};

static ReduceCall prepare_reduce(int entry_id, const hpt_view* in, const int64_t* axes, int naxes) {
    check_view(in, "reduce input", false);
    if (naxes < 0 || naxes > kMaxRank || (naxes > 0 && !axes))
        fail(HPT_ERR_PARAM, "reduce: bad axes argument");
    int64_t norm[kMaxRank];
    process_axes(axes, naxes, in->ndim, norm);
    if (in->ndim == 0) naxes = 0;
    ReduceCall c;
    c.entry = &reduce_entry_for(entry_id);
    c.out_dtype = entry_id < HPT_REDUCE_OP_COUNT ? reduce_out_dtype(entry_id, in->dtype) : HPT_I64;
    // an exponential per element (two-byte results take the hardware exp2: cheap), or squares in f64
    const bool heavy = (entry_id == HPT_LOGSUMEXP && dtype_size(c.out_dtype) > 2) ||
                       ((entry_id == HPT_SUM_SQUARE || entry_id == HPT_REDUCEL2) && in->dtype == HPT_F32);
    c.plan = plan_reduce(in->data, in->shape, in->strides, in->ndim, norm, naxes,
                         dtype_size(in->dtype), c.entry->acc_size[in->dtype], heavy);
    return c;
}

// use_static: the partials go to the library's static device array instead of allocated
// scratch; a plan that needs more than the array holds is refused.
static void run_reduce(int dev, void* stream, int entry_id, const hpt_view* in, const int64_t* axes,
                       int naxes, int init_out, hpt_view* out, bool use_static = false) {
    ReduceCall c = prepare_reduce(entry_id, in, axes, naxes);
    check_out(out, c.out_dtype, c.plan.K, "reduce output");
    check_alias(in, out, false, "reduce", "the input");
    if (c.plan.kind == ReduceKind::Empty) return;
    if (!in->data && c.plan.kind != ReduceKind::Identity)
        fail(HPT_ERR_PARAM, "reduce input: data pointer is null");
    if (!init_out && !(entry_id == HPT_SUM || entry_id == HPT_NANSUM))
        fail(HPT_ERR_PARAM, "init_out = 0 (accumulate into out) is only defined for sum and nansum");
    const size_t pbytes = scratch_need(c.plan, c.entry->acc_size[in->dtype]);
    if (use_static && pbytes > kStaticScratchBytes)
        fail(HPT_ERR_MEMORY,
             "reduce_static: this reduction needs %zu bytes of scratch, the static scratch holds %zu; "
             "use hpt_hip_reduce",
             pbytes, kStaticScratchBytes);
    use_device(dev);
    hipStream_t st = (hipStream_t)stream;
    ReduceLaunchFn fn = c.entry->launch[in->dtype];
    if (pbytes && use_static) {
        ReduceScratch sc;
        sc.partial = static_scratch_of(dev);
        fn(c.plan, in->data, out->data, sc, st, init_out);
        check_launch("reduce_static");
    } else if (pbytes) {
        StreamScratch& s = scratch_entry(dev, st);
        std::lock_guard<std::mutex> g(s.mu);
        ReduceScratch sc;
        sc.partial = scratch_reserve(dev, s, pbytes);
        fn(c.plan, in->data, out->data, sc, st, init_out);
        check_launch("reduce");
    } else {
        fn(c.plan, in->data, out->data, ReduceScratch{}, st, init_out);
        check_launch("reduce");
    }
}

struct NormCall {
    NormPlan plan;
    NormArgs args;
};

// Output dtype of the normalisations: FloatBinaryType<T> (the input's own dtype for floats).
static int norm_out_dtype(int in_dtype) { return reduce_out_dtype(HPT_MEAN, in_dtype); }

// A non-float input is promoted inside the kernel; the plan is made for the output's element size and
// cut down to what the promoting kernel runs. `float_only`: the fused kinds.
static NormCall prepare_norm(const hpt_view* in, const void* out_data, int64_t axis, int n_norm_dims,
                             bool float_only = false) {
    check_view(in, "normalize input", false);
    if (float_only && !is_float_dtype(in->dtype))
        fail(HPT_ERR_DTYPE, "this fused normalisation needs a float dtype, got %s", dtype_name(in->dtype));
    if (in->ndim == 0) fail(HPT_ERR_SHAPE, "normalize: input has no dimensions");
    if (n_norm_dims <= 0) {
        int64_t a = axis;
        int64_t na;
        process_axes(&a, 1, in->ndim, &na);
        axis = na;
    } else if (n_norm_dims > in->ndim) {
        fail(HPT_ERR_SHAPE, "layernorm: %d normalized dims but input has %d", n_norm_dims, in->ndim);
    }
    NormCall c;
    c.plan = plan_normalize(in->data, out_data, in->shape, in->strides, in->ndim, axis, n_norm_dims,
                            dtype_size(norm_out_dtype(in->dtype)), float_only);
    if (!is_float_dtype(in->dtype)) restrict_to_row_stream(c.plan);
    NormArgs& a = c.args;
    memset(&a, 0, sizeof a);
    a.in = in->data;
    a.out = const_cast<void*>(out_data);
    a.kept_in = c.plan.kept_in;
    a.kept_out = c.plan.kept_out;
    a.norm_in = c.plan.norm_in;
    a.rows = c.plan.rows;
    a.cols = c.plan.cols;
    a.sa = c.plan.norm_in.n == 1 ? c.plan.norm_in.stride[0] : 0;
    a.out_axis_stride = c.plan.out_axis_stride;
    return c;
}

// Launch a normalisation; plans that need scratch (partial row statistics) get
// the per-stream buffer, held under its lock from lookup to launch.
static void launch_norm(int dev, hipStream_t st, NormLaunchFn fn, NormCall& c, const char* what) {
    if (c.plan.scratch_bytes) {
        StreamScratch& s = scratch_entry(dev, st);
        std::lock_guard<std::mutex> g(s.mu);
        c.args.scratch = scratch_reserve(dev, s, c.plan.scratch_bytes);
        fn(c.plan, c.args, st);
        check_launch(what);
    } else {
        fn(c.plan, c.args, st);
        check_launch(what);
    }
}

}  // namespace hpt

using namespace hpt;

extern "C" {

const char* hpt_hip_last_error(void) { return g_last_error.c_str(); }

size_t hpt_hip_dtype_size(int32_t dtype) { return dtype_size(dtype); }

int32_t hpt_hip_device_count(int32_t* n) {
    return guarded([&] {
        if (!n) fail(HPT_ERR_PARAM, "device_count: null output");
        int c = 0;
        hip_check(hipGetDeviceCount(&c), HPT_ERR_DEVICE, "hipGetDeviceCount");
        *n = c;
    });
}

int32_t hpt_hip_alloc(int32_t dev, size_t bytes, size_t align, int32_t zeroed, void** out) {
    return guarded([&] {
        if (!out) fail(HPT_ERR_PARAM, "alloc: null output");
        if (align == 0 || (align & (align - 1))) fail(HPT_ERR_PARAM, "alloc: align %zu is not a power of two", align);
        use_device(dev);
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        void* p = a.allocate(bytes, align);
        if (zeroed && bytes) {
            hipError_t e = hipMemset(p, 0, bytes);
            if (e != hipSuccess) {
                a.deallocate(p, bytes, align);
                hip_check(e, HPT_ERR_MEMORY, "hipMemset");
            }
        }
        *out = p;
    });
}

int32_t hpt_hip_free(int32_t dev, void* p, size_t bytes, size_t align) {
    return guarded([&] {
        if (!p) return;
        use_device(dev);
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        a.deallocate(p, bytes, align);
    });
}

int32_t hpt_hip_forget(int32_t dev, void* p) {
    return guarded([&] {
        if (!p) return;
        use_device(dev);  // (validates `dev`, as hpt_hip_free does)
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        (void)a.forget(p);  // a pointer the allocator does not know is left alone, as in the reference
    });
}

int32_t hpt_hip_cache_resize(int32_t dev, size_t entries) {
    return guarded([&] {
        use_device(dev);
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        a.capacity = entries;
        while (a.cache.size() > a.capacity) a.evict_one();
    });
}

int32_t hpt_hip_cache_clear(int32_t dev) {
    return guarded([&] {
        use_device(dev);
        // the scratch buffers go back first (work that uses them may still be queued: waited for inside)
        scratch_release_all(dev);
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        a.clear();
    });
}

int32_t hpt_hip_alloc_stats(int32_t dev, uint64_t* live_blocks, uint64_t* cached_blocks,
                            uint64_t* device_mallocs) {
    return guarded([&] {
        DeviceAllocator& a = allocator_of(dev);
        std::lock_guard<std::mutex> g(a.mu);
        if (live_blocks) *live_blocks = a.live.size() - a.internal_blocks;
        if (cached_blocks) *cached_blocks = a.cached_blocks();
        if (device_mallocs) *device_mallocs = a.device_mallocs;
    });
}

int32_t hpt_hip_memcpy_h2d_sync(int32_t dev, void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        if (!bytes) return;
        if (!dst || !src) fail(HPT_ERR_PARAM, "memcpy: null pointer");
        use_device(dev);
        hip_check(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), HPT_ERR_DEVICE, "hipMemcpy(h2d)");
    });
}

int32_t hpt_hip_memcpy_d2h_sync(int32_t dev, void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        if (!bytes) return;
        if (!dst || !src) fail(HPT_ERR_PARAM, "memcpy: null pointer");
        use_device(dev);
        hip_check(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), HPT_ERR_DEVICE, "hipMemcpy(d2h)");
    });
}

int32_t hpt_hip_memcpy_d2d_sync(int32_t dev, void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        if (!bytes) return;
        if (!dst || !src) fail(HPT_ERR_PARAM, "memcpy: null pointer");
        use_device(dev);
        hip_check(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice), HPT_ERR_DEVICE, "hipMemcpy(d2d)");
    });
}

int32_t hpt_hip_stream_synchronize(int32_t dev, void* stream) {
    return guarded([&] {
        use_device(dev);
        hip_check(hipStreamSynchronize((hipStream_t)stream), HPT_ERR_KERNEL, "hipStreamSynchronize");
    });
}

int32_t hpt_hip_device_synchronize(int32_t dev) {
    return guarded([&] {
        use_device(dev);
        hip_check(hipDeviceSynchronize(), HPT_ERR_KERNEL, "hipDeviceSynchronize");
    });
}

int32_t hpt_hip_process_axes(const int64_t* axes, int32_t naxes, int32_t ndim, int64_t* out) {
    return guarded([&] {
        if (naxes < 0 || (naxes > 0 && (!axes || !out))) fail(HPT_ERR_PARAM, "process_axes: bad arguments");
        process_axes(axes, naxes, ndim, out);
    });
}

int32_t hpt_hip_reduce_shape(const int64_t* shape, int32_t ndim, const int64_t* axes, int32_t naxes,
                             int32_t keep_dims, int64_t* out_shape, int32_t* out_ndim) {
    return guarded([&] {
        if (ndim < 0 || ndim > kMaxRank || naxes < 0 || naxes > kMaxRank || !out_shape || !out_ndim)
            fail(HPT_ERR_PARAM, "reduce_shape: bad arguments");
        int64_t norm[kMaxRank];
        process_axes(axes, naxes, ndim, norm);
        bool red[kMaxRank] = {};
        if (ndim > 0)
            for (int i = 0; i < naxes; ++i) red[norm[i]] = true;
        int n = 0;
        for (int i = 0; i < ndim; ++i) {
            if (red[i]) {
                if (keep_dims) out_shape[n++] = 1;
            } else {
                out_shape[n++] = shape[i];
            }
        }
        if (n == 0) out_shape[n++] = 1;
        *out_ndim = n;
    });
}

int32_t hpt_hip_reduce_out_dtype(int32_t op, int32_t in_dtype, int32_t* out_dtype) {
    return guarded([&] {
        if (!out_dtype) fail(HPT_ERR_PARAM, "reduce_out_dtype: null output");
        if (op < 0 || op >= HPT_REDUCE_OP_COUNT) fail(HPT_ERR_PARAM, "invalid reduce op %d", op);
        *out_dtype = reduce_out_dtype(op, in_dtype);
    });
}

int32_t hpt_hip_reduce_plan(int32_t op, const hpt_view* in, const int64_t* axes, int32_t naxes,
                            char* buf, size_t buflen) {
    return guarded([&] {
        if (!buf || !buflen) fail(HPT_ERR_PARAM, "reduce_plan: no buffer");
        if (op < 0 || op >= kReduceEntryCount) fail(HPT_ERR_PARAM, "invalid reduce op %d", op);
        ReduceCall c = prepare_reduce(op, in, axes, naxes);
        snprintf(buf, buflen, "%s", describe(c.plan).c_str());
    });
}

int32_t hpt_hip_normalize_plan(const hpt_view* in, int64_t axis, int32_t n_norm_dims, char* buf,
                               size_t buflen) {
    return guarded([&] {
        if (!buf || !buflen) fail(HPT_ERR_PARAM, "normalize_plan: no buffer");
        NormCall c = prepare_norm(in, nullptr, axis, n_norm_dims);
        snprintf(buf, buflen, "%s", describe(c.plan).c_str());
    });
}

int32_t hpt_hip_reduce(int32_t dev, void* stream, int32_t op, const hpt_view* in, const int64_t* axes,
                       int32_t naxes, int32_t init_out, hpt_view* out) {
    return guarded([&] {
        if (op < 0 || op >= HPT_REDUCE_OP_COUNT) fail(HPT_ERR_PARAM, "invalid reduce op %d", op);
        run_reduce(dev, stream, op, in, axes, naxes, init_out, out);
    });
}

int32_t hpt_hip_reduce_static(int32_t dev, void* stream, int32_t op, const hpt_view* in, const int64_t* axes,
                              int32_t naxes, int32_t init_out, hpt_view* out) {
    return guarded([&] {
        if (op < 0 || op >= HPT_REDUCE_OP_COUNT) fail(HPT_ERR_PARAM, "invalid reduce op %d", op);
        run_reduce(dev, stream, op, in, axes, naxes, init_out, out, true);
    });
}

int32_t hpt_hip_argreduce(int32_t dev, void* stream, int32_t is_max, const hpt_view* in, int64_t axis,
                          hpt_view* out) {
    return guarded([&] {
        check_view(in, "argreduce input", false);
        if (in->ndim == 0) fail(HPT_ERR_SHAPE, "argreduce: input has no dimensions");
        int64_t na;
        process_axes(&axis, 1, in->ndim, &na);
        if (in->shape[na] > INT32_MAX)
            fail(HPT_ERR_SHAPE, "argreduce: axis of %lld elements exceeds 2^31-1", (long long)in->shape[na]);
        run_reduce(dev, stream, is_max ? kArgMaxEntry : kArgMinEntry, in, &na, 1, 1, out);
    });
}

int32_t hpt_hip_softmax(int32_t dev, void* stream, int32_t log, const hpt_view* in, int64_t axis,
                        hpt_view* out) {
    return guarded([&] {
        check_view(in, "softmax input", true);
        check_out(out, norm_out_dtype(in->dtype), view_size(in), "softmax output");
        check_alias(in, out, true, "softmax", "the input");
        NormCall c = prepare_norm(in, out->data, axis, 0);
        if (c.plan.kind == NormKind::Empty) return;
        const int kind = log ? NORM_LOGSOFTMAX : NORM_SOFTMAX;
        NormLaunchFn fn = is_float_dtype(in->dtype) ? norm_launcher_for(kind, in->dtype)
                                                    : norm_promoting_launcher_for(kind, in->dtype);
        if (!fn) fail(HPT_ERR_DTYPE, "softmax: unsupported dtype %s", dtype_name(in->dtype));
        use_device(dev);
        launch_norm(dev, (hipStream_t)stream, fn, c, "softmax");
    });
}

// layernorm, optionally of (in + residual)
static void run_layernorm(int dev, void* stream, const hpt_view* in, const hpt_view* residual, int n_norm_dims,
                          const hpt_view* gamma, const hpt_view* beta, double eps, hpt_view* out) {
    check_view(in, "layernorm input", true);
    if (n_norm_dims <= 0) fail(HPT_ERR_SHAPE, "layernorm: normalized_shape must not be empty");
    const int odt = norm_out_dtype(in->dtype);
    check_out(out, odt, view_size(in), "layernorm output");
    check_alias(in, out, true, "layernorm", "the input");
    NormCall c = prepare_norm(in, out->data, 0, n_norm_dims, residual != nullptr);
    const hpt_view* gb[2] = {gamma, beta};
    const char* names[2] = {"layernorm gamma", "layernorm beta"};
    for (int k = 0; k < 2; ++k) {
        if (!gb[k]) continue;
        check_view(gb[k], names[k], true);
        if (gb[k]->dtype != odt)
            fail(HPT_ERR_DTYPE, "%s: dtype is %s, expected %s", names[k], dtype_name(gb[k]->dtype),
                 dtype_name(odt));
        if (!view_contiguous(gb[k])) fail(HPT_ERR_SHAPE, "%s: must be contiguous", names[k]);
        check_alias(gb[k], out, false, "layernorm", k == 0 ? "gamma" : "beta");
        // shape must equal the normalised dims (leading 1s aside)
        if (view_size(gb[k]) != c.plan.cols && c.plan.kind != NormKind::Empty)
            fail(HPT_ERR_SHAPE, "%s: Size mismatch: expected %lld, got %lld", names[k],
                 (long long)c.plan.cols, (long long)view_size(gb[k]));
    }
    if (residual) {
        check_view(residual, "layernorm residual", true);
        if (residual->dtype != in->dtype)
            fail(HPT_ERR_DTYPE, "layernorm residual: dtype is %s, expected %s", dtype_name(residual->dtype),
                 dtype_name(in->dtype));
        if (!view_contiguous(residual)) fail(HPT_ERR_SHAPE, "layernorm residual: must be contiguous");
        bool same = residual->ndim == in->ndim;
        for (int i = 0; same && i < in->ndim; ++i) same = residual->shape[i] == in->shape[i];
        if (!same) fail(HPT_ERR_SHAPE, "layernorm residual: shape differs from the input's");
        check_alias(residual, out, true, "layernorm", "the residual");
    }
    if (c.plan.kind == NormKind::Empty) return;
    c.args.gamma = gamma ? gamma->data : nullptr;
    c.args.beta = beta ? beta->data : nullptr;
    c.args.residual = residual ? residual->data : nullptr;
    c.args.eps = eps;
    // the fused form runs on the row kernels only
    if (residual && (c.plan.kind == NormKind::Transposed || c.plan.kind == NormKind::TransposedTile))
        demote_to_generic(c.plan);
    // shifted rows: the residual's rows must be misaligned like the output's
    if (c.plan.shift && residual && (((uintptr_t)residual->data ^ (uintptr_t)out->data) & 15) != 0) demote_to_generic(c.plan);
    // vector loads of gamma / beta / residual need 16-byte alignment too (the shifted streaming
    // kernel reads gamma / beta element by element and the residual with the rows' own shift)
    if (c.plan.vec > 1 && !c.plan.shift &&
        (((uintptr_t)c.args.gamma | (uintptr_t)c.args.beta | (uintptr_t)c.args.residual) % 16) != 0)
        demote_to_generic(c.plan);
    NormLaunchFn fn = is_float_dtype(in->dtype)
                          ? norm_launcher_for(residual ? NORM_ADD_LAYERNORM : NORM_LAYERNORM, in->dtype)
                          : norm_promoting_launcher_for(NORM_LAYERNORM, in->dtype);
    if (!fn) fail(HPT_ERR_DTYPE, "layernorm: unsupported dtype %s", dtype_name(in->dtype));
    use_device(dev);
    launch_norm(dev, (hipStream_t)stream, fn, c, "layernorm");
}

int32_t hpt_hip_layernorm(int32_t dev, void* stream, const hpt_view* in, int32_t n_norm_dims,
                          const hpt_view* gamma, const hpt_view* beta, double eps, hpt_view* out) {
    return guarded([&] { run_layernorm(dev, stream, in, nullptr, n_norm_dims, gamma, beta, eps, out); });
}

int32_t hpt_hip_add_layernorm(int32_t dev, void* stream, const hpt_view* in, const hpt_view* residual,
                              int32_t n_norm_dims, const hpt_view* gamma, const hpt_view* beta, double eps,
                              hpt_view* out) {
    return guarded([&] {
        if (!residual) fail(HPT_ERR_PARAM, "add_layernorm: residual is null");
        run_layernorm(dev, stream, in, residual, n_norm_dims, gamma, beta, eps, out);
    });
}

int32_t hpt_hip_softmax_causal(int32_t dev, void* stream, int32_t log, const hpt_view* in, double scale,
                               int64_t causal_offset, hpt_view* out) {
    return guarded([&] {
        check_view(in, "softmax_causal input", true);
        check_out(out, in->dtype, view_size(in), "softmax_causal output");
        check_alias(in, out, true, "softmax_causal", "the input");
        if (in->ndim < 2) fail(HPT_ERR_SHAPE, "softmax_causal: needs at least 2 dims (queries x keys)");
        NormCall c = prepare_norm(in, out->data, in->ndim - 1, 0, true);
        if (c.plan.kind == NormKind::Empty) return;
        if (c.plan.kind == NormKind::Transposed || c.plan.kind == NormKind::TransposedTile ||
            c.plan.kind == NormKind::ColSplit || c.plan.kind == NormKind::RowSplit || c.plan.kind == NormKind::ColReg)
            demote_to_generic(c.plan);
        c.args.scale = scale;
        c.args.q_rows = in->shape[in->ndim - 2];
        c.args.causal_offset = causal_offset;
        NormLaunchFn fn = norm_launcher_for(log ? NORM_LOGSOFTMAX_CAUSAL : NORM_SOFTMAX_CAUSAL, in->dtype);
        if (!fn) fail(HPT_ERR_DTYPE, "softmax_causal: unsupported dtype %s", dtype_name(in->dtype));
        use_device(dev);
        launch_norm(dev, (hipStream_t)stream, fn, c, "softmax_causal");
    });
}

// ---- the steps either side of the path ------------------------------------------------

static void check_same_shape(const hpt_view* a, const hpt_view* b, const char* what) {
    bool same = a->ndim == b->ndim;
    for (int i = 0; same && i < a->ndim; ++i) same = a->shape[i] == b->shape[i];
    if (!same) fail(HPT_ERR_SHAPE, "%s: shapes differ", what);
}

static EwPlan prepare_copy(const hpt_view* in, const hpt_view* out) {
    check_view(in, "contiguous input", true);
    check_out(out, in->dtype, view_size(in), "contiguous output");
    check_same_shape(in, out, "contiguous");
    check_alias(in, out, false, "contiguous", "the input");
    const void* datas[1] = {in->data};
    const int64_t* strides[1] = {in->strides};
    return plan_elementwise(out->data, in->shape, in->ndim, 1, datas, strides, dtype_size(in->dtype), true);
}

int32_t hpt_hip_contiguous(int32_t dev, void* stream, const hpt_view* in, hpt_view* out) {
    return guarded([&] {
        const EwPlan p = prepare_copy(in, out);
        if (p.kind == EwKind::Empty) return;
        use_device(dev);
        launch_strided_copy(in->dtype, p, out->data, in->data, (hipStream_t)stream);
        check_launch("contiguous");
    });
}

int32_t hpt_hip_contiguous_plan(const hpt_view* in, const hpt_view* out, char* buf, size_t buflen) {
    return guarded([&] {
        if (!buf || !buflen) fail(HPT_ERR_PARAM, "contiguous_plan: no buffer");
        snprintf(buf, buflen, "%s", describe(prepare_copy(in, out)).c_str());
    });
}

int32_t hpt_hip_cast(int32_t dev, void* stream, const hpt_view* in, hpt_view* out) {
    return guarded([&] {
        check_view(in, "cast input", true);
        check_view(out, "cast output", true);
        if (!view_contiguous(out)) fail(HPT_ERR_SHAPE, "cast output: output tensor must be contiguous");
        check_same_shape(in, out, "cast");
        check_alias(in, out, false, "cast", "the input");
        if (in->dtype == out->dtype) {
            const EwPlan p = prepare_copy(in, out);
            if (p.kind == EwKind::Empty) return;
            use_device(dev);
            launch_strided_copy(in->dtype, p, out->data, in->data, (hipStream_t)stream);
            check_launch("cast");
            return;
        }
        const size_t es = std::max(dtype_size(in->dtype), dtype_size(out->dtype));
        const void* datas[1] = {in->data};
        const int64_t* strides[1] = {in->strides};
        const EwPlan p = plan_elementwise(out->data, in->shape, in->ndim, 1, datas, strides, es, false);
        if (p.kind == EwKind::Empty) return;
        use_device(dev);
        launch_cast(in->dtype, out->dtype, p, out->data, in->data, (hipStream_t)stream);
        check_launch("cast");
    });
}

int32_t hpt_hip_fill(int32_t dev, void* stream, hpt_view* out, const void* value) {
    return guarded([&] {
        check_view(out, "fill output", true);
        if (!view_contiguous(out)) fail(HPT_ERR_SHAPE, "fill output: output tensor must be contiguous");
        if (!value) fail(HPT_ERR_PARAM, "fill: value pointer is null");
        const int64_t n = view_size(out);
        if (n == 0) return;
        use_device(dev);
        launch_fill(out->dtype, out->data, n, value, (hipStream_t)stream);
        check_launch("fill");
    });
}

// Argument checks of a binary op and the plan its kernels run.
static EwPlan prepare_binary(const hpt_view* lhs, const hpt_view* rhs, const hpt_view* out) {
    check_view(lhs, "binary lhs", true);
    check_view(rhs, "binary rhs", true);
    if (lhs->dtype != rhs->dtype)
        fail(HPT_ERR_DTYPE, "binary: operands must share one dtype, got %s and %s", dtype_name(lhs->dtype),
             dtype_name(rhs->dtype));
    check_out(out, lhs->dtype, view_size(lhs), "binary output");
    check_same_shape(lhs, out, "binary lhs / out");
    check_same_shape(rhs, out, "binary rhs / out");
    // The output may be one of the operands (in place) but must not overlap one otherwise:
    // every element is read before it is written only when the two walk the same addresses.
    check_alias(lhs, out, true, "binary", "lhs");
    check_alias(rhs, out, true, "binary", "rhs");
    const void* datas[2] = {lhs->data, rhs->data};
    const int64_t* strides[2] = {lhs->strides, rhs->strides};
    return plan_elementwise(out->data, out->shape, out->ndim, 2, datas, strides, dtype_size(out->dtype), true);
}

int32_t hpt_hip_binary(int32_t dev, void* stream, int32_t op, const hpt_view* lhs, const hpt_view* rhs,
                       hpt_view* out) {
    return guarded([&] {
        const EwPlan p = prepare_binary(lhs, rhs, out);
        if (p.kind == EwKind::Empty) return;
        use_device(dev);
        launch_binary(op, out->dtype, p, out->data, lhs->data, rhs->data, (hipStream_t)stream);
        check_launch("binary");
    });
}

int32_t hpt_hip_binary_plan(const hpt_view* lhs, const hpt_view* rhs, const hpt_view* out, char* buf, size_t buflen) {
    return guarded([&] {
        if (!buf || !buflen) fail(HPT_ERR_PARAM, "binary_plan: no buffer");
        snprintf(buf, buflen, "%s", describe(prepare_binary(lhs, rhs, out)).c_str());
    });
}

}  // extern "C"
