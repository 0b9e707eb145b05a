"""Host-side mirror of Hpt's tensor API for the reduction / normalisation path.

`Tensor` plays the role of `hpt::Tensor<T, B, DEVICE>` (hpt/src/tensor.rs:31-37):
a shape + element strides + an already-offset data pointer over shared storage.
Two backends exist here:

  * "cpu": a host tensor over a numpy buffer. It only carries data; like the
    reference's `to_cuda` (hpt/src/backends/cpu/tensor_impls.rs:295-313) the way
    onto the device is `to_hip()`. No operator runs on it in this package.
  * "hip": device memory obtained from the caching allocator of libhpt_hip.so.
    The reduce / normalisation traits of the reference
    (hpt-traits/src/ops/reduce.rs:6-358, hpt-traits/src/ops/normalization.rs:6-64)
    are methods of the same names with the same arguments, and every one of them
    is a call into the C ABI: there is no other execution path.

Views (`permute`, `transpose`, `slice`, `__getitem__`) share storage and follow
hpt/src/backends/common/shape_manipulate.rs:144-167 and hpt-common/src/slice.rs:41-120.
"""
from __future__ import annotations

import ctypes as C
from typing import Iterable, Optional, Sequence

import numpy as np

from . import _ffi
from ._ffi import ParamError, ShapeError, check, make_view

ALIGN = 64  # every tensor's mem_layout alignment (hpt/src/lib.rs:560)


class DType:
    """hpt_dtype values and their numpy carriers (bf16 travels as uint16 bit patterns)."""

    def __init__(self, code: int, name: str, np_dtype, size: int):
        self.code, self.name, self.np_dtype, self.size = code, name, np.dtype(np_dtype), size

    def __repr__(self):
        return f"hpt.{self.name}"


bool_ = DType(0, "bool", np.bool_, 1)
i8 = DType(1, "i8", np.int8, 1)
i16 = DType(2, "i16", np.int16, 2)
i32 = DType(3, "i32", np.int32, 4)
i64 = DType(4, "i64", np.int64, 8)
u8 = DType(5, "u8", np.uint8, 1)
u16 = DType(6, "u16", np.uint16, 2)
u32 = DType(7, "u32", np.uint32, 4)
u64 = DType(8, "u64", np.uint64, 8)
f16 = DType(9, "f16", np.float16, 2)
bf16 = DType(10, "bf16", np.uint16, 2)
f32 = DType(11, "f32", np.float32, 4)
f64 = DType(12, "f64", np.float64, 8)
DTYPES = [bool_, i8, i16, i32, i64, u8, u16, u32, u64, f16, bf16, f32, f64]
_BY_NP = {d.np_dtype: d for d in DTYPES if d is not bf16}

# hpt_reduce_op
SUM, PROD, MAX, MIN, MEAN, NANSUM, NANPROD, REDUCEL1, REDUCEL2, REDUCEL3, SUM_SQUARE, LOGSUMEXP, ALL, ANY = range(14)
BIN_ADD, BIN_SUB, BIN_MUL, BIN_DIV = range(4)  # hpt_binary_op


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round float32 to bfloat16 (nearest even, NaN quieted); returns uint16 bit patterns."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x0040).astype(np.uint16)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


class _HostStorage:
    def __init__(self, arr: np.ndarray):
        self.arr = arr  # C-contiguous 1-D view keeps the buffer alive
        self.ptr = arr.ctypes.data


def _stream_key(stream) -> int:
    """A hipStream_t given as None / int / ctypes pointer -> its address (0 = the default stream)."""
    if stream is None:
        return 0
    if isinstance(stream, int):
        return stream
    return int(getattr(stream, "value", None) or 0)


class _StreamTracked:
    """Which streams have work queued that reads or writes this memory. The library's free hands a
    block to the next caller at once (include/hpt_hip.h), and the synchronous copies only wait for
    the default stream, so the owner waits for these streams itself before it frees or copies."""

    device = 0

    def _init_streams(self):
        self.pending = set()

    def touch(self, stream) -> None:
        self.pending.add(_stream_key(stream))

    def wait(self) -> None:
        """Wait for every stream that has touched this memory. A stream its owner has destroyed in the
        meantime cannot be waited for by handle: the whole device is waited for instead (a destroyed
        stream's work has either finished or is covered by that)."""
        while self.pending:
            k = self.pending.pop()
            try:
                check(_ffi.lib().hpt_hip_stream_synchronize(self.device, C.c_void_p(k) if k else None))
            except Exception:
                check(_ffi.lib().hpt_hip_device_synchronize(self.device))

    def forget_streams(self) -> None:
        """The caller has waited for (or destroyed) the streams this memory was used on."""
        self.pending.clear()


class _DeviceStorage(_StreamTracked):
    """A block owned through the library's caching allocator (hpt-allocator's Backend<B>)."""

    def __init__(self, device: int, nbytes: int, zeroed: bool = False):
        p = C.c_void_p()
        check(_ffi.lib().hpt_hip_alloc(device, nbytes, ALIGN, int(zeroed), C.byref(p)))
        self.ptr = p.value or 0
        self.nbytes, self.device = nbytes, device
        self._init_streams()

    def __del__(self):
        if not self.ptr:
            return
        try:
            self.wait()  # kernels still queued on a caller's stream may use the block
        except Exception:
            pass  # (interpreter shutdown, or the device is gone: nothing more can be waited for)
        try:
            # the block always goes back to the allocator, whatever the wait did
            _ffi.lib().hpt_hip_free(self.device, C.c_void_p(self.ptr), self.nbytes, ALIGN)
        except Exception:
            pass
        self.ptr = 0


class _RawStorage(_StreamTracked):
    """Device memory somebody else owns (Tensor.from_raw): never freed here (`should_drop = false`,
    hpt/src/backends/cuda/tensor_impls.rs; hpt-allocator/src/backend.rs:12-168)."""

    def __init__(self, device: int, ptr: int, nbytes: int):
        self.ptr, self.nbytes, self.device = ptr, nbytes, device
        self._init_streams()


def _contiguous_strides(shape: Sequence[int]):
    st, s = [0] * len(shape), 1
    for i in range(len(shape) - 1, -1, -1):
        st[i] = s
        s *= shape[i]
    return st


def _tdiv(a: int, b: int) -> int:
    """Integer division truncating toward zero (Rust's `/`)."""
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


def _touch(stream, *tensors) -> None:
    """Record that work on `stream` now uses the storage of these device tensors."""
    for t in tensors:
        st = getattr(t, "_storage", None) if t is not None else None
        if isinstance(st, _StreamTracked):
            st.touch(stream)


def _as_axes(axes) -> list:
    if isinstance(axes, (int, np.integer)):
        return [int(axes)]
    return [int(a) for a in axes]


class Tensor:
    def __init__(self, storage, ptr: int, shape, strides, dtype: DType, backend: str, device: int,
                 parent: Optional[int] = None):
        self._storage = storage
        self.ptr = ptr                      # already-offset element pointer (Pointer<T>)
        self.shape = [int(s) for s in shape]
        self.strides = [int(s) for s in strides]  # in elements
        self.dtype = dtype
        self.backend = backend
        self.device = device
        self.parent = parent                # set on views, as _Tensor.parent is

    # ---- construction / transfer --------------------------------------------
    @classmethod
    def from_numpy(cls, arr: np.ndarray, dtype: Optional[DType] = None) -> "Tensor":
        """A host ("cpu") tensor over a copy of `arr`. Pass dtype=bf16 with uint16 bit patterns."""
        arr = np.ascontiguousarray(arr)
        if dtype is None:
            dtype = _BY_NP.get(arr.dtype)
            if dtype is None:
                raise _ffi.DTypeError(_ffi.ERR_DTYPE, f"unsupported numpy dtype {arr.dtype}")
        if arr.dtype != dtype.np_dtype:
            raise _ffi.DTypeError(_ffi.ERR_DTYPE, f"{dtype} is carried by {dtype.np_dtype}, got {arr.dtype}")
        flat = arr.reshape(-1).copy()
        st = _HostStorage(flat)
        return cls(st, st.ptr, arr.shape, _contiguous_strides(arr.shape), dtype, "cpu", 0)

    @classmethod
    def empty(cls, shape, dtype: DType, device: int = 0, zeroed: bool = False) -> "Tensor":
        """TensorCreator::empty for the Hip backend (cuda/tensor_internal/normal_creation.rs:34-69)."""
        shape = [int(s) for s in shape]
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        st = _DeviceStorage(device, n * dtype.size, zeroed)
        return cls(st, st.ptr, shape, _contiguous_strides(shape), dtype, "hip", device)

    @classmethod
    def from_raw(cls, ptr: int, shape, dtype: DType, device: int = 0, strides=None) -> "Tensor":
        """Tensor::from_raw (hpt/src/backends/cpu/tensor_impls.rs:123-147, :269): a tensor over device
        memory the caller owns; dropping the tensor frees nothing. The reference takes a contiguous
        shape and asserts 64-byte alignment; here `strides` (elements) may describe any view and the
        pointer only has to be aligned to the element size: the kernels take unaligned rows."""
        if not ptr:
            raise ParamError(_ffi.ERR_PARAM, "data is null")
        if ptr % dtype.size:
            raise ParamError(_ffi.ERR_PARAM, f"data is not aligned, it must be aligned to {dtype.size}")
        shape = [int(s) for s in shape]
        strides = _contiguous_strides(shape) if strides is None else [int(s) for s in strides]
        if len(strides) != len(shape):
            raise ShapeError(_ffi.ERR_SHAPE, f"from_raw: {len(shape)} dims but {len(strides)} strides")
        lo = sum((d - 1) * s for d, s in zip(shape, strides) if s < 0 and d > 0)
        hi = sum((d - 1) * s for d, s in zip(shape, strides) if s > 0 and d > 0)
        n = 0 if 0 in shape else (hi - lo + 1)
        st = _RawStorage(device, ptr + lo * dtype.size, n * dtype.size)
        return cls(st, ptr, shape, strides, dtype, "hip", device)

    def forget(self):
        """Tensor::forget (hpt/src/backends/cuda/tensor_impls.rs:277-306): give the allocation up. Returns
        (pointer, (bytes, align)); the allocator stops tracking the block (Allocator::forget,
        hpt-allocator/src/allocators/cuda.rs:140-146) and the caller releases it with hipFree. Fails, as the
        reference does, for a view and while another tensor shares the storage; the tensor is empty after."""
        import sys
        self._require_hip("forget")
        if self.parent is not None:
            raise ParamError(_ffi.ERR_PARAM, "Can't forget tensor: tensor is a view, cannot forget")
        st = self._storage
        refs = sys.getrefcount(st) - 2  # the local name and getrefcount's own argument
        if refs > 1:
            raise ParamError(_ffi.ERR_PARAM, f"Can't forget tensor: ref_count: {refs}")
        st.wait()
        ptr, nbytes = st.ptr, st.nbytes
        if isinstance(st, _DeviceStorage):
            check(_ffi.lib().hpt_hip_forget(self.device, C.c_void_p(ptr)))
            st.ptr = 0  # its __del__ must not hand the block back to the cache
        self._storage, self.ptr, self.shape, self.strides = None, 0, [0], [1]
        return ptr, (nbytes, ALIGN)

    def allclose(self, other: "Tensor", rtol: float = 1e-5, atol: float = 1e-8) -> bool:
        """allclose of the reference (hpt/src/backends/cuda/tensor_impls.rs:259-271: both sides go to the
        host; hpt/src/backends/cpu/tensor_impls.rs:218-248: shapes must match, NaN equals NaN, infinities by
        sign, else |a - b| <= atol + rtol * |b|)."""
        if self.shape != other.shape:
            return False
        a, b = self._host_f64(), other._host_f64()
        both_nan = np.isnan(a) & np.isnan(b)
        inf = np.isinf(a) & np.isinf(b)
        with np.errstate(invalid="ignore"):
            ok = np.abs(a - b) <= atol + rtol * np.abs(b)
        ok = np.where(inf, np.sign(a) == np.sign(b), ok) | both_nan
        return bool(ok.all())

    def _host_f64(self) -> np.ndarray:
        h = self.to_cpu().numpy() if self.backend == "hip" else self.numpy()
        if self.dtype is bf16:
            h = bf16_bits_to_f32(h)
        return h.astype(np.float64)

    def size(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    @property
    def ndim(self) -> int:
        return len(self.shape)

    def is_contiguous(self) -> bool:
        """Layout::is_contiguous (hpt-common/src/layout/layout_utils.rs:363-375)."""
        expected = 1
        for d, s in zip(reversed(self.shape), reversed(self.strides)):
            if d == 0:
                continue
            if s != expected:
                return False
            expected *= d
        return True

    def to_hip(self, device: int = 0) -> "Tensor":
        """to_cuda's twin: allocate on the device, make contiguous if needed, synchronous copy."""
        if self.backend != "cpu":
            raise ParamError(_ffi.ERR_PARAM, "to_hip expects a cpu tensor")
        host = self.numpy()
        out = Tensor.empty(self.shape, self.dtype, device)
        check(_ffi.lib().hpt_hip_memcpy_h2d_sync(device, C.c_void_p(out.ptr), C.c_void_p(host.ctypes.data),
                                                 host.nbytes))
        return out

    def to_cpu(self) -> "Tensor":
        """to_cpu (hpt/src/backends/cuda/tensor_impls.rs:142-169): a view is first made contiguous ON
        THE DEVICE (:154-160), then copied back with one synchronous transfer."""
        if self.backend != "hip":
            raise ParamError(_ffi.ERR_PARAM, "to_cpu expects a hip tensor")
        src = self if (self.is_contiguous() and self.parent is None) else self.contiguous()
        arr = np.empty(self.shape, self.dtype.np_dtype)
        if arr.nbytes:
            src._storage.wait()
            check(_ffi.lib().hpt_hip_stream_synchronize(self.device, None))
            check(_ffi.lib().hpt_hip_memcpy_d2h_sync(self.device, C.c_void_p(arr.ctypes.data),
                                                     C.c_void_p(src.ptr), arr.nbytes))
        return Tensor.from_numpy(arr, self.dtype)

    def numpy(self) -> np.ndarray:
        """Contiguous numpy copy of this (possibly strided) tensor; bf16 comes back as uint16 bits."""
        if not self.size():
            return np.empty(self.shape, self.dtype.np_dtype)
        st = self._storage
        if self.backend == "cpu":
            base = st.arr
        else:
            # device: copy the whole allocation once, then gather through the strides
            raw = np.empty(st.nbytes, np.uint8)
            st.wait()
            check(_ffi.lib().hpt_hip_stream_synchronize(self.device, None))
            check(_ffi.lib().hpt_hip_memcpy_d2h_sync(self.device, C.c_void_p(raw.ctypes.data),
                                                     C.c_void_p(st.ptr), st.nbytes))
            base = raw.view(self.dtype.np_dtype)
        off = (self.ptr - st.ptr) // self.dtype.size
        if self.is_contiguous():
            return base[off:off + self.size()].reshape(self.shape).copy()
        idx = np.full(self.shape, off, dtype=np.int64)
        for ax, (d, stride) in enumerate(zip(self.shape, self.strides)):
            sh = [1] * self.ndim
            sh[ax] = d
            idx = idx + (np.arange(d, dtype=np.int64) * stride).reshape(sh)
        return base[idx]

    # ---- views -----------------------------------------------------------------
    def _view(self, ptr, shape, strides) -> "Tensor":
        return Tensor(self._storage, ptr, shape, strides, self.dtype, self.backend, self.device,
                      parent=self.parent if self.parent is not None else self.ptr)

    def permute(self, axes) -> "Tensor":
        axes = _as_axes(axes)
        if sorted(a % max(1, self.ndim) for a in axes) != list(range(self.ndim)):
            raise ShapeError(_ffi.ERR_SHAPE, f"permute: axes {axes} are not a permutation of 0..{self.ndim}")
        axes = [a % self.ndim for a in axes]
        t = Tensor(self._storage, self.ptr, [self.shape[a] for a in axes], [self.strides[a] for a in axes],
                   self.dtype, self.backend, self.device, parent=self.parent)
        return t

    def transpose(self, a: int, b: int) -> "Tensor":
        axes = list(range(self.ndim))
        axes[a], axes[b] = axes[b], axes[a]
        return self.permute(axes)

    def t(self) -> "Tensor":
        return self.permute(list(range(self.ndim))[::-1])

    def slice(self, index: Sequence) -> "Tensor":
        """slice_process (hpt-common/src/slice.rs:41-120). `index` holds (start, end, step)
        triples, one per leading dim; end=None means "to the end"."""
        BIG = 0x7FFFFFFFFFFFFFFF
        shape, strides, ptr_off = list(self.shape), list(self.strides), 0
        if len(index) > self.ndim:
            raise ShapeError(_ffi.ERR_SHAPE, f"index length is greater than the shape length, shape: {self.shape}")
        for d, (start, end, step) in enumerate(index):
            dim = self.shape[d]
            end = dim if end is None or end == BIG else end
            start = start if start >= 0 else start + dim
            end = end if end >= 0 else end + dim
            if start >= dim:
                start = dim - 1
            if end > dim:
                end = dim
            if step > 0:
                length = _tdiv(end - start + step - 1, step)
            elif step < 0:
                length = _tdiv(end - start + step + 1, step)
            else:
                length = 0
            if length > 0:
                shape[d] = length
                ptr_off += start * strides[d]
                strides[d] *= step
            else:
                shape[d] = 0
        keep = [i for i, s in enumerate(shape) if s != 0]
        return self._view(self.ptr + ptr_off * self.dtype.size, [shape[i] for i in keep],
                          [strides[i] for i in keep])

    def __getitem__(self, key) -> "Tensor":
        if not isinstance(key, tuple):
            key = (key,)
        index = []
        for d, k in enumerate(key):
            if not isinstance(k, slice):
                raise ParamError(_ffi.ERR_PARAM, "only slices are supported in __getitem__")
            step = 1 if k.step is None else k.step
            if step > 0:
                start = 0 if k.start is None else k.start
                end = None if k.stop is None else k.stop
            else:
                start = self.shape[d] - 1 if k.start is None else k.start
                end = -self.shape[d] - 1 if k.stop is None else k.stop
            index.append((start, end, step))
        return self.slice(index)

    # ---- ABI plumbing ------------------------------------------------------------
    def _require_hip(self, what: str):
        if self.backend != "hip":
            raise NotImplementedError(
                f"{what}: this package implements the Hip backend only; move the tensor with to_hip()")

    def _c_view(self):
        return make_view(self.ptr, self.shape, self.strides, self.dtype.code)

    def _reduce_shape(self, axes, keep_dims: bool):
        l = _ffi.lib()
        sh = _ffi.i64_array(self.shape)
        ax = _ffi.i64_array(axes)
        out = (C.c_int64 * max(1, self.ndim))()
        n = C.c_int32()
        check(l.hpt_hip_reduce_shape(sh, self.ndim, ax, len(axes), int(keep_dims), out, C.byref(n)))
        return [out[i] for i in range(n.value)]

    def _reduce(self, op: int, axes, keep_dims: bool, init_out: bool = True, out: "Tensor" = None,
                stream=None, static_scratch: bool = False) -> "Tensor":
        """static_scratch: go through hpt_hip_reduce_static (no device allocation inside the call;
        pass `out` as well to keep this wrapper from allocating the result)."""
        self._require_hip("reduce")
        l = _ffi.lib()
        axes = _as_axes(axes)
        od = C.c_int32()
        check(l.hpt_hip_reduce_out_dtype(op, self.dtype.code, C.byref(od)))
        out_dtype = DTYPES[od.value]
        flat_shape = self._reduce_shape(axes, False)
        final_shape = self._reduce_shape(axes, keep_dims)
        if out is None:
            res = Tensor.empty(flat_shape, out_dtype, self.device)
        else:
            if not out.is_contiguous():
                raise ShapeError(_ffi.ERR_SHAPE, "out tensor must be contiguous")
            res = Tensor(out._storage, out.ptr, flat_shape, _contiguous_strides(flat_shape), out.dtype,
                         out.backend, out.device)
            if out.size() != res.size():
                raise ShapeError(_ffi.ERR_SHAPE,
                                 f"Size mismatch: expected {res.size()}, got {out.size()}")
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        ax = _ffi.i64_array(axes)
        entry = l.hpt_hip_reduce_static if static_scratch else l.hpt_hip_reduce
        check(entry(self.device, stream, op, C.byref(vin), ax, len(axes), int(init_out), C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return Tensor(res._storage, res.ptr, final_shape, _contiguous_strides(final_shape), res.dtype, "hip",
                      self.device)

    def _argreduce(self, is_max: bool, axis, keep_dims: bool, stream=None) -> "Tensor":
        self._require_hip("argreduce")
        l = _ffi.lib()
        axes = _as_axes(axis)
        if len(axes) != 1:
            raise ParamError(_ffi.ERR_PARAM, "argmax/argmin reduce exactly one axis")
        flat_shape = self._reduce_shape(axes, False)
        final_shape = self._reduce_shape(axes, keep_dims)
        res = Tensor.empty(flat_shape, i64, self.device)
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        check(l.hpt_hip_argreduce(self.device, stream, int(is_max), C.byref(vin), axes[0], C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return Tensor(res._storage, res.ptr, final_shape, _contiguous_strides(final_shape), i64, "hip", self.device)

    # ---- NormalReduce (hpt-traits/src/ops/reduce.rs:45-176) ----------------------
    def sum(self, axes, keep_dims: bool = False, **kw):
        return self._reduce(SUM, axes, keep_dims, **kw)

    def sum_(self, axes, keep_dims: bool, init_out: bool, out: "Tensor", **kw):
        return self._reduce(SUM, axes, keep_dims, init_out=init_out, out=out, **kw)

    def prod(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(PROD, axis, keep_dims, **kw)

    def min(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(MIN, axis, keep_dims, **kw)

    def max(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(MAX, axis, keep_dims, **kw)

    def reducel1(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(REDUCEL1, axis, keep_dims, **kw)

    def sum_square(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(SUM_SQUARE, axis, keep_dims, **kw)

    # ---- EvalReduce / NormalEvalReduce (reduce.rs:179-277) -----------------------
    def all(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(ALL, axis, keep_dims, **kw)

    def any(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(ANY, axis, keep_dims, **kw)

    def nansum(self, axes, keep_dims: bool = False, **kw):
        return self._reduce(NANSUM, axes, keep_dims, **kw)

    def nansum_(self, axes, keep_dims: bool, init_out: bool, out: "Tensor", **kw):
        return self._reduce(NANSUM, axes, keep_dims, init_out=init_out, out=out, **kw)

    def nanprod(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(NANPROD, axis, keep_dims, **kw)

    # ---- FloatReduce (reduce.rs:280-358) -----------------------------------------
    def mean(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(MEAN, axis, keep_dims, **kw)

    def reducel2(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(REDUCEL2, axis, keep_dims, **kw)

    def reducel3(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(REDUCEL3, axis, keep_dims, **kw)

    def logsumexp(self, axis, keep_dims: bool = False, **kw):
        return self._reduce(LOGSUMEXP, axis, keep_dims, **kw)

    # ---- IndexReduce (reduce.rs:6-42) --------------------------------------------
    def argmax(self, axis, keep_dims: bool = False, **kw):
        return self._argreduce(True, axis, keep_dims, **kw)

    def argmin(self, axis, keep_dims: bool = False, **kw):
        return self._argreduce(False, axis, keep_dims, **kw)

    # ---- NormalizationOps (hpt-traits/src/ops/normalization.rs:6-64) ------------
    def _norm_out(self, out: Optional["Tensor"], dtype: DType) -> "Tensor":
        """The result tensor of a normalisation: fresh, or the caller's `out` (which may be `self`: the
        ABI allows a normalisation in place over one contiguous tensor)."""
        if out is None:
            return Tensor.empty(self.shape, dtype, self.device)
        out._require_hip("out")
        return out

    def _softmax(self, log: bool, axis: int, stream=None, out: Optional["Tensor"] = None) -> "Tensor":
        self._require_hip("softmax")
        # NormalizationOps::Output = Tensor<FloatBinaryType<T>>: a non-float input is promoted inside the
        # kernel (one launch, no promoted copy), as the reference promotes inside the op
        res = self._norm_out(out, self._float_binary_type())
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        check(_ffi.lib().hpt_hip_softmax(self.device, stream, int(log), C.byref(vin), int(axis), C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return res

    def softmax(self, axis: int, **kw) -> "Tensor":
        return self._softmax(False, axis, **kw)

    def log_softmax(self, axis: int, **kw) -> "Tensor":
        return self._softmax(True, axis, **kw)

    def layernorm(self, normalized_shape, gamma: Optional["Tensor"] = None, beta: Optional["Tensor"] = None,
                  eps: float = 1e-5, stream=None, residual: Optional["Tensor"] = None,
                  out: Optional["Tensor"] = None) -> "Tensor":
        self._require_hip("layernorm")
        ns = [int(s) for s in (normalized_shape if isinstance(normalized_shape, Iterable) else [normalized_shape])]
        if len(ns) > self.ndim or (ns and self.shape[self.ndim - len(ns):] != ns) or not ns:
            # the reference panics with this text (cpu/tensor_internal/normalization.rs:68-70)
            raise ShapeError(_ffi.ERR_SHAPE,
                             "normalized dims must match last dims of input tensor, "
                             f"shape: {self.shape}, normalized_shape: {ns}")
        ft = self._float_binary_type()
        if ft is not self.dtype and residual is not None:
            # (the fused add + layernorm takes float tensors; the promoted copy is kept alive by `_touch`)
            return self.astype(ft, stream=stream).layernorm(normalized_shape, gamma, beta, eps, stream=stream,
                                                            residual=residual, out=out)
        res = self._norm_out(out, ft)
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        keep = [k1, k2]
        gv = bv = None
        if gamma is not None:
            gamma._require_hip("layernorm gamma")
            gv, k = gamma._c_view()
            keep.append(k)
        if beta is not None:
            beta._require_hip("layernorm beta")
            bv, k = beta._c_view()
            keep.append(k)
        gp = C.byref(gv) if gv is not None else None
        bp = C.byref(bv) if bv is not None else None
        if residual is not None:
            residual._require_hip("layernorm residual")
            rv, k = residual._c_view()
            keep.append(k)
            check(_ffi.lib().hpt_hip_add_layernorm(self.device, stream, C.byref(vin), C.byref(rv), len(ns), gp, bp,
                                                   float(eps), C.byref(vout)))
        else:
            check(_ffi.lib().hpt_hip_layernorm(self.device, stream, C.byref(vin), len(ns), gp, bp, float(eps),
                                               C.byref(vout)))
        _touch(stream, self, res, gamma, beta, residual)
        del keep
        return res

    # ---- fused forms of what the callers do around softmax / layernorm -----------------
    def softmax_causal(self, scale: float = 1.0, causal_offset: int = 0, log: bool = False, stream=None) -> "Tensor":
        """softmax(-1) of scale * self with keys above query + causal_offset masked out: the sequence
        `scores.mul_(scaling)`, fill -inf where key > query, `softmax(-1)` of
        hpt-examples/examples/transformer/main.rs:233-246 in one pass; the masked part is never read."""
        self._require_hip("softmax_causal")
        res = Tensor.empty(self.shape, self.dtype, self.device)
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        check(_ffi.lib().hpt_hip_softmax_causal(self.device, stream, int(log), C.byref(vin), float(scale),
                                                int(causal_offset), C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return res

    def add_layernorm(self, residual: "Tensor", normalized_shape, gamma: Optional["Tensor"] = None,
                      beta: Optional["Tensor"] = None, eps: float = 1e-5, stream=None) -> "Tensor":
        """layernorm(self + residual) (hpt-examples/examples/transformer/main.rs:87-91) in one pass."""
        return self.layernorm(normalized_shape, gamma, beta, eps, stream=stream, residual=residual)

    # ---- the steps either side of the path ------------------------------------------
    def astype(self, dtype: DType, stream=None) -> "Tensor":
        """astype (hpt/src/backends/cuda/tensor_impls.rs:129-140) to a float dtype (or to the same dtype)."""
        self._require_hip("astype")
        res = Tensor.empty(self.shape, dtype, self.device)
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        check(_ffi.lib().hpt_hip_cast(self.device, stream, C.byref(vin), C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return res

    def _float_binary_type(self) -> DType:
        """FloatBinaryType<T> (hpt-types/src/type_promote.rs): the output dtype of the float-valued entries."""
        out = C.c_int32()
        check(_ffi.lib().hpt_hip_reduce_out_dtype(MEAN, self.dtype.code, C.byref(out)))
        return DTYPES[out.value]

    def contiguous(self, stream=None) -> "Tensor":
        """Contiguous::contiguous (hpt/src/backends/cuda/tensor_internal/normal_out_unary.rs:286-310):
        a new contiguous tensor with this view's elements."""
        self._require_hip("contiguous")
        res = Tensor.empty(self.shape, self.dtype, self.device)
        vin, k1 = self._c_view()
        vout, k2 = res._c_view()
        check(_ffi.lib().hpt_hip_contiguous(self.device, stream, C.byref(vin), C.byref(vout)))
        _touch(stream, self, res)
        del k1, k2
        return res

    @classmethod
    def full(cls, value, shape, dtype: DType, device: int = 0, stream=None) -> "Tensor":
        """TensorCreator::full on the device (set_val, hpt-cudakernels/src/set_val.cu:4-12). For bf16 `value`
        is a float (rounded to nearest even)."""
        res = cls.empty(shape, dtype, device)
        if dtype.name == "bf16":
            host = f32_to_bf16_bits(np.array([value], np.float32))
        else:
            host = np.array([value]).astype(dtype.np_dtype)
        v, k = res._c_view()
        check(_ffi.lib().hpt_hip_fill(device, stream, C.byref(v), C.c_void_p(host.ctypes.data)))
        _touch(stream, res)
        del k
        return res

    @classmethod
    def zeros(cls, shape, dtype: DType, device: int = 0) -> "Tensor":
        return cls.full(0, shape, dtype, device)

    @classmethod
    def ones(cls, shape, dtype: DType, device: int = 0) -> "Tensor":
        return cls.full(1, shape, dtype, device)

    def expand(self, shape) -> "Tensor":
        """ShapeManipulate::expand (hpt-common/src/layout/layout_utils.rs:107-): broadcast size-1 dims (and
        missing leading dims) to `shape` with stride 0."""
        shape = [int(x) for x in shape]
        if len(shape) < self.ndim:
            raise ShapeError(_ffi.ERR_SHAPE, f"expand: cannot expand {self.shape} to {shape}")
        pad = len(shape) - self.ndim
        strides = [0] * len(shape)
        for i, d in enumerate(shape):
            if i < pad:
                continue
            old = self.shape[i - pad]
            if old == d:
                strides[i] = self.strides[i - pad]
            elif old != 1:
                raise ShapeError(_ffi.ERR_SHAPE, f"expand: cannot broadcast {self.shape} to {shape}")
        return self._view(self.ptr, shape, strides)

    def _binary(self, op: int, rhs: "Tensor", out: Optional["Tensor"] = None, stream=None) -> "Tensor":
        self._require_hip("binary op")
        rhs._require_hip("binary op rhs")
        # predict_broadcast_shape (hpt-common/src/shape/shape_utils.rs): numpy's rule
        nd = max(self.ndim, rhs.ndim)
        sa = [1] * (nd - self.ndim) + list(self.shape)
        sb = [1] * (nd - rhs.ndim) + list(rhs.shape)
        shape = []
        for x, y in zip(sa, sb):
            if x != y and x != 1 and y != 1:
                raise ShapeError(_ffi.ERR_SHAPE, f"broadcast failed: lhs shape {self.shape}, rhs shape {rhs.shape}")
            shape.append(max(x, y) if min(x, y) != 0 else 0)
        a, b = self.expand(shape), rhs.expand(shape)
        res = out if out is not None else Tensor.empty(shape, self.dtype, self.device)
        va, k1 = a._c_view()
        vb, k2 = b._c_view()
        vo, k3 = res._c_view()
        check(_ffi.lib().hpt_hip_binary(self.device, stream, op, C.byref(va), C.byref(vb), C.byref(vo)))
        _touch(stream, self, rhs, res)
        del k1, k2, k3
        return res

    def add(self, rhs: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_ADD, rhs, **kw)

    def sub(self, rhs: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_SUB, rhs, **kw)

    def mul(self, rhs: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_MUL, rhs, **kw)

    def div(self, rhs: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_DIV, rhs, **kw)

    def add_(self, rhs: "Tensor", out: "Tensor", **kw) -> "Tensor":
        """NormalBinOps::add_ (hpt-traits/src/ops/binary.rs:34): the result goes to `out` (which may be self)."""
        return self._binary(BIN_ADD, rhs, out=out, **kw)

    def sub_(self, rhs: "Tensor", out: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_SUB, rhs, out=out, **kw)

    def mul_(self, rhs: "Tensor", out: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_MUL, rhs, out=out, **kw)

    def div_(self, rhs: "Tensor", out: "Tensor", **kw) -> "Tensor":
        return self._binary(BIN_DIV, rhs, out=out, **kw)

    __add__, __sub__, __mul__, __truediv__ = add, sub, mul, div

    def __repr__(self):
        return f"Tensor<{self.dtype.name}, {self.backend}, {self.device}>(shape={self.shape}, strides={self.strides})"


def reduce_plan(t: Tensor, op: int, axes) -> str:
    """The kernel family and launch shape the library would use (no device needed)."""
    axes = _as_axes(axes)
    v, k = t._c_view()
    buf = C.create_string_buffer(512)
    check(_ffi.lib().hpt_hip_reduce_plan(op, C.byref(v), _ffi.i64_array(axes), len(axes), buf, 512))
    del k
    return buf.value.decode()


def contiguous_plan(t: Tensor) -> str:
    """The kernel `t.contiguous()` would use (no device needed; the output is assumed 16-byte aligned)."""
    v, k = t._c_view()
    out, k2 = make_view(4096, t.shape, _contiguous_strides(t.shape), t.dtype.code)
    buf = C.create_string_buffer(512)
    check(_ffi.lib().hpt_hip_contiguous_plan(C.byref(v), C.byref(out), buf, 512))
    del k, k2
    return buf.value.decode()


def binary_plan(lhs: Tensor, rhs: Tensor) -> str:
    """The kernel `lhs.add(rhs)` (any of the four operators) would use, for operands already expanded to one
    shape (no device needed; the output is assumed 16-byte aligned)."""
    va, k1 = lhs._c_view()
    vb, k2 = rhs._c_view()
    out, k3 = make_view(4096, lhs.shape, _contiguous_strides(lhs.shape), lhs.dtype.code)
    buf = C.create_string_buffer(512)
    check(_ffi.lib().hpt_hip_binary_plan(C.byref(va), C.byref(vb), C.byref(out), buf, 512))
    del k1, k2, k3
    return buf.value.decode()


def normalize_plan(t: Tensor, axis: int = 0, n_norm_dims: int = 0) -> str:
    v, k = t._c_view()
    buf = C.create_string_buffer(512)
    check(_ffi.lib().hpt_hip_normalize_plan(C.byref(v), int(axis), int(n_norm_dims), buf, 512))
    del k
    return buf.value.decode()


def synchronize(device: int = 0, stream=None) -> None:
    check(_ffi.lib().hpt_hip_stream_synchronize(device, stream))


def device_count() -> int:
    n = C.c_int32()
    check(_ffi.lib().hpt_hip_device_count(C.byref(n)))
    return n.value
