"""``tv``: the tensor handle and device backend of the operator API, on HIP.

Mirrors the Python face of the reference's ``cumm.tensorview``
(cumm/tensorview/__init__.py:40-62 dtype constants, :659-811 factories;
Tensor methods bound in cumm/tensorview_bind.py:585-760) with device memory
managed through the C ABI of libcummhip.so (hipMalloc / hipMemcpyAsync /
hipMemsetAsync) instead of the CUDA runtime
(include/tensorview/tensor.h:181-330, 1395, 1525-1766 of the reference).
"""
from typing import List, Optional, Sequence, Union

import ctypes
import numpy as np

from .. import _capi
from . import gemm  # noqa: F401  (tv.gemm.*, as in the reference)


def _prod(shape) -> int:
    """Product of the extents (1 for no extents); plain Python integers: this runs on every call of an operator."""
    n = 1
    for v in shape:
        n *= int(v)
    return n


# tv::DType values are ABI: include/tensorview/dtypes.h:39-64 of the reference
bool_ = 5
float16 = 7
float32 = 0
float64 = 4
int8 = 3
int16 = 2
int32 = 1
int64 = 8
uint8 = 6
uint16 = 9
uint32 = 10
uint64 = 11
bfloat16 = 12
tf32 = 13
custom16 = 100
custom32 = 101
custom48 = 102
custom64 = 103
custom80 = 104
custom96 = 105
custom128 = 106
unknown = -1

NPDTYPE_TO_TENSOR_MAP = {
    np.dtype(np.float32): float32,
    np.dtype(np.int32): int32,
    np.dtype(np.int16): int16,
    np.dtype(np.int8): int8,
    np.dtype(np.float64): float64,
    np.dtype(np.bool_): bool_,
    np.dtype(np.uint8): uint8,
    np.dtype(np.float16): float16,
    np.dtype(np.int64): int64,
    np.dtype(np.uint16): uint16,
    np.dtype(np.uint32): uint32,
    np.dtype(np.uint64): uint64,
}
TENSOR_TO_NPDTYPE_MAP = {v: k for k, v in NPDTYPE_TO_TENSOR_MAP.items()}
TENSOR_TO_NPDTYPE_MAP[tf32] = np.dtype(np.float32)

_ITEMSIZE = {bool_: 1, float16: 2, float32: 4, float64: 8, int8: 1, int16: 2, int32: 4, int64: 8,
             uint8: 1, uint16: 2, uint32: 4, uint64: 8, bfloat16: 2, tf32: 4, custom16: 2,
             custom32: 4, custom48: 6, custom64: 8, custom80: 10, custom96: 12, custom128: 16}
ALL_TV_TENSOR_DTYPES = set(_ITEMSIZE)

# numpy has no bfloat16: host views of bf16 tensors are uint16 bit patterns
_HOST_VIEW_DTYPE = dict(TENSOR_TO_NPDTYPE_MAP)
_HOST_VIEW_DTYPE[bfloat16] = np.dtype(np.uint16)


def tvdtype_itemsize(dtype: int) -> int:
    return _ITEMSIZE[dtype]


def tvdtype_bitsize(dtype: int) -> int:
    return _ITEMSIZE[dtype] * 8


def _to_tv_dtype(dtype) -> int:
    if isinstance(dtype, (int, np.integer)) and not isinstance(dtype, bool):
        assert int(dtype) in ALL_TV_TENSOR_DTYPES, dtype
        return int(dtype)
    return NPDTYPE_TO_TENSOR_MAP[np.dtype(dtype)]


class Context:
    """Stream holder (tv::Context, include/tensorview/contexts/core.h:429-500)."""

    def __init__(self):
        self._stream = 0
        self._owned = False

    def create_cuda_stream(self):
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().cumm_hip_stream_create(ctypes.byref(out)))
        self._stream = out.value or 0
        self._owned = True
        return self

    def set_cuda_stream(self, stream: int):
        self._stream = int(stream)
        self._owned = False

    def has_cuda_stream(self) -> bool:
        return self._stream != 0

    def cuda_stream_int(self) -> int:
        return self._stream

    def synchronize_stream(self):
        _capi.check(_capi.lib().cumm_hip_stream_synchronize(self._stream))

    def __del__(self):
        if getattr(self, "_owned", False) and self._stream:
            try:
                _capi.lib().cumm_hip_stream_destroy(self._stream)
            except Exception:
                pass


class _DeviceStorage:
    """One hipMalloc allocation, freed with its last tensor (shared ownership as
    tv::TensorStorage, include/tensorview/tensor.h:181-330)."""

    def __init__(self, nbytes: int, device: int):
        self.nbytes = nbytes
        self.device = device
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().cumm_hip_malloc(ctypes.byref(out), max(nbytes, 1)))
        self.ptr = out.value or 0
        self.owned = True

    def __del__(self):
        if getattr(self, "owned", False) and self.ptr:
            try:
                _capi.lib().cumm_hip_free(self.ptr)
            except Exception:
                pass
            self.ptr = 0


class _BlobStorage:
    """Memory owned by someone else (tv::from_blob never frees, tensor.h:286-288)."""

    def __init__(self, ptr: int, nbytes: int, device: int, keepalive=None):
        self.ptr = int(ptr)
        self.nbytes = nbytes
        self.device = device
        self.keepalive = keepalive
        self.owned = False


class _HostStorage:
    def __init__(self, arr: np.ndarray):
        self.arr = arr  # 1-D uint8, C contiguous
        self.nbytes = arr.nbytes
        self.device = -1
        self.ptr = arr.ctypes.data


def _contig_stride(shape: Sequence[int]) -> List[int]:
    stride = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        stride[i] = stride[i + 1] * int(shape[i + 1])
    return stride


class Tensor:
    """tv::Tensor: shape/stride/dtype/device over shared storage."""

    def __init__(self, shape: Optional[Sequence[int]] = None, dtype: int = float32,
                 device: int = -1, pinned: bool = False, managed: bool = False):
        self._dtype = int(dtype)
        self._offset = 0  # bytes
        if shape is None:
            self._shape, self._stride, self._storage = [], [], None
            self._dtype = unknown if dtype == float32 else int(dtype)
            return
        self._shape = [int(s) for s in shape]
        self._stride = _contig_stride(self._shape)
        nbytes = _prod(self._shape) * _ITEMSIZE[self._dtype]
        if device == -1:
            self._storage = _HostStorage(np.empty(nbytes, dtype=np.uint8))
        else:
            self._storage = _DeviceStorage(nbytes, device)

    # ---- construction helpers
    @classmethod
    def _make(cls, storage, shape, stride, dtype, offset):
        t = cls.__new__(cls)
        t._storage, t._shape, t._stride = storage, [int(s) for s in shape], [int(s) for s in stride]
        t._dtype, t._offset = int(dtype), int(offset)
        return t

    # ---- queries
    @property
    def shape(self) -> List[int]:
        return list(self._shape)

    @property
    def stride(self) -> List[int]:
        return list(self._stride)

    @property
    def dtype(self) -> int:
        return self._dtype

    @property
    def device(self) -> int:
        return -1 if self._storage is None else self._storage.device

    @property
    def ndim(self) -> int:
        return len(self._shape)

    @property
    def size(self) -> int:
        return _prod(self._shape) if self._storage is not None else 0

    @property
    def itemsize(self) -> int:
        return _ITEMSIZE[self._dtype]

    def dim(self, i: int) -> int:
        return self._shape[i]

    def empty(self) -> bool:
        return self._storage is None or self.size == 0

    def bytesize(self) -> int:
        return self.size * self.itemsize

    nbytes = property(lambda self: self.bytesize())

    def storage_bytesize(self) -> int:
        return 0 if self._storage is None else self._storage.nbytes

    def byte_offset(self) -> int:
        return self._offset

    def byte_pointer(self) -> int:
        return 0 if self._storage is None else self._storage.ptr + self._offset

    def is_contiguous(self) -> bool:
        if self.empty():
            return True
        expect = 1
        for s, st in zip(reversed(self._shape), reversed(self._stride)):
            if s != 1 and st != expect:
                return False
            expect *= s
        return True

    def pinned(self) -> bool:
        return False

    # ---- views
    def view(self, shape: Sequence[int]) -> "Tensor":
        assert self.is_contiguous(), "view needs a contiguous tensor"
        shape = [int(s) for s in shape]
        if -1 in shape:
            known = _prod([s for s in shape if s != -1])
            shape[shape.index(-1)] = self.size // max(known, 1)
        assert _prod(shape) == self.size, (shape, self._shape)
        return Tensor._make(self._storage, shape, _contig_stride(shape), self._dtype, self._offset)

    def type_view(self, dtype: int, shape: Optional[Sequence[int]] = None) -> "Tensor":
        assert self.is_contiguous()
        if shape is None:
            assert _ITEMSIZE[dtype] == self.itemsize, "type_view without a shape keeps the item size"
            shape = self._shape
        assert _prod(shape) * _ITEMSIZE[dtype] <= self.bytesize()
        return Tensor._make(self._storage, shape, _contig_stride(shape), dtype, self._offset)

    def as_strided(self, shape, stride, storage_byte_offset: int = 0) -> "Tensor":
        return Tensor._make(self._storage, shape, stride, self._dtype, storage_byte_offset)

    def slice_axis(self, dim: int, start, stop, step=None) -> "Tensor":
        n = self._shape[dim]
        start, stop, step = slice(start, stop, step).indices(n)
        assert step > 0
        count = max(0, (stop - start + step - 1) // step)
        shape, stride = list(self._shape), list(self._stride)
        shape[dim] = count
        stride[dim] = self._stride[dim] * step
        off = self._offset + start * self._stride[dim] * self.itemsize
        return Tensor._make(self._storage, shape, stride, self._dtype, off)

    def slice_first_axis(self, start: int, end: int) -> "Tensor":
        return self.slice_axis(0, start, end)

    def select(self, dim: int, index: int) -> "Tensor":
        if index < 0:
            index += self._shape[dim]
        assert 0 <= index < self._shape[dim]
        shape, stride = list(self._shape), list(self._stride)
        off = self._offset + index * stride[dim] * self.itemsize
        del shape[dim], stride[dim]
        return Tensor._make(self._storage, shape, stride, self._dtype, off)

    def unsqueeze(self, dim: int) -> "Tensor":
        shape, stride = list(self._shape), list(self._stride)
        shape.insert(dim, 1)
        stride.insert(dim, stride[dim] * self._shape[dim] if dim < len(self._stride) else 1)
        return Tensor._make(self._storage, shape, stride, self._dtype, self._offset)

    def squeeze(self, dim: Optional[int] = None) -> "Tensor":
        keep = [i for i, s in enumerate(self._shape) if not (s == 1 and (dim is None or i == dim))]
        return Tensor._make(self._storage, [self._shape[i] for i in keep],
                            [self._stride[i] for i in keep], self._dtype, self._offset)

    def transpose(self, d0: int, d1: int) -> "Tensor":
        shape, stride = list(self._shape), list(self._stride)
        shape[d0], shape[d1] = shape[d1], shape[d0]
        stride[d0], stride[d1] = stride[d1], stride[d0]
        return Tensor._make(self._storage, shape, stride, self._dtype, self._offset)

    @property
    def T(self) -> "Tensor":
        if self.ndim != 2:
            raise ValueError("you can only use .T with 2d tensor.")
        return self.transpose(0, 1)

    def __getitem__(self, key) -> "Tensor":
        if not isinstance(key, tuple):
            key = (key,)
        res, dim = self, 0
        n_spec = sum(1 for k in key if k is not Ellipsis and k is not None)
        for k in key:
            if k is Ellipsis:
                dim += self.ndim - n_spec
            elif isinstance(k, slice):
                res = res.slice_axis(dim, k.start, k.stop, k.step)
                dim += 1
            elif isinstance(k, (int, np.integer)):
                res = res.select(dim, int(k))
            elif k is None:
                res = res.unsqueeze(dim)
                dim += 1
            else:
                raise ValueError("tv::Tensor only support .../None/int/slice slicing")
        return res

    # ---- host access
    def _host_array(self) -> np.ndarray:
        assert self.device == -1
        dt = _HOST_VIEW_DTYPE[self._dtype]
        return np.ndarray(self._shape, dtype=dt, buffer=self._storage.arr, offset=self._offset,
                          strides=[s * dt.itemsize for s in self._stride])

    def numpy_view(self) -> np.ndarray:
        if self.device != -1:
            raise RuntimeError("you need to call .cpu() before convert cuda tensor to numpy")
        if self._storage is None:
            return np.empty([0], dtype=np.float32)
        return self._host_array()

    def numpy(self) -> np.ndarray:
        return np.array(self.numpy_view(), copy=True)

    # ---- transfers
    def _contiguous_span(self):
        assert self.is_contiguous(), "device transfers need contiguous tensors"
        return self.byte_pointer(), self.bytesize()

    def cpu(self, ctx: Optional[Context] = None) -> "Tensor":
        if self._storage is None:
            return Tensor()
        if self.device == -1:
            return self.clone()
        src = self if self.is_contiguous() else self.clone()
        out = Tensor(self._shape, self._dtype, -1)
        ptr, n = src._contiguous_span()
        stream = ctx.cuda_stream_int() if ctx else 0
        _capi.check(_capi.lib().cumm_hip_memcpy_d2h(out.byte_pointer(), ptr, n, stream))
        return out

    def cuda(self, ctx: Optional[Context] = None) -> "Tensor":
        if self._storage is None:
            return Tensor()
        if self.device != -1:
            return self.clone()
        host = np.ascontiguousarray(self._host_array())
        out = Tensor(self._shape, self._dtype, 0)
        stream = ctx.cuda_stream_int() if ctx else 0
        _capi.check(_capi.lib().cumm_hip_memcpy_h2d(out.byte_pointer(), host.ctypes.data,
                                                    host.nbytes, stream))
        return out

    def clone(self, pinned: bool = False, use_cpu_copy: bool = False) -> "Tensor":
        if self._storage is None:
            return Tensor()
        out = Tensor(self._shape, self._dtype, self.device)
        out.copy_(self)
        return out

    def copy_(self, other: "Tensor", ctx: Optional[Context] = None) -> None:
        assert self._shape == other._shape and self._dtype == other._dtype, "shape/dtype mismatch"
        stream = ctx.cuda_stream_int() if ctx else 0
        L = _capi.lib()
        if self.device == -1 and other.device == -1:
            self._host_array()[...] = other._host_array()
            return
        if self.device == -1:
            src = other if other.is_contiguous() else other.clone()
            assert self.is_contiguous()
            _capi.check(L.cumm_hip_memcpy_d2h(self.byte_pointer(), src.byte_pointer(),
                                              self.bytesize(), stream))
            return
        if other.device == -1:
            host = np.ascontiguousarray(other._host_array())
            assert self.is_contiguous()
            _capi.check(L.cumm_hip_memcpy_h2d(self.byte_pointer(), host.ctypes.data, host.nbytes,
                                              stream))
            return
        if self.is_contiguous() and other.is_contiguous():
            _capi.check(L.cumm_hip_memcpy_d2d(self.byte_pointer(), other.byte_pointer(),
                                              self.bytesize(), stream))
            return
        # strided device copies go through the host (not on any hot path)
        tmp = Tensor(self._shape, self._dtype, -1)
        full_o = Tensor._make(other._storage, [other._storage.nbytes], [1], uint8, 0).cpu()
        src_view = Tensor._make(full_o._storage, other._shape, other._stride, other._dtype,
                                other._offset)
        tmp._host_array()[...] = src_view._host_array()
        full_s = Tensor._make(self._storage, [self._storage.nbytes], [1], uint8, 0).cpu()
        dst_view = Tensor._make(full_s._storage, self._shape, self._stride, self._dtype,
                                self._offset)
        dst_view._host_array()[...] = tmp._host_array()
        _capi.check(L.cumm_hip_memcpy_h2d(self._storage.ptr, full_s._storage.ptr,
                                          self._storage.nbytes, stream))

    def zero_(self, ctx: Optional[Context] = None) -> "Tensor":
        if self.empty():
            return self
        if self.device == -1:
            self._host_array()[...] = 0
        else:
            ptr, n = self._contiguous_span()
            stream = ctx.cuda_stream_int() if ctx else 0
            _capi.check(_capi.lib().cumm_hip_memset(ptr, 0, n, stream))
        return self

    def _fill_host_pattern(self, host: np.ndarray, ctx: Optional[Context]) -> "Tensor":
        src = from_numpy(host)
        if src.dtype != self._dtype:      # bf16 travels as uint16 bit patterns
            src = src.type_view(self._dtype)
        self.copy_(src, ctx)
        return self

    def fill_int_(self, val: int, ctx: Optional[Context] = None) -> "Tensor":
        if self._dtype == bfloat16:
            return self.fill_float_(float(val), ctx)
        return self._fill_host_pattern(np.full(self._shape, val, dtype=_HOST_VIEW_DTYPE[self._dtype]), ctx)

    def fill_float_(self, val: float, ctx: Optional[Context] = None) -> "Tensor":
        if self._dtype == bfloat16:
            # round to nearest even on bit 16 of the float32 pattern, NaN -> 0x7FFF
            # (bfloat16_t(float), include/tensorview/gemm/dtypes/bfloat16.h:86-111 of the reference)
            u = int(np.float32(val).view(np.uint32))
            bits = 0x7FFF if val != val else ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF
            return self._fill_host_pattern(np.full(self._shape, bits, dtype=np.uint16), ctx)
        return self._fill_host_pattern(np.full(self._shape, val, dtype=_HOST_VIEW_DTYPE[self._dtype]), ctx)

    def __repr__(self):
        return "Tensor[%s|%s|%s]" % (self._shape, self._dtype, self.device)


# ---- factories (cumm/tensorview/__init__.py:687-811 of the reference)
def zeros(shape, dtype=np.float32, device: int = -1, pinned: bool = False,
          managed: bool = False) -> Tensor:
    return Tensor(shape, _to_tv_dtype(dtype), device).zero_()


def empty(shape, dtype=np.float32, device: int = -1, pinned: bool = False,
          managed: bool = False) -> Tensor:
    return Tensor(shape, _to_tv_dtype(dtype), device)


def full(shape, val, dtype=np.float32, device: int = -1, pinned: bool = False,
         managed: bool = False) -> Tensor:
    t = Tensor(shape, _to_tv_dtype(dtype), device)
    return t.fill_float_(val) if t.dtype in (float32, float16, float64, bfloat16, tf32) else t.fill_int_(val)


def from_numpy(arr: np.ndarray) -> Tensor:
    arr = np.asarray(arr)
    dtype = NPDTYPE_TO_TENSOR_MAP[arr.dtype]
    if not arr.flags.c_contiguous:
        arr = np.ascontiguousarray(arr)
    flat = arr.reshape(-1).view(np.uint8)
    return Tensor._make(_HostStorage(flat), arr.shape, _contig_stride(arr.shape), dtype, 0)


def from_blob_strided(ptr: int, shape, stride, dtype, device: int, storage_offset: int = 0,
                      keepalive=None) -> Tensor:
    """Wrap existing memory; never frees it."""
    dt = _to_tv_dtype(dtype)
    extent = 1 + sum((int(s) - 1) * int(st) for s, st in zip(shape, stride)) if len(shape) else 1
    nbytes = (storage_offset + extent) * _ITEMSIZE[dt]
    if device == -1:
        buf = (ctypes.c_uint8 * nbytes).from_address(int(ptr))
        st = _HostStorage(np.frombuffer(buf, dtype=np.uint8))
        st.keepalive = keepalive
    else:
        st = _BlobStorage(ptr, nbytes, device, keepalive)
    return Tensor._make(st, shape, stride, dt, storage_offset * _ITEMSIZE[dt])


def from_blob(ptr: int, shape, dtype, device: int, storage_offset: int = 0, keepalive=None) -> Tensor:
    return from_blob_strided(ptr, shape, _contig_stride(shape), dtype, device, storage_offset,
                             keepalive)


from_const_blob = from_blob
from_const_blob_strided = from_blob_strided


def cat_first_axis(tens: List[Tensor]) -> Tensor:
    host = np.concatenate([t.cpu().numpy_view() if t.device != -1 else t.numpy_view() for t in tens])
    out = from_numpy(host)
    out._dtype = tens[0].dtype
    return out.cuda() if tens[0].device != -1 else out


def is_cpu_only() -> bool:
    return False


def device_count() -> int:
    n = ctypes.c_int(0)
    _capi.lib().cumm_hip_device_count(ctypes.byref(n))
    return n.value


# ---- timers (tv::CUDAEvent / CUDAKernelTimer, include/tensorview/profile/cuda_profiler.h:97-406)
class CUDAEvent:
    def __init__(self, name: str = ""):
        self.name = name
        out = ctypes.c_void_p()
        _capi.check(_capi.lib().cumm_hip_event_create(ctypes.byref(out)))
        self._ev = out.value

    def record(self, stream: int = 0):
        _capi.check(_capi.lib().cumm_hip_event_record(self._ev, stream))
        return self

    def sync(self):
        _capi.check(_capi.lib().cumm_hip_event_synchronize(self._ev))
        return self

    @staticmethod
    def duration(start: "CUDAEvent", stop: "CUDAEvent") -> float:
        ms = ctypes.c_float(0)
        _capi.check(_capi.lib().cumm_hip_event_elapsed_ms(start._ev, stop._ev, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        if getattr(self, "_ev", None):
            try:
                _capi.lib().cumm_hip_event_destroy(self._ev)
            except Exception:
                pass


class CUDAKernelTimer:
    """Named event pairs around kernel launches; disabled timers record nothing."""

    def __init__(self, enable: bool = True):
        self.enable = bool(enable)
        self._pairs = {}
        self._ns = []

    def push(self, name: str):
        self._ns.append(name)

    def pop(self):
        self._ns.pop()

    def _key(self, name):
        return ".".join(self._ns + [name])

    def record(self, name: str, stream: int = 0):
        if not self.enable:
            return
        key = self._key(name)
        ev = CUDAEvent(key).record(stream)
        self._pairs.setdefault(key, []).append(ev)

    def insert_pair(self, name: str, start: str, stop: str):
        pass

    def has_pair(self, name: str) -> bool:
        return len(self._pairs.get(self._key(name), [])) >= 2

    def get_all_pair_time(self):
        out = {}
        for key, evs in self._pairs.items():
            if len(evs) >= 2:
                evs[-1].sync()
                out[key] = CUDAEvent.duration(evs[-2], evs[-1])
        return out

    def get_pair_time(self, name: str) -> float:
        return self.get_all_pair_time()[self._key(name)]

    get_pair_duration = get_pair_time


KernelTimer = CUDAKernelTimer
