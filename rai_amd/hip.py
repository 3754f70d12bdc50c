"""Host-side handle for tensors resident in MI355X HBM, over the C ABI.

`HipTensor` mirrors what rai's `TensorLike` storage exposes
(rai-core/src/tensor.rs:19-26: shape, dtype, as_vec/as_bytes) plus the zero-copy
view operations candle layouts give the reference backend (transpose, narrow,
broadcast, reshape of contiguous data: backend/candle.rs:555-593, 891-899).
NumPy is used only to carry host bytes; bf16 travels as uint16 bit patterns.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import BF16, DTYPE_BY_NAME, DTYPE_NAMES, DTYPE_SIZE, F16, F32, F64, I64, U8, U32, TensorDesc, call

_NP_STORAGE = {U8: np.uint8, U32: np.uint32, I64: np.int64, F16: np.float16, BF16: np.uint16, F32: np.float32,
               F64: np.float64}


class Buffer:
    """Ref-counted device allocation (rai_hip_alloc / rai_hip_release)."""

    def __init__(self, dev, nbytes):
        p = C.c_void_p()
        call("rai_hip_alloc", dev, max(int(nbytes), 1), C.byref(p))
        self.ptr, self.dev, self.nbytes = p.value, dev, int(nbytes)

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                _lib.load().rai_hip_release(C.c_void_p(self.ptr))
                self.ptr = None
        except Exception:
            pass


def _contig_strides(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


class HipTensor:
    def __init__(self, buf, dtype, shape, strides=None, offset=0):
        self.buf = buf
        self.dtype = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(strides) if strides is not None else _contig_strides(self.shape)
        self.offset = int(offset)
        if len(self.shape) > _lib.MAX_RANK:
            raise ValueError("rank > 8")

    # ------------------------------------------------------------ creation
    @classmethod
    def empty(cls, shape, dtype, dev=0):
        dt = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)
        n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        return cls(Buffer(dev, n * DTYPE_SIZE[dt]), dt, shape)

    @classmethod
    def from_storage(cls, arr, dtype, dev=0):
        """Upload host bytes (`arr` already in the storage representation)."""
        dt = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)
        arr = np.ascontiguousarray(arr, dtype=_NP_STORAGE[dt])
        t = cls.empty(arr.shape, dt, dev)
        if arr.nbytes:
            call("rai_hip_h2d", dev, C.c_void_p(t.buf.ptr), arr.ctypes.data_as(C.c_void_p), arr.nbytes)
        return t

    # ------------------------------------------------------------ metadata
    @property
    def dev(self):
        return self.buf.dev

    @property
    def dtype_name(self):
        return DTYPE_NAMES[self.dtype]

    @property
    def rank(self):
        return len(self.shape)

    def numel(self):
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def is_contiguous(self):
        return all(s == 1 or st == c for s, st, c in zip(self.shape, self.strides, _contig_strides(self.shape)))

    def desc(self):
        d = TensorDesc()
        d.data = self.buf.ptr
        d.dtype = self.dtype
        d.rank = len(self.shape)
        for i, (s, st) in enumerate(zip(self.shape, self.strides)):
            d.shape[i] = s
            d.stride[i] = st
        d.offset = self.offset
        return d

    # ------------------------------------------------------------ views (zero copy)
    def transpose(self, d0, d1):
        d0 %= self.rank
        d1 %= self.rank
        sh, st = list(self.shape), list(self.strides)
        sh[d0], sh[d1] = sh[d1], sh[d0]
        st[d0], st[d1] = st[d1], st[d0]
        return HipTensor(self.buf, self.dtype, sh, st, self.offset)

    def permute(self, dims):
        return HipTensor(self.buf, self.dtype, [self.shape[d] for d in dims], [self.strides[d] for d in dims],
                         self.offset)

    def narrow(self, dim, start, length):
        dim %= self.rank
        if start < 0 or start + length > self.shape[dim]:
            raise ValueError("narrow out of range")
        sh = list(self.shape)
        sh[dim] = length
        return HipTensor(self.buf, self.dtype, sh, self.strides, self.offset + start * self.strides[dim])

    def broadcast_to(self, shape):
        shape = tuple(shape)
        pad = len(shape) - self.rank
        if pad < 0:
            raise ValueError("broadcast to lower rank")
        sh = (1,) * pad + self.shape
        st = (0,) * pad + self.strides
        out = []
        for s, t, tgt in zip(sh, st, shape):
            if s == tgt:
                out.append(t)
            elif s == 1:
                out.append(0)
            else:
                raise ValueError(f"cannot broadcast {self.shape} to {shape}")
        return HipTensor(self.buf, self.dtype, shape, out, self.offset)

    def reshape(self, shape):
        shape = tuple(int(s) for s in shape)
        if int(np.prod(shape, dtype=np.int64)) != self.numel():
            raise ValueError(f"cannot reshape {self.shape} to {shape}")
        src = self if self.is_contiguous() else self.contiguous()
        return HipTensor(src.buf, src.dtype, shape, None, src.offset)

    def contiguous(self):
        if self.is_contiguous():
            return self
        out = HipTensor.empty(self.shape, self.dtype, self.dev)
        call("rai_hip_copy", self.dev, C.byref(self.desc()), C.byref(out.desc()))
        return out

    # ------------------------------------------------------------ host access
    def to_storage(self):
        """Device -> host, as the storage representation (bf16 as uint16 bits)."""
        src = self.contiguous()
        out = np.empty(src.shape, dtype=_NP_STORAGE[src.dtype])
        if out.nbytes:
            base = src.buf.ptr + src.offset * DTYPE_SIZE[src.dtype]
            call("rai_hip_d2h", src.dev, out.ctypes.data_as(C.c_void_p), C.c_void_p(base), out.nbytes)
        return out

    def to_float(self):
        """Device -> host as float32/float64/int arrays (bf16/f16 widened exactly)."""
        a = self.to_storage()
        if self.dtype == BF16:
            return (a.astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(a.shape)
        if self.dtype == F16:
            return a.astype(np.float32)
        return a


def sync(dev=0):
    call("rai_hip_sync", dev)


def device_count():
    n = C.c_int(0)
    st = _lib.load().rai_hip_device_count(C.byref(n))
    return n.value if st == 0 else 0


def measure_peak(kind, nbytes=0, launches=10, dev=0):
    """One of the library's ceiling loops (include/rai_hip_peaks.h; kind: a key of _lib.PEAK_KINDS): returns
    (seconds per launch, work per launch in flops or bytes)."""
    sec, work = C.c_double(0.0), C.c_double(0.0)
    call("rai_hip_measure_peak", dev, _lib.PEAK_KINDS[kind], int(nbytes), int(launches), C.byref(sec), C.byref(work))
    return sec.value, work.value
