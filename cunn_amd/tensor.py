"""Host-side handles for the THCudaTensor / THCudaLongTensor structs of the C ABI.

This is plumbing for callers that are not LuaJIT: it builds the same structs
cutorch would hand to ``THNN_Cuda*`` (include/THCShim.h), moves data in and out
and turns TH error callbacks into Python exceptions. Device memory is either
owned by the library (hipMalloc, resizable - what an nn module's output buffers
are) or borrowed from a torch tensor (not resizable).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


class THError(RuntimeError):
    """Raised where Lua-torch would raise a Lua error from THError / THArgCheck."""


_pending = []
_ERR_CB = C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)
_ARG_CB = C.CFUNCTYPE(None, C.c_int, C.c_char_p, C.c_void_p)


@_ERR_CB
def _on_error(msg, _data):
    _pending.append(msg.decode(errors="replace"))


@_ARG_CB
def _on_arg_error(arg, msg, _data):
    _pending.append(f"bad argument #{arg}: " + (msg.decode(errors="replace") if msg else ""))


def check():
    """Raise the error the last library call reported, if any."""
    if _pending:
        msg = _pending[0]
        del _pending[:]
        raise THError(msg)


_state = None


def state():
    """The process-wide THCState (cutorch.getState(), THCUNN.lua:14-16)."""
    global _state
    if _state is None:
        lib = _lib.load()
        lib.THSetErrorHandler(C.cast(_on_error, C.c_void_p), None)
        lib.THSetArgErrorHandler(C.cast(_on_arg_error, C.c_void_p), None)
        _state = lib.THCState_alloc()
        check()
        if not _state:
            raise THError("THCState_alloc failed")
    return _state


def set_stream(stream_handle: int):
    """Make ``stream_handle`` (a hipStream_t, e.g. torch.cuda.Stream.cuda_stream) current."""
    _lib.load().THCState_setCurrentStream(state(), C.c_void_p(stream_handle))


def synchronize():
    _lib.load().THCState_synchronize(state())
    check()


def _longs(seq):
    seq = [int(v) for v in seq]
    return (C.c_long * max(len(seq), 1))(*seq), len(seq)


class _Base:
    _prefix = ""
    _dtype = None

    def __init__(self, handle=None, keepalive=None):
        self._lib = _lib.load()
        st = state()
        self._h = handle if handle is not None else getattr(self._lib, self._prefix + "_new")(st)
        self._keep = keepalive

    # -- construction -------------------------------------------------------
    @classmethod
    def with_size(cls, *size):
        lib = _lib.load()
        arr, n = _longs(size)
        h = getattr(lib, cls._prefix + "_newWithSize")(state(), n, arr)
        check()
        return cls(h)

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a, dtype=cls._dtype)
        t = cls.with_size(*a.shape)
        if a.size:
            getattr(t._lib, cls._prefix + "_copyFromHost")(state(), t._h, a.ctypes.data_as(C.c_void_p))
            check()
        return t

    @classmethod
    def from_torch(cls, t):
        """Borrow the memory of a contiguous-or-strided torch CUDA tensor (not resizable)."""
        lib = _lib.load()
        size, n = _longs(t.shape)
        stride, _ = _longs(t.stride())
        span = 1 + sum((s - 1) * st for s, st in zip(t.shape, t.stride())) if t.numel() else 0
        h = getattr(lib, cls._prefix + "_newWithData")(state(), C.c_void_p(t.data_ptr()), span, 0, n, size, stride)
        check()
        return cls(h, keepalive=t)

    # -- inspection ---------------------------------------------------------
    def dim(self):
        return int(getattr(self._lib, self._prefix + "_nDimension")(state(), self._h))

    def size(self):
        f = getattr(self._lib, self._prefix + "_size")
        return tuple(int(f(state(), self._h, d)) for d in range(self.dim()))

    def nelement(self):
        return int(getattr(self._lib, self._prefix + "_nElement")(state(), self._h))

    def data_ptr(self):
        return getattr(self._lib, self._prefix + "_data")(state(), self._h) or 0

    def resize(self, *size):
        arr, n = _longs(size)
        getattr(self._lib, self._prefix + "_resizeNd")(state(), self._h, n, arr)
        check()
        return self

    def numpy(self):
        out = np.empty(self.size(), self._dtype)
        if out.size:
            getattr(self._lib, self._prefix + "_copyToHost")(state(), self._h, out.ctypes.data_as(C.c_void_p))
            check()
        return out

    def copy_(self, a):
        a = np.ascontiguousarray(a, dtype=self._dtype)
        assert a.shape == self.size(), (a.shape, self.size())
        if a.size:
            getattr(self._lib, self._prefix + "_copyFromHost")(state(), self._h, a.ctypes.data_as(C.c_void_p))
            check()
        return self

    @property
    def handle(self):
        return self._h

    def __del__(self):
        try:
            if self._h and _state is not None:
                getattr(self._lib, self._prefix + "_free")(_state, self._h)
        except Exception:
            pass
        self._h = None


class CudaTensor(_Base):
    """THCudaTensor (fp32)."""
    _prefix = "THCudaTensor"
    _dtype = np.float32

    def stride(self):
        f = self._lib.THCudaTensor_stride
        return tuple(int(f(state(), self._h, d)) for d in range(self.dim()))

    def is_contiguous(self):
        return bool(self._lib.THCudaTensor_isContiguous(state(), self._h))

    def fill(self, v):
        self._lib.THCudaTensor_fill(state(), self._h, float(v))
        check()
        return self

    def copy_from(self, other):
        """Device-to-device copy of another CudaTensor with the same number of elements."""
        self._lib.THCudaTensor_copy(state(), self._h, other._h)
        check()
        return self

    def view(self, offset, size, stride):
        """A strided view sharing this tensor's storage (narrow/select/transpose by hand)."""
        sz, n = _longs(size)
        st, _ = _longs(stride)
        h = self._lib.THCudaTensor_newView(state(), self._h, int(offset), n, sz, st)
        check()
        return CudaTensor(h, keepalive=self)

    @classmethod
    def noncontiguous_from_numpy(cls, a, rng):
        """The reference tests' makeNonContiguous (test.lua:62-83): inflate up to three
        random dimensions by 4..15, narrow back to the wanted size at a random
        offset, and copy the data into that view."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        osize = list(a.shape)
        for _ in range(3):
            d = int(rng.integers(0, a.ndim))
            osize[d] += int(rng.integers(4, 16))
        big = cls.with_size(*osize)
        big.fill(float("nan"))  # anything read outside the view poisons the result
        strides = [1] * a.ndim
        for d in range(a.ndim - 2, -1, -1):
            strides[d] = strides[d + 1] * osize[d + 1]
        offset = 0
        for d in range(a.ndim):
            if osize[d] != a.shape[d]:
                offset += int(rng.integers(0, osize[d] - a.shape[d] + 1)) * strides[d]
        v = big.view(offset, a.shape, strides)
        v.copy_(a)
        return v


class CudaLongTensor(_Base):
    """THCudaLongTensor (int64 indices)."""
    _prefix = "THCudaLongTensor"
    _dtype = np.int64
