"""The binder: what ``THNN.bind(THCUNN.C, function_names, 'Cuda', THCUNN.getState)``
produces at THCUNN.lua:129-133 - one function per entry point that prepends the
THCState and forwards the remaining arguments unchanged. Tensor arguments are
`CudaTensor` / `CudaLongTensor` handles or ``None`` for ``[OPTIONAL]`` ones."""
from __future__ import annotations

import ctypes as C

from . import _lib
from .tensor import _Base, check, state


def _arg(a):
    if a is None:
        return None
    if isinstance(a, _Base):
        return a.handle
    return a


class _Namespace:
    def __init__(self):
        self._fns = {}

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        fn = self._fns.get(name)
        if fn is None:
            if name not in _lib.SIGNATURES:
                raise AttributeError(f"THNN has no function {name!r}")
            cfn = getattr(_lib.load(), "THNN_Cuda" + name)

            def fn(*args, _cfn=cfn):
                _cfn(state(), *[_arg(a) for a in args])
                check()

            fn.__name__ = name
            self._fns[name] = fn
        return fn


THNN = _Namespace()
