"""CPU-side checks of the drop-in boundary: the library loads and exports every
symbol include/*.h declares, with C linkage; struct layouts match the header."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(THNN_Cuda\w+|THCState_\w+|THCuda(?:Long)?Tensor_\w+|THSet\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from cunn_amd import _lib
    lib = _lib.load()
    declared = _declared("THCUNN.h") + _declared("THCShim.h")
    # 14 hot-path + 9 dilated / transposed convolution + 2 Threshold + the no-allocation accGradParameters variant
    assert len([n for n in declared if n.startswith("THNN_Cuda")]) == 26
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"


def test_entry_point_names_follow_the_reference_binder():
    """THCUNN.lua:25,42-48,129 builds 'THNN_' .. 'Cuda' .. name for torch.CudaTensor."""
    from cunn_amd import _lib
    assert sorted(_lib.ENTRY_POINTS) == sorted(_lib.SIGNATURES)
    assert sorted("THNN_Cuda" + n for n in _lib.ENTRY_POINTS) == \
        [n for n in _declared("THCUNN.h") if n.startswith("THNN_Cuda")]


def test_struct_layout_matches_cutorch_field_order(tmp_path):
    """Compile a tiny C program against include/THCShim.h and check the offsets the
    LuaJIT FFI cdef of cutorch 1.0 implies on LP64 (size, stride, nDimension,
    storage, storageOffset, refcount, flag / data, size, refcount, flag, ...)."""
    import subprocess
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "THCUNN.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu\n",
    offsetof(THCudaTensor, size), offsetof(THCudaTensor, stride), offsetof(THCudaTensor, nDimension),
    offsetof(THCudaTensor, storage), offsetof(THCudaTensor, storageOffset), offsetof(THCudaTensor, refcount),
    offsetof(THCudaTensor, flag), sizeof(THCudaTensor));
  printf("%zu %zu %zu %zu %zu %zu %zu %zu\n",
    offsetof(THCudaStorage, data), offsetof(THCudaStorage, size), offsetof(THCudaStorage, refcount),
    offsetof(THCudaStorage, flag), offsetof(THCudaStorage, allocator), offsetof(THCudaStorage, allocatorContext),
    offsetof(THCudaStorage, view), offsetof(THCudaStorage, device));
  printf("%zu %zu\n", sizeof(long), sizeof(THCudaLongTensor));
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode().split("\n")
    assert out[0].split() == ["0", "8", "16", "24", "32", "40", "44", "48"]
    assert out[1].split() == ["0", "8", "16", "20", "24", "32", "40", "48"]
    assert out[2].split() == ["8", "48"]


def test_missing_library_fails_loudly(monkeypatch):
    from cunn_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libTHCUNN.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
