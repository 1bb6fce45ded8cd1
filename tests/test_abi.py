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
    names = re.findall(r"\b(THNN_Cuda\w+|THCState_\w+|THCuda(?:Long)?Tensor_\w+|THSet\w+|THCUNN_\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from cunn_amd import _lib
    lib = _lib.load()
    declared = _declared("THCUNN.h") + _declared("THCShim.h") + _declared("THCUNN_fused.h")
    # BatchNormalization + ReLU, forward and backward; SpatialConvolutionMM + ReLU, forward
    assert len(_declared("THCUNN_fused.h")) == 3
    # 14 hot-path + 9 dilated / transposed convolution + 2 Threshold + the no-allocation accGradParameters variant
    assert len(_declared("THCUNN.h")) == 26
    # the test hooks: the two column kernels and the kernel-family switch
    assert {"THNN_Cuda_im2col", "THNN_Cuda_col2im", "THCUNN_setSwitch"} <= set(_declared("THCShim.h"))
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"


def test_entry_point_names_follow_the_reference_binder():
    """THCUNN.lua:25,42-48,129 builds 'THNN_' .. 'Cuda' .. name for torch.CudaTensor."""
    from cunn_amd import _lib
    assert sorted(_lib.ENTRY_POINTS) == sorted(_lib.SIGNATURES)
    assert sorted("THNN_Cuda" + n for n in _lib.ENTRY_POINTS) == \
        sorted(n for n in _declared("THCUNN.h") + _declared("THCUNN_fused.h") if n.startswith("THNN_Cuda"))


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


# ---- the prototypes are what the reference's binder would hand to ffi.cdef ---------------------------------
REFERENCE_HEADER = "/root/reference/lib/THCUNN/generic/THCUNN.h"


def _binder_cdef(text):
    """THCUNN.lua:22-69 restated: strip preprocessor lines, `TH_API void THNN_(X)` -> `void THNN_TYPEX`, then
    the plain substring replacements of the 'Cuda' (fp32) instantiation."""
    text = re.sub(r"\n#[^\n]*", "", text)
    text = re.sub(r"^#[^\n]*\n", "", text)
    text = re.sub(r"TH_API void THNN_\(([A-Za-z0-9_]+)\)", r"void THNN_TYPE\1", text)
    for k, v in (("THCTensor", "THCudaTensor"), ("THCIndexTensor", "THCudaLongTensor"), ("TYPE", "Cuda"), ("accreal", "float")):
        text = text.replace(k, v)
    return text


def _prototypes(text):
    """{name: [parameter type, ...]} of every `void THNN_Cuda<name>(...)` in C text (comments dropped,
    parameter names dropped, whitespace normalised: 'THCudaTensor *', 'int', 'bool', 'float', 'double')."""
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for name, args in re.findall(r"void\s+THNN_Cuda(\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        for a in args.split(","):
            a = " ".join(a.split())
            m = re.match(r"^(.*?)(\w+)$", a)            # everything before the parameter name
            t = m.group(1).replace(" *", "*").replace("* ", "*").strip()
            types.append(re.sub(r"\s*\*", " *", t))
        out[name] = types
    return out


@pytest.mark.skipif(not os.path.exists(REFERENCE_HEADER), reason="the reference tree is not on this machine")
def test_prototypes_equal_the_binder_rewrite_of_the_reference_header():
    """What LuaJIT would cdef from the reference's own header (THCUNN.lua:22-69) is, for every entry point this
    library declares with a reference counterpart, exactly the prototype in include/THCUNN.h - and the ctypes
    signatures of the Python harness say the same."""
    import ctypes as C
    from cunn_amd import _lib
    ref = _prototypes(_binder_cdef(open(REFERENCE_HEADER).read()))
    ours = _prototypes(open(os.path.join(ROOT, "include", "THCUNN.h")).read())
    extensions = {"SpatialDepthWiseConvolution_accGradParameters_noAlloc"}   # no counterpart in the reference
    assert set(ours) - set(ref) == extensions
    assert len(set(ours) & set(ref)) == 25
    ctype = {"THCState *": C.c_void_p, "THCudaTensor *": C.c_void_p, "THCudaLongTensor *": C.c_void_p, "int": C.c_int,
             "bool": C.c_bool, "float": C.c_float, "double": C.c_double}
    for name in sorted(set(ours) - extensions):
        assert ours[name] == ref[name], f"{name}: {ours[name]} != {ref[name]}"
        assert _lib.SIGNATURES[name] == [ctype[t] for t in ref[name]], name
