"""The C ABI driven by a caller that is not this repository's harness: tests/c_caller/caller.c, plain C compiled
with gcc, takes only the prototypes from include/THCUNN.h and include/THCUNN_fused.h and declares the tensor and
storage structs itself (as cutorch under LuaJIT would: THCUNN.lua:129-133), passes empty result tensors the library
must resize, a 2-D depthwise weight, a strided input, NULL for optional tensors, and compares with the committed
golden vectors, which this test dumps to raw files for it. Every exported entry point is called at least once: the 14
of the hot path (BatchNormalization with its `bool, double, double` tail, both pooling families forward and backward,
dilated max pooling), dilated and transposed convolution, Threshold out of place and in place, the three fused entry
points and the variant that allocates nothing."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_caller", "caller.c")
PREBUILT = os.path.join(ROOT, "tests", "c_caller", "caller_bin")   # written by __graft_entry__.build()
LIBDIR = os.path.join(ROOT, "cunn_amd", "lib")
CASES = ("dw_s2", "conv_3x3", "conv_s2", "bn_4d", "bnrelu_4d", "pool_3s2p1_ceil", "pool_2s2", "pool_dil2", "dilconv_d2",
         "fullconv_s2", "thr")


def build_caller(out):
    """gcc on the one C file; links libTHCUNN.so and the HIP runtime (for hipMalloc / hipMemcpy)."""
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-O1", "-I", os.path.join(ROOT, "include"), SRC, "-o", out,
                           "-L", LIBDIR, "-lTHCUNN", "-L", "/opt/rocm/lib", "-lamdhip64", "-lm",
                           "-Wl,-rpath," + LIBDIR, "-Wl,-rpath,/opt/rocm/lib"])
    return out


def dump_vectors(directory):
    G = np.load(os.path.join(ROOT, "tests", "golden", "thnn_golden.npz"))
    lines = []
    for key in G.files:
        case, name = key.split("/", 1)
        if case not in CASES:
            continue
        a = G[key]
        a = np.ascontiguousarray(a, dtype=np.float32 if a.dtype.kind == "f" else np.int64)
        a.tofile(os.path.join(directory, f"{case}.{name}.bin"))
        lines.append(f"{case}.{name} {'f' if a.dtype == np.float32 else 'l'} {a.ndim} " + " ".join(str(d) for d in a.shape))
    with open(os.path.join(directory, "manifest.txt"), "w") as f:
        f.write("\n".join(lines) + "\n")


def test_plain_c_caller_with_its_own_tensor_structs(tmp_path):
    exe = PREBUILT if os.path.exists(PREBUILT) and os.path.getmtime(PREBUILT) >= os.path.getmtime(SRC) \
        else build_caller(str(tmp_path / "caller"))
    dump_vectors(str(tmp_path))
    print("running", exe, flush=True)
    r = subprocess.run([exe, str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=100)
    out = r.stdout.decode(errors="replace")
    print(out)
    assert r.returncode == 0, out
    assert "0 failure(s)" in out and "FAILED" not in out and out.count(" ok ") >= 65
    for module in ("depthwise", "SpatialConvolutionMM ", "SpatialConvolutionMMReLU", "BatchNormalization ", "BatchNormalizationReLU",
                   "SpatialMaxPooling", "SpatialAveragePooling", "SpatialDilatedMaxPooling", "SpatialDilatedConvolution",
                   "SpatialFullConvolution", "SpatialFullDilatedConvolution", "Threshold", "noAlloc"):
        assert module in out, module
