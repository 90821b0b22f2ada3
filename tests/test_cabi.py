"""The C-ABI library loads and exports exactly what include/jaxhip.h declares (no compute without a GPU),
and every kernel class generates source that hiprtc compiles for gfx950 on the CPU."""
import ctypes
import os
import re
import subprocess

import pytest

from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker
from jaxjs_hip.errors import HipRuntimeError
from jaxjs_hip.kernelgen import generate
from jaxjs_hip.lowering import mapKernel, matmulKernel, matvecKernel, reduceKernel
from jaxjs_hip.runtime import EXPORTED_SYMBOLS, LIB_PATH, compile_source, load_library

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "jaxhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jh_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == EXPORTED_SYMBOLS


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB_PATH), "build the runtime first (__graft_entry__.build())"
    out = subprocess.run(["nm", "-D", "--defined-only", LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = sorted(set(re.findall(r" T (jh_[a-z0-9_]+)", out)))
    assert exported == _declared()
    lib = load_library()
    assert lib.jh_abi_version() == 1
    for name in EXPORTED_SYMBOLS:
        assert getattr(lib, name) is not None


def test_calls_before_init_fail_loudly():
    lib = load_library()
    p = ctypes.c_void_p()
    assert lib.jh_malloc(16, ctypes.byref(p)) != 0
    assert b"jh_init" in lib.jh_last_error()
    assert lib.jh_sync() != 0


def test_compile_error_is_reported():
    with pytest.raises(HipRuntimeError, match="hiprtc failed"):
        compile_source("extern \"C\" __global__ void k() { this is not C++; }", use_cache=False)


@pytest.mark.parametrize("name,kernel,klass", [
    ("map", mapKernel([70, 33], [(DType.Float32, ShapeTracker.fromShape([70, 33]))], lambda x: AluExp.erf(x)), "map"),
    ("row", reduceKernel([64, 4096], [(DType.Float32, ShapeTracker.fromShape([64, 4096]))], lambda x: x, AluOp.Max), "reduce_row"),
    ("col", reduceKernel([4096, 64], [(DType.Int32, ShapeTracker.fromShape([64, 4096]).permute([1, 0]))], lambda x: x, AluOp.Add), "reduce_col"),
    ("fold", reduceKernel([1, 1 << 22], [(DType.Float32, ShapeTracker.fromShape([1, 1 << 22]))], lambda x: x, AluOp.Add), "reduce_row+fold"),
    ("matvec", matvecKernel(11008, 4096, DType.Float16), "reduce_row"),
    ("gemm_nn", matmulKernel(512, 512, 512, DType.Float16), "gemm"),
    ("gemm_nt", matmulKernel(256, 256, 64, DType.Float16, b_transposed=True), "gemm"),
    ("gemm_f32", matmulKernel(256, 256, 64, DType.Float32), "gemm"),
], ids=lambda v: v if isinstance(v, str) else "")
def test_every_class_compiles_for_gfx950(name, kernel, klass):
    ks = generate(kernel)
    assert ks.klass == klass
    for src in ks.sources:
        assert len(compile_source(src, f"{name}.hip", use_cache=False)) > 1000
