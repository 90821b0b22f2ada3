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
    assert lib.jh_abi_version() == 2
    for name in EXPORTED_SYMBOLS:
        assert getattr(lib, name) is not None


def test_calls_before_init_fail_loudly():
    lib = load_library()
    p = ctypes.c_void_p()
    assert lib.jh_malloc(16, ctypes.byref(p)) != 0
    assert b"jh_init" in lib.jh_last_error()
    assert lib.jh_sync() != 0


def test_library_honours_option_lines_of_a_source_and_refuses_unknown_ones():
    """`jh_compile` itself reads the leading `// hiprtc-option:` lines (a host that replays exported plans passes the
    plan's common options only): a listed option compiles with no options passed at all, any other is an error."""
    import ctypes
    lib = load_library()

    def compile_raw(text):
        code, size = ctypes.c_void_p(), ctypes.c_size_t()
        opts = (ctypes.c_char_p * 1)(b"--offload-arch=gfx950")
        rc = lib.jh_compile(text.encode(), b"k.hip", opts, 1, ctypes.byref(code), ctypes.byref(size), None, 0)
        if rc == 0:
            lib.jh_code_free(code)
        return rc, size.value

    body = 'extern "C" __global__ void k(float* p) { p[0] = 1.0f; }\n'
    rc, size = compile_raw("// hiprtc-option: -fno-slp-vectorize\n" + body)
    assert rc == 0 and size > 1000
    rc, _ = compile_raw("// hiprtc-option: -DANYTHING\n" + body)
    assert rc != 0 and b"not on the list" in lib.jh_last_error()


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


def test_direct_lds_gemm_pipeline_choice_and_limits():
    """Slab depth and LDS pipeline of the f16 fast path: 64-deep slabs only when both operands run along k, the
    five-unit ring for the 256x256 tile, classical stages otherwise; configurations that exceed the 160 KiB of LDS are
    refused when the source is generated, not at launch."""
    def info(M, N, K, bt, **tile):
        return generate(matmulKernel(M, N, K, DType.Float16, b_transposed=bt), gemm_tile=tuple(sorted(tile.items())) if tile else None).info

    nn = info(8192, 8192, 8192, False)
    assert (nn["BM"], nn["BN"], nn["BK"], nn["stages"], nn["ring"]) == (256, 256, 32, 4, 0)
    nt = info(8192, 8192, 8192, True)
    assert (nt["BM"], nt["BN"], nt["BK"], nt["ring"]) == (256, 256, 64, 5)
    assert info(512, 512, 1024, True, BM=128, BN=128)["stages"] == 4
    assert info(512, 512, 1024, True, BM=256, BN=128)["stages"] == 3
    assert info(512, 512, 96, True, BM=128, BN=128)["BK"] == 32      # K is no multiple of 64
    assert info(512, 512, 64, True, BM=128, BN=128)["BK"] == 32      # a single 64-deep slab: nothing to pipeline
    for bad in (dict(BK=64, STAGES=3), dict(BK=64, RING=4), dict(BK=48)):
        with pytest.raises(ValueError):
            info(8192, 8192, 8192, True, **bad)
    with pytest.raises(ValueError):
        info(512, 512, 1024, True, BM=256, BN=128, BK=64, RING=5)    # the ring needs a square block tile
    ks = generate(matmulKernel(512, 512, 1024, DType.Float16, b_transposed=True))
    assert len(compile_source(ks.sources[0], "gemm_nt64.hip", use_cache=False)) > 1000
