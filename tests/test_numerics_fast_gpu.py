"""The backend's default numerics ("fast"): exp on the hardware exp2 and reciprocal on the hardware rcp, everything
else as under the Wasm-faithful numerics.  Bar: rel 1e-5 + abs 1e-7 against the Wasm-mode checker (the f32 map
tolerance; test/setup.ts toBeAllclose defaults), stated exceptions below.  Also: every kernel class compiled by hiprtc
on this machine (no on-disk code objects) and run."""
import numpy as np
import pytest

from gpu_util import WARM_ONLY, backend, fast_backend
from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker, numpyDtype
from jaxjs_hip.lowering import mapKernel, matmulKernel, matvecKernel, reduceKernel
from oracle import oracle

pytestmark = pytest.mark.gpu
F32 = DType.Float32


def run_on(be, kernel, inputs):
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(kernel, be if isinstance(be, str) else "fast").sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    exe = be.prepareKernelSync(kernel)
    slots = [be.malloc(np.ascontiguousarray(x).nbytes, np.ascontiguousarray(x).tobytes()) for x in inputs]
    out = be.malloc(kernel.bytes)
    try:
        be.dispatch(exe, slots, [out])
        return np.frombuffer(be.readSync(out), dtype=numpyDtype(kernel.dtype)).copy(), exe.data.ks
    finally:
        for s in slots + [out]:
            be.decRef(s)


def fast():
    return "fast" if WARM_ONLY else fast_backend()


def _map1(n, fn):
    return mapKernel([n], [(F32, ShapeTracker.fromShape([n]))], fn)


def test_exp_fast_against_checker_over_the_whole_range():
    rng = np.random.default_rng(11)
    x = np.concatenate([np.linspace(-104, 88.37, 200001), rng.normal(0, 4, 100000), rng.uniform(-1e-3, 1e-3, 1000),
                        [0.0, -0.0, 1.0, -1.0, 88.0, -87.0, -1000.0, 1000.0, np.inf, -np.inf, np.nan, 1e-30, -1e-30]]).astype(np.float32)
    k = _map1(x.size, lambda v: AluExp.exp(v))
    got, _ = run_on(fast(), k, [x])
    want = oracle.run_kernel(k, [x], oracle.MODE_WASM)
    # Exception 1: below 2^-126 the checker's polynomial returns 0 and the hardware a denormal: inside the 1e-7 abs.
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7, equal_nan=True)
    assert np.isnan(got[np.isnan(x)]).all() and got[x == np.inf][0] == np.inf and got[x == -np.inf][0] == 0
    assert got[x == 1000][0] == np.inf and got[x == -1000][0] == 0 and (got[x == 0] == 1).all()
    # and against exp itself: closer than the polynomial is (whose k*ln2 is rounded once)
    fin = np.isfinite(x) & (x > -87) & (x < 88.37)
    true = np.exp(x[fin].astype(np.float64))
    assert np.max(np.abs(got[fin] - true) / true) < 2e-6
    # Exception 2: x*log2(e) in [127.5, 128): the polynomial's `k > 127 -> Inf` fires although exp(x) < FLT_MAX;
    # the hardware path returns the finite value.
    band = np.linspace(88.38, 88.72, 50).astype(np.float32)
    kb = _map1(band.size, lambda v: AluExp.exp(v))
    gb, _ = run_on(fast(), kb, [band])
    assert np.all(np.isinf(oracle.run_kernel(kb, [band], oracle.MODE_WASM)))
    np.testing.assert_allclose(gb, np.exp(band.astype(np.float64)), rtol=2e-6)


def test_reciprocal_fast_against_checker():
    rng = np.random.default_rng(12)
    x = np.concatenate([rng.normal(0, 1, 100000), rng.uniform(-1e-6, 1e-6, 1000), 10.0 ** rng.uniform(-37, 37, 20000),
                        -(10.0 ** rng.uniform(-37, 37, 20000)), [1.0, -1.0, 3.0, 0.0, -0.0, np.inf, -np.inf, np.nan, 2.0 ** -126, 2.0 ** 126]]).astype(np.float32)
    k = _map1(x.size, lambda v: AluExp.reciprocal(v))
    got, _ = run_on(fast(), k, [x])
    want = oracle.run_kernel(k, [x], oracle.MODE_WASM)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7, equal_nan=True)
    assert got[x == 1.0][0] == 1.0 and np.signbit(got[-6]) and np.isinf(got[-6]) and got[-7] == np.inf  # 1/-0 = -Inf, 1/0 = Inf


def test_fused_softmax_style_row_kernel_fast():
    """The benchmark's sum(exp(x - m) * sigmoid(x)) row kernel: K-scaled bound against the f64 value and rel 1e-5
    against the Wasm-mode checker (a sum of positive terms that each meet the map tolerance)."""
    rows, L = 64, 4096
    rng = np.random.default_rng(13)
    X = rng.normal(0, 1, (rows, L)).astype(np.float32)
    m = X.max(axis=1)
    st = ShapeTracker.fromShape([rows, L])
    stm = ShapeTracker.fromShape([rows]).reshape([rows, 1]).expand([rows, L])

    def body(v, mm):
        sig = AluExp.reciprocal(AluExp.add(AluExp.exp(AluExp.sub(AluExp.f32(0), v)), AluExp.f32(1)))
        return AluExp.mul(AluExp.exp(AluExp.add(v, AluExp.sub(AluExp.f32(0), mm))), sig)
    k = reduceKernel([rows, L], [(F32, st), (F32, stm)], body, AluOp.Add)
    got, ks = run_on(fast(), k, [X, m])
    assert ks.klass == "reduce_row"
    want = oracle.run_kernel(k, [X, m], oracle.MODE_WASM)
    np.testing.assert_allclose(got, want, rtol=1e-5)
    x64 = X.astype(np.float64)
    ref = np.sum(np.exp(x64 - m[:, None]) / (1 + np.exp(-x64)), axis=1)
    np.testing.assert_allclose(got, ref, rtol=1e-5)


def test_library_compositions_fast():
    """sigmoid, tanh (exp(+-2x) form) and the tanh-gelu as the library composes them (src/library/nn.ts:65-67, 222-238),
    fast numerics against the Wasm-mode checker replaying the same program."""
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as Lb
    from jaxjs_hip.jit import ShapedArray
    from jit_util import run_program
    from oracle.backend import OracleBackend
    x = np.concatenate([np.linspace(-12, 12, 4001), [0.0, 1e-4, -1e-4, 30.0, -30.0]]).astype(np.float32)
    for fn, atol in ((Lb.sigmoid, 1e-7), (Lb.tanh, 3e-7), (Lb.gelu, 1e-6)):
        prog = J.jit(lambda a: fn(a), [ShapedArray(x.shape, F32)])
        if WARM_ONLY:
            from test_programs_gpu import warm
            warm(prog)
        (got,) = run_program(fast_backend(), prog, [x])
        (want,) = run_program(OracleBackend(), prog, [x])
        # tanh and gelu subtract two exps of nearly equal size near 0: one ulp of either is `atol` of the result
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=atol)


CASES = [
    ("map", "map", mapKernel([70, 33], [(F32, ShapeTracker.fromShape([70, 33]))], lambda x: AluExp.sin(x)), F32, 1e-5),
    ("reduce_row", "reduce_row", reduceKernel([64, 4096], [(F32, ShapeTracker.fromShape([64, 4096]))], lambda x: x, AluOp.Max), F32, 0),
    ("reduce_col", "reduce_col", reduceKernel([4096, 64], [(DType.Int32, ShapeTracker.fromShape([64, 4096]).permute([1, 0]))], lambda x: x, AluOp.Add), DType.Int32, 0),
    ("fold", "reduce_row+fold", reduceKernel([1, 1 << 22], [(F32, ShapeTracker.fromShape([1, 1 << 22]))], lambda x: x, AluOp.Add), F32, 1e-4),
    ("matvec", "reduce_row", matvecKernel(1024, 512, DType.Float16), DType.Float16, 1e-2),
    ("matvec_t", "reduce_col+fold", matvecKernel(11008, 2048, DType.Float16, w_transposed=True), DType.Float16, 1e-2),
    ("gemm_dlds", "gemm", matmulKernel(256, 256, 128, DType.Float16), DType.Float16, 1e-2),
    ("gemm_dlds_ring", "gemm", matmulKernel(256, 256, 256, DType.Float16, b_transposed=True), DType.Float16, 1e-2),
    ("gemm_ragged", "gemm", matmulKernel(100, 72, 40, DType.Float16), DType.Float16, 1e-2),
    ("gemm_f32", "gemm", matmulKernel(128, 128, 64, F32), F32, 1e-4),
]


@pytest.mark.parametrize("name,klass,kernel,dt,rtol", CASES, ids=[c[0] for c in CASES])
def test_every_class_compiles_with_hiprtc_on_this_machine(name, klass, kernel, dt, rtol, monkeypatch):
    """No code object from the on-disk cache: the source of each kernel class goes through hiprtc here, is loaded and
    run, and matches the checker."""
    if WARM_ONLY:
        pytest.skip("warm-up run: this test compiles on the GPU machine on purpose")
    import jaxjs_hip.backend as B
    from jaxjs_hip import runtime
    backend()
    monkeypatch.setattr(runtime, "DISK_CACHE", False)
    compiled = []
    orig = B.compile_source

    def counting(src, nm="kernel.hip", *a, **kw):
        assert kw.get("use_cache") is None and not runtime.DISK_CACHE
        compiled.append(nm)
        return orig(src, nm, *a, **kw)
    monkeypatch.setattr(B, "compile_source", counting)
    be = B.HipBackend(numerics="wasm")  # its in-memory cache is empty: prepare must compile
    exe = be.prepareKernelSync(kernel)
    assert compiled and exe.data.ks.klass == klass, (compiled, exe.data.ks.klass)
    need = exe.data.ks.min_input_bytes
    rng = np.random.default_rng(14)
    host = []
    for gid in range(kernel.nargs):
        nbytes = need.get(gid, 0)
        if dt == DType.Int32:
            host.append(rng.integers(-100, 100, nbytes // 4).astype(np.int32))
        elif dt == DType.Float16:
            host.append(rng.normal(0, 0.5, nbytes // 2).astype(np.float16))
        else:
            host.append(rng.normal(0, 0.5, nbytes // 4).astype(np.float32))
    got, ks = run_on(be, kernel, host)
    want = oracle.run_kernel(kernel, host, oracle.MODE_WASM)
    if rtol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=rtol, atol=rtol)
    be.clearCache()
