"""Native Sort / Argsort routines on the GPU against the reference's tables (test/numpy.test.ts:4631-4800) and
against the CPU checker's restatement of src/routine.ts:185-213 on random data."""
import numpy as np
import pytest

from gpu_util import WARM_ONLY, backend
from jaxjs_hip import DType
from jaxjs_hip.alu import numpyDtype
from jaxjs_hip.errors import UnsupportedRoutineError
from jaxjs_hip.routine import Routine, Routines, RoutineType
from oracle.routines import runCpuRoutine

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(21)


def make(name, shape, dtype):
    shape = list(shape)
    if name == Routines.Sort:
        return Routine(name, RoutineType([shape], [dtype], [shape], [dtype]))
    return Routine(name, RoutineType([shape], [dtype], [shape, shape], [dtype, DType.Int32]))


def run(name, x, dtype):
    routine = make(name, x.shape, dtype)
    if WARM_ONLY:
        from jaxjs_hip.routinegen import generateRoutine
        from jaxjs_hip.runtime import compile_source
        ks = generateRoutine(routine)
        for src in (ks.sources if ks else []):
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    exe = be.prepareRoutineSync(routine)
    src = be.malloc(x.nbytes, x.tobytes())
    outs = [be.malloc(x.size * 4 if i == 1 else x.nbytes) for i in range(len(routine.type.outputShapes))]
    be.dispatch(exe, [src], outs)
    got = [np.frombuffer(be.readSync(o), dtype=numpyDtype(dt)).reshape(x.shape).copy()
           for o, dt in zip(outs, routine.type.outputDtypes)]
    for s in [src] + outs:
        be.decRef(s)
    host_out = [bytearray(x.nbytes)] + ([bytearray(x.size * 4)] if name == Routines.Argsort else [])
    runCpuRoutine(routine, [x.tobytes()], host_out)
    want = [np.frombuffer(bytes(b), dtype=numpyDtype(dt)).reshape(x.shape) for b, dt in zip(host_out, routine.type.outputDtypes)]
    return got, want


def test_sort_tables():
    (y,), _ = run(Routines.Sort, np.array([3, 1, 4, 1, 5, 9, 2, 6], np.float32), DType.Float32)
    np.testing.assert_array_equal(y, [1, 1, 2, 3, 4, 5, 6, 9])
    (y,), _ = run(Routines.Sort, np.array([[3, 1, 2], [6, 4, 5]], np.float32), DType.Float32)
    np.testing.assert_array_equal(y, [[1, 2, 3], [4, 5, 6]])
    (y,), _ = run(Routines.Sort, np.array([3, np.nan, 1, np.nan, 2], np.float32), DType.Float32)
    np.testing.assert_array_equal(y, np.array([1, 2, 3, np.nan, np.nan], np.float32))
    for dt, npdt in ((DType.Int32, np.int32), (DType.Uint32, np.uint32)):
        (y,), _ = run(Routines.Sort, np.array([3, 1, 4, 1, 5], npdt), dt)
        np.testing.assert_array_equal(y, [1, 1, 3, 4, 5])
    (y,), _ = run(Routines.Sort, np.array([1, 0, 1, 0, 1], np.int32), DType.Bool)
    np.testing.assert_array_equal(y, [0, 0, 1, 1, 1])
    x = np.linspace(0, 1, 8192).astype(np.float32)
    (y,), _ = run(Routines.Sort, x[::-1].copy(), DType.Float32)
    np.testing.assert_array_equal(y, x)


def test_argsort_tables_and_stability():
    (v, i), _ = run(Routines.Argsort, np.array([3, 1, 4, 2, 5], np.float32), DType.Float32)
    np.testing.assert_array_equal(i, [1, 3, 0, 2, 4])
    assert i.dtype == np.int32
    (v, i), _ = run(Routines.Argsort, np.array([[3, 1, 2], [6, 4, 5]], np.float32), DType.Float32)
    np.testing.assert_array_equal(i, [[1, 2, 0], [1, 2, 0]])
    x = np.array([3, 1, 1, np.nan, np.inf, 2, np.nan, 1, 0, -0.0, np.inf], np.float32)
    (v, i), _ = run(Routines.Argsort, x, DType.Float32)
    np.testing.assert_array_equal(i, [8, 9, 1, 2, 7, 5, 0, 4, 10, 3, 6])
    np.testing.assert_array_equal(v.view(np.uint32), x[i].view(np.uint32))  # original values, bit for bit (signed zero, NaN payload)
    x = np.linspace(0, 1, 8191).astype(np.float32)[::-1].copy()
    (v, i), _ = run(Routines.Argsort, x, DType.Float32)
    np.testing.assert_array_equal(i, np.arange(8190, -1, -1))


def _data(shape, dtype):
    if dtype in (DType.Float32, DType.Float16, DType.Float64):
        x = RNG.normal(0, 10, shape).astype(numpyDtype(dtype))
        if dtype == DType.Float64:  # keys that differ only below float32 resolution
            x += RNG.integers(-3, 4, shape) * 2.0 ** -40
        flat = x.reshape(-1)
        n = flat.size
        if n >= 8:
            picks = RNG.integers(0, n, max(n // 50, 4))
            flat[picks[0::4]] = np.nan
            flat[picks[1::4]] = np.inf
            flat[picks[2::4]] = -np.inf
            flat[picks[3::4]] = -0.0
            flat[RNG.integers(0, n, max(n // 10, 2))] = 1.5  # many duplicates: exercises stability
        return x
    if dtype == DType.Int32:
        return RNG.integers(-50, 50, shape).astype(np.int32)
    if dtype == DType.Uint32:
        return RNG.integers(0, 1 << 32, shape, dtype=np.uint64).astype(np.uint32)
    return RNG.integers(0, 2, shape).astype(np.int32)  # bool storage


SHAPES = [(1,), (2,), (7, 3), (5, 100), (3, 2048), (4, 4096), (2, 5000), (33, 8192), (2, 8193), (3, 100000), (1, (1 << 17) + 3), (1000, 17)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype", [DType.Float32, DType.Int32, DType.Uint32, DType.Float16, DType.Bool, DType.Float64], ids=lambda d: d.value)
def test_sort_matches_host_routine(shape, dtype):
    x = _data(shape, dtype)
    (y,), (want,) = run(Routines.Sort, x, dtype)
    np.testing.assert_array_equal(y, want)  # NaNs compare equal position-wise; -0 sorts before +0 on both sides
    if x.dtype.kind == "f":  # signed zeros land in the same places
        ok = ~np.isnan(want)
        np.testing.assert_array_equal(np.signbit(y[ok]), np.signbit(want[ok]))


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype", [DType.Float32, DType.Int32, DType.Float16, DType.Float64], ids=lambda d: d.value)
def test_argsort_matches_host_routine(shape, dtype):
    x = _data(shape, dtype)
    (v, i), (wv, wi) = run(Routines.Argsort, x, dtype)
    np.testing.assert_array_equal(i, wi)
    np.testing.assert_array_equal(v.view(np.uint8), wv.view(np.uint8))


def test_zero_sized_rows_and_unsupported_dtype_path():
    if WARM_ONLY:
        pytest.skip("nothing to compile")
    be = backend()
    routine = make(Routines.Sort, (3, 0), DType.Float32)
    exe = be.prepareRoutineSync(routine)
    a, b = be.malloc(0), be.malloc(0)
    be.dispatch(exe, [a], [b])
    assert be.readSync(b) == b""
    be.decRef(a)
    be.decRef(b)
    # An element type a routine's kernels do not cover is refused at prepare time, never run on the host.
    import routine_util as R
    with pytest.raises(UnsupportedRoutineError):
        be.prepareRoutineSync(R.routine_for(Routines.Cholesky, [np.zeros((4, 4), np.int32)], [(4, 4)], [DType.Int32]))
