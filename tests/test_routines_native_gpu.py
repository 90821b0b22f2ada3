"""Scatter, TriangularSolve, Cholesky, LU, JacobiEigh and Fft as GPU kernels against the CPU checker.

The linear-algebra kernels keep the reference's arithmetic (double scalars, stores rounded to the element type --
float32, float64 or float16 --, the same order per stored element), so their results must be bit-identical to the checker's.  Scatter is bit-identical except float
accumulation onto repeated destinations (atomic adds in any order: compared within a sum-scaled bound).  Fft takes
its sines and cosines from the device math library, whose last-place differences from the host's can decide a
float32 rounding tie in a butterfly (seen for radix-3 stages behind an even stride; power-of-two and prime sizes come
out bit-identical): compared within 1e-5 of the row's largest magnitude."""
import numpy as np
import pytest

import routine_util as R
from jaxjs_hip import DType
from jaxjs_hip.errors import UnsupportedRoutineError

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(77)
F32 = np.float32


def both(routine, arrays):
    got, ks = R.run_gpu(routine, arrays)
    return got, R.run_oracle(routine, arrays), ks


def assert_bits(got, want, what=""):
    for i, (g, w) in enumerate(zip(got, want)):
        if not R.bits_equal(g, w):
            bad = np.flatnonzero((g.reshape(-1) != w.reshape(-1)) & ~(np.isnan(g.reshape(-1)) & np.isnan(w.reshape(-1)))) if g.dtype.kind == "f" else np.flatnonzero(g.reshape(-1) != w.reshape(-1))
            raise AssertionError(f"{what} output {i}: {len(bad)} of {g.size} elements differ; first at {bad[:5]}: "
                                 f"{g.reshape(-1)[bad[:5]]} vs {w.reshape(-1)[bad[:5]]}")


def spd(batch, n):
    a = RNG.standard_normal(batch + (n, n))
    return (a @ np.swapaxes(a, -1, -2) + n * np.eye(n)).astype(F32)


@pytest.mark.parametrize("shape", [(1, 1), (2, 2), (3, 3), (5, 17, 17), (2, 3, 64, 64), (191, 191), (192, 192), (200, 200), (2, 333, 333),
                                   (1100, 1100), (2048, 2048)], ids=str)
def test_cholesky(shape):
    x = spd(tuple(shape[:-2]), shape[-1])
    x = x + np.triu(RNG.standard_normal(x.shape), 1).astype(F32)  # the upper triangle must not matter
    got, want, ks = both(R.cholesky(x), [x])
    assert ("panels" in ks.info) == (shape[-1] >= 192)  # large matrices run panel by panel over the whole chip
    assert_bits(got, want, f"cholesky {shape} {ks.info}")


@pytest.mark.parametrize("shape", [(200, 200), (2, 333, 333), (1100, 1100)], ids=str)
def test_cholesky_left_looking_panels_when_the_double_copy_is_too_large(shape, monkeypatch):
    """The right-looking variant keeps a double-precision copy of every matrix; beyond its size limit the left-looking
    panels run instead.  Same sums in the same order: identical bits."""
    from jaxjs_hip import routinegen
    x = spd(tuple(shape[:-2]), shape[-1])
    right, k1 = R.run_gpu(R.cholesky(x), [x])
    monkeypatch.setattr(routinegen, "CHOLESKY_RIGHT_LOOKING_MAX_BYTES", 0)
    from gpu_util import backend
    backend().clearCache()  # prepared routines are cached by structure: the limit is read when a plan is generated
    left, k2 = R.run_gpu(R.cholesky(x), [x])
    backend().clearCache()
    assert k1.info.get("variant") == "right-looking" and "variant" not in k2.info and "panels" in k2.info
    assert_bits(left, right, f"cholesky variants {shape}")


def test_cholesky_not_positive_definite_and_empty():
    x = np.array([[[1, 2], [2, 1]], [[4, 2], [2, 3]]], F32)
    got, want, _ = both(R.cholesky(x), [x])
    assert np.isnan(got[0][0, 1, 1]) and got[0][1, 1, 1] == np.float32(np.sqrt(2.0))
    assert_bits(got, want)
    big = spd((), 256)
    big[100, 100] = -5.0  # pivot 100 goes negative: NaNs from there on, in the same places, also panel by panel
    got, want, ks = both(R.cholesky(big), [big])
    assert "panels" in ks.info and np.isnan(got[0][100, 100]) and np.isfinite(got[0][:100, :100]).all()
    assert_bits(got, want, "non-PD through panels")
    e = np.zeros((0, 4, 4), F32)
    got, _ = R.run_gpu(R.cholesky(e), [e])
    assert got[0].shape == (0, 4, 4)
    with pytest.raises(ValueError):
        R.run_gpu(R.cholesky(np.zeros((2, 3), F32)), [np.zeros((2, 3), F32)])


@pytest.mark.parametrize("case", [((2, 2), 1), ((9, 9), 4), ((3, 30, 30), 7), ((2, 2, 16, 16), 100), ((300, 300), 300), ((64, 64), 1000),
                                  ((2, 131, 131), 70), ((128, 128), 3), ((1024, 1024), 64)], ids=str)
@pytest.mark.parametrize("unit", [False, True])
def test_triangular_solve(case, unit):
    ashape, m = case
    n = ashape[-1]
    a = (np.triu(RNG.standard_normal(ashape)) * (0.3 if unit else 1.0) + (0 if unit else 1) * np.sqrt(n) * np.eye(n)
         + np.tril(RNG.standard_normal(ashape), -1)).astype(F32)  # the strictly lower part must not matter
    b = RNG.standard_normal(ashape[:-2] + (m, n)).astype(F32)
    got, want, ks = both(R.triangular_solve(a, b, unit), [a, b])
    assert ks.info["staged"] == (n >= 128)  # from 128 on helper waves stage the matrix in LDS as doubles
    assert_bits(got, want, f"triangular_solve {case} {ks.info}")


@pytest.mark.parametrize("shape", [(2, 2), (1, 5), (5, 1), (2, 7, 5), (3, 12, 20), (2, 2, 30, 30), (150, 97), (260, 300), (255, 400),
                                   (2, 300, 256), (513, 300), (1024, 1024)], ids=str)
def test_lu(shape):
    a = RNG.uniform(-1, 1, shape).astype(F32)
    got, want, ks = both(R.lu(a), [a])
    # from 192 rows and columns on: two launches per column, the trailing update over the whole chip
    assert (ks.info.get("variant") == "by columns") == (min(shape[-2:]) >= 192)
    assert_bits(got, want, f"lu {shape} {ks.info}")


def test_lu_by_columns_zero_pivot_and_nan_columns():
    """The special cases of the small kernel's test, embedded in matrices large enough for the by-columns variant: a zero
    pivot column (that step eliminates nothing), equal magnitudes (the first row wins), a NaN that must not win."""
    a = RNG.uniform(-1, 1, (2, 260, 260)).astype(F32)
    a[0, :, 3] = 0.0   # stays zero through every update: step 3 meets a zero pivot
    a[1, 10, 5] = np.nan
    a[1, 20:23, 7] = [0.75, -0.75, 0.75]
    got, want, ks = both(R.lu(a), [a])
    assert ks.info["variant"] == "by columns"
    assert_bits(got, want, "lu by columns, special columns")


def test_lu_ties_zero_pivots_and_nans():
    a = np.array([[[1, 2, 3], [-1, 5, 6], [1, 8, 9]],      # equal magnitudes: the first row wins
                  [[0, 1, 2], [0, 2, 3], [0, 5, 1]],       # zero pivot column: nothing eliminated in that step
                  [[np.nan, 1, 2], [3, 2, 3], [4, 5, 1]],  # NaN in the starting row keeps it
                  [[1, 1, 2], [np.nan, 2, 3], [4, 5, 1]]], F32)  # NaN elsewhere never wins
    got, want, _ = both(R.lu(a), [a])
    assert_bits(got, want, "lu special rows")
    got, want, _ = both(R.lu(np.zeros((2, 3, 0), F32)), [np.zeros((2, 3, 0), F32)])
    assert got[2].tolist() == [[0, 1, 2]] * 2
    assert_bits(got, want)


@pytest.mark.parametrize("shape", [(1, 1), (2, 2), (3, 3), (4, 20, 20), (2, 64, 64), (100, 100), (2, 128, 128), (150, 150)], ids=str)
def test_jacobi_eigh(shape):
    a = RNG.standard_normal(shape)
    sym = (a + np.swapaxes(a, -1, -2)).astype(F32) + np.triu(RNG.standard_normal(shape), 1).astype(F32)
    got, want, ks = both(R.jacobi_eigh(sym), [sym])
    assert ks.info["in_lds"] == (shape[-1] <= 138)
    assert_bits(got, want, f"jacobi_eigh {shape} {ks.info}")


def test_jacobi_eigh_sweep_limits_and_special_values():
    a = RNG.standard_normal((3, 12, 12))
    sym = (a + np.swapaxes(a, -1, -2)).astype(F32)
    for sweeps, tol in ((0, 1e-7), (1, 1e-7), (2, 0.0), (30, 1e-3)):
        got, want, _ = both(R.jacobi_eigh(sym, sweeps, tol), [sym])
        assert_bits(got, want, f"maxSweeps={sweeps} tolerance={tol}")
    d = np.diag(np.array([3, 1, 2], F32))
    got, want, _ = both(R.jacobi_eigh(d), [d])
    assert np.diagonal(got[0]).tolist() == [3, 1, 2]
    assert_bits(got, want)
    bad = sym.copy()
    bad[1, 5, 2] = np.nan  # a NaN makes the threshold NaN: no sweep runs (Math.max propagates it)
    got, want, _ = both(R.jacobi_eigh(bad), [bad])
    assert_bits(got, want, "NaN input")


@pytest.mark.parametrize("n", [1, 2, 3, 4, 8, 12, 30, 49, 64, 11, 97, 210, 1024, 4096, 1009])
@pytest.mark.parametrize("inverse", [False, True])
def test_fft(n, inverse):
    rows = (2, 3) if n < 1000 else (3,)
    re, im = RNG.standard_normal(rows + (n,)).astype(F32), RNG.standard_normal(rows + (n,)).astype(F32)
    got, want, ks = both(R.fft(re, im, inverse), [re, im])
    scale = max(np.abs(want[0]).max(), np.abs(want[1]).max())
    for g, w in zip(got, want):
        np.testing.assert_allclose(g, w, rtol=0, atol=1e-5 * scale, err_msg=str(ks.info))


@pytest.mark.parametrize("shape", [(3, 8), (2, 60), (1, 1000), (5, 1024), (70, 4096), (2, 8192)], ids=str)
def test_fft_single_launch_and_staged_paths_give_the_same_bits(shape):
    """Short rows run in one launch with the stages in LDS, long or few rows one launch per stage through HBM: the
    same operations per element in the same order, so not a bit may differ (forward and inverse)."""
    from jaxjs_hip.routine import Routine
    re, im = RNG.standard_normal(shape).astype(F32), RNG.standard_normal(shape).astype(F32)
    for inverse in (False, True):
        base = R.fft(re, im, inverse)
        one = Routine(base.name, base.type, dict(base.params, singleLaunch=True))
        many = Routine(base.name, base.type, dict(base.params, singleLaunch=False))
        a, ka = R.run_gpu(one, [re, im])
        b, kb = R.run_gpu(many, [re, im])
        assert ka.info["launches"] == 1 and kb.info["launches"] == 1 + len(base.params["factors"])
        assert_bits(a, b, f"{shape} inverse={inverse}")


def test_fft_factor_orders_and_validation():
    re, im = RNG.standard_normal((2, 60)).astype(F32), RNG.standard_normal((2, 60)).astype(F32)
    for factors in ([4, 3, 5], [5, 3, 4], [2, 2, 15], [60]):
        got, want, _ = both(R.fft(re, im, False, factors), [re, im])
        for g, w in zip(got, want):
            np.testing.assert_allclose(g, w, rtol=0, atol=1e-5 * np.abs(w).max())
    with pytest.raises(ValueError):
        R.run_gpu(R.fft(re, im, False, [4, 4]), [re, im])


# ---- float64 and float16 elements: the same kernels with another stored type (every kernel variant once per type)
ELEMS = [np.float64, np.float16]


@pytest.mark.parametrize("dt", ELEMS, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("shape", [(3, 3), (2, 3, 64, 64), (200, 200), (2, 333, 333)], ids=str)
def test_cholesky_other_element_types(shape, dt, monkeypatch):
    n = shape[-1]
    x = (spd(tuple(shape[:-2]), n).astype(np.float64) / (1.0 if dt == np.float64 else n)).astype(dt)
    got, want, ks = both(R.cholesky(x), [x])
    assert got[0].dtype == dt and ("panels" in ks.info) == (n >= 192)
    assert_bits(got, want, f"cholesky {shape} {np.dtype(dt).name} {ks.info}")
    if n >= 192:  # and the left-looking panels
        from jaxjs_hip import routinegen
        from gpu_util import backend
        monkeypatch.setattr(routinegen, "CHOLESKY_RIGHT_LOOKING_MAX_BYTES", 0)
        backend().clearCache()
        left, k2 = R.run_gpu(R.cholesky(x), [x])
        backend().clearCache()
        assert "variant" not in k2.info and "panels" in k2.info
        assert_bits(left, want, f"cholesky left-looking {shape} {np.dtype(dt).name}")


@pytest.mark.parametrize("dt", ELEMS, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("case", [((9, 9), 4), ((2, 2, 16, 16), 100), ((2, 131, 131), 70), ((300, 300), 300)], ids=str)
@pytest.mark.parametrize("unit", [False, True])
def test_triangular_solve_other_element_types(case, unit, dt):
    ashape, m = case
    n = ashape[-1]
    a = (np.triu(RNG.standard_normal(ashape)) * (0.3 if unit else 1.0) + (0 if unit else 1) * np.sqrt(n) * np.eye(n)
         + np.tril(RNG.standard_normal(ashape), -1)).astype(dt)
    b = RNG.standard_normal(ashape[:-2] + (m, n)).astype(dt)
    got, want, ks = both(R.triangular_solve(a, b, unit), [a, b])
    assert got[0].dtype == dt and ks.info["staged"] == (n >= 128)
    assert_bits(got, want, f"triangular_solve {case} {np.dtype(dt).name} {ks.info}")


@pytest.mark.parametrize("dt", ELEMS, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("shape", [(2, 7, 5), (3, 12, 20), (150, 97), (260, 300), (2, 300, 256)], ids=str)
def test_lu_other_element_types(shape, dt):
    a = RNG.uniform(-1, 1, shape).astype(dt)
    if shape == (260, 300):
        a[:, 3] = 0       # a zero pivot column
        a[10, 5] = np.nan  # a NaN that must not win the pivot search
        a[20:23, 7] = [0.75, -0.75, 0.75]
    got, want, ks = both(R.lu(a), [a])
    assert got[0].dtype == dt and (ks.info.get("variant") == "by columns") == (min(shape[-2:]) >= 192)
    assert_bits(got, want, f"lu {shape} {np.dtype(dt).name} {ks.info}")


@pytest.mark.parametrize("dt", ELEMS, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("shape", [(2, 2), (4, 20, 20), (2, 64, 64), (100, 100), (150, 150)], ids=str)
def test_jacobi_eigh_other_element_types(shape, dt):
    a = RNG.standard_normal(shape)
    sym = (a + np.swapaxes(a, -1, -2)).astype(dt) + np.triu(RNG.standard_normal(shape), 1).astype(dt)
    tol = 1e-14 if dt == np.float64 else 1e-3
    got, want, ks = both(R.jacobi_eigh(sym, 30 if dt == np.float64 else 6, tol), [sym])
    eb = np.dtype(dt).itemsize
    assert got[0].dtype == dt and ks.info["in_lds"] == (2 * shape[-1] ** 2 * eb <= 150 * 1024)
    assert_bits(got, want, f"jacobi_eigh {shape} {np.dtype(dt).name} {ks.info}")


@pytest.mark.parametrize("dt", ELEMS, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("n", [1, 4, 12, 49, 97, 210, 1024, 4096])
def test_fft_other_element_types(n, dt):
    """float64 results carry the device sine/cosine's last-place differences from the host's unrounded: compared within
    1e-13 of the row's magnitude per stage; float16 within one unit of its last place of that magnitude."""
    from jaxjs_hip.routine import Routine
    rows = (2, 3) if n < 1000 else (70,)
    re, im = RNG.standard_normal(rows + (n,)).astype(dt), RNG.standard_normal(rows + (n,)).astype(dt)
    for inverse in (False, True):
        base = R.fft(re, im, inverse)
        got, want, ks = both(base, [re, im])
        scale = float(max(np.abs(want[0].astype(np.float64)).max(), np.abs(want[1].astype(np.float64)).max()))
        atol = (1e-13 * max(1, len(base.params["factors"])) if dt == np.float64 else 1e-3) * scale
        for g, w in zip(got, want):
            assert g.dtype == dt
            np.testing.assert_allclose(g.astype(np.float64), w.astype(np.float64), rtol=0, atol=atol, err_msg=str(ks.info))
        if n <= (4096 if dt == np.float64 else 8192) and n > 1:  # single launch and one launch per stage: the same bits
            one = Routine(base.name, base.type, dict(base.params, singleLaunch=True))
            many = Routine(base.name, base.type, dict(base.params, singleLaunch=False))
            a, ka = R.run_gpu(one, [re, im])
            b, kb = R.run_gpu(many, [re, im])
            assert ka.info["launches"] == 1 and kb.info["launches"] == 1 + len(base.params["factors"])
            assert_bits(a, b, f"fft paths n={n} {np.dtype(dt).name} inverse={inverse}")


def _sc(updates, indices, op, shape, axis, out_dim, unique=False, dtype=None):
    return R.scatter(updates, indices, op, shape, axis, out_dim, unique, dtype), [updates] + list(indices)


def test_scatter_reference_tables():
    i32 = lambda x: np.array(x, np.int32)  # noqa: E731
    cases = [
        _sc(np.array([[10, 20], [30, 40], [50, 60]], F32), [i32([1, 3]), i32([0, 1])], "update", [2, 3, 4], [2, 0], 1, True),
        _sc(np.array([1, 2, 3], F32), [i32([1, 1, 3])], "add", [4], [0], 0),
        _sc(np.array([1, 2, 3, 4], np.float16), [i32([0, 1, 0, 1])], "add", [2], [0], 0),
        _sc(np.array([1, 2, 3], np.int32), [i32([1, 1, 3])], "add", [4], [0], 0),
        _sc(np.array([1, 2, 3], np.uint32), [i32([1, 1, 3])], "add", [4], [0], 0),
        _sc(np.array([0, 1, 1], np.int32), [i32([1, 1, 3])], "add", [4], [0], 0, dtype=DType.Bool),
        _sc(np.array([10, 20, 30], F32), [i32([3, 0, 2])], "add", [4], [0], 0, True),
        _sc(np.array([[1, 2, 3], [4, 5, 6]], F32), [i32([[0], [2]]), i32([[0, 1, 1]])], "add", [3, 4], [0, 1], 0),
    ]
    expected = [[[[0, 10, 0, 0], [0, 30, 0, 0], [0, 50, 0, 0]], [[0, 0, 0, 20], [0, 0, 0, 40], [0, 0, 0, 60]]],
                [0, 3, 0, 3], [4, 6], [0, 3, 0, 3], [0, 3, 0, 3], [0, 1, 0, 1], [20, 0, 30, 10],
                [[1, 5, 0, 0], [0, 0, 0, 0], [4, 11, 0, 0]]]
    for (routine, arrays), exp in zip(cases, expected):
        got, want, _ = both(routine, arrays)
        np.testing.assert_array_equal(got[0], np.array(exp))
        assert_bits(got, want)


SCATTER_CASES = [
    ((7,), [(7,)], (5,), [0], 0),
    ((6, 3), [(6,)], (4, 3), [0], 0),
    ((3, 6), [(6,)], (3, 4), [1], 1),
    ((2, 5, 3), [(5,), (5,)], (2, 4, 6, 3), [1, 2], 1),
    ((4, 3, 2), [(4, 1), (1, 3)], (5, 2, 5), [2, 0], 0),
    ((2, 2, 3, 2), [(2, 3)], (2, 6, 2), [1], 1),
    ((5000, 8), [(5000,)], (300, 8), [0], 0),       # many repeated destinations
    ((100000,), [(100000,)], (1000003,), [0], 0),   # sparse
]


@pytest.mark.parametrize("case", SCATTER_CASES, ids=lambda c: "x".join(map(str, c[0])))
@pytest.mark.parametrize("op", ["add", "update"])
@pytest.mark.parametrize("dtype", [DType.Float32, DType.Int32, DType.Uint32, DType.Float16, DType.Bool, DType.Float64], ids=lambda d: d.value)
def test_scatter_random(case, op, dtype):
    ushape, ishapes, oshape, axis, out_dim = case
    npdt = {DType.Float32: F32, DType.Int32: np.int32, DType.Uint32: np.uint32, DType.Float16: np.float16, DType.Bool: np.int32,
            DType.Float64: np.float64}[dtype]
    if dtype == DType.Bool:
        upd = RNG.integers(0, 2, ushape).astype(npdt)
    elif dtype in (DType.Int32, DType.Uint32):
        upd = RNG.integers(0, 1 << 32, ushape, dtype=np.uint64).astype(np.uint32).view(npdt).reshape(ushape)  # sums wrap
    else:
        upd = RNG.integers(-9, 10, ushape).astype(npdt)  # small integers: float sums are exact in any order
    idx = [RNG.integers(-1, oshape[a] + 1, s).astype(np.int32) for s, a in zip(ishapes, axis)]  # some out of range
    got, want, ks = both(*_sc(upd, idx, op, list(oshape), axis, out_dim, dtype=dtype))
    assert_bits(got, want, f"scatter {case} {op} {dtype} {ks.info}")


def test_scatter_float_accumulation_within_bound_and_unique_promise():
    upd = RNG.standard_normal((20000,)).astype(F32)
    idx = RNG.integers(0, 50, (20000,)).astype(np.int32)
    got, want, _ = both(*_sc(upd, [idx], "add", [50], [0], 0))
    bound = np.zeros(50)
    np.add.at(bound, idx, np.abs(upd))
    assert np.all(np.abs(got[0].astype(np.float64) - want[0]) <= 400 * 2.0 ** -24 * bound + 1e-30)  # ~K/50 adds per slot
    perm = RNG.permutation(1000).astype(np.int32)
    vals = RNG.standard_normal((1000, 4)).astype(F32)
    for op in ("add", "update"):
        got, want, ks = both(*_sc(vals, [perm], op, [1000, 4], [0], 0, True))
        assert ks.info["mode"] == 0
        assert_bits(got, want)
    with pytest.raises(UnsupportedRoutineError):
        R.run_gpu(*_sc(np.zeros(3, F32), [np.zeros(3, F32)], "add", [4], [0], 0))  # index arrays must be integers


def test_outputs_are_fully_initialised_without_updates():
    got, want, _ = both(*_sc(np.zeros((0, 3), F32), [np.zeros((0,), np.int32)], "add", [4, 3], [0], 0))
    assert np.all(got[0] == 0)
    assert_bits(got, want)
