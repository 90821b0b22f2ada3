"""Pins the CPU checker of the routines (oracle/routines.py, oracle/routines_oracle.c) before the GPU tests trust it:
the tables of the reference's own tests (src/frontend/array.test.ts:52-176 scatter; test/lax-linalg.test.ts:23-55,
140-167, 276-289, 332-436; test/numpy-fft.test.ts:60-100, 165-175), identities the mathematics fixes, independent
library routines (numpy.linalg, numpy.fft, scipy.linalg) and brute force on small inputs."""
import itertools

import numpy as np
import pytest
import scipy.linalg

import routine_util as R
from jaxjs_hip import DType

RNG = np.random.default_rng(5)
F32 = np.float32


def test_scatter_reference_tables():
    i32 = lambda x: np.array(x, np.int32)  # noqa: E731
    (out,) = R.run_oracle(*_sc(np.array([[10, 20], [30, 40], [50, 60]], F32), [i32([1, 3]), i32([0, 1])], "update", [2, 3, 4], [2, 0], 1, True))
    np.testing.assert_array_equal(out, [[[0, 10, 0, 0], [0, 30, 0, 0], [0, 50, 0, 0]], [[0, 0, 0, 20], [0, 0, 0, 40], [0, 0, 0, 60]]])
    (out,) = R.run_oracle(*_sc(np.array([1, 2, 3], F32), [i32([1, 1, 3])], "add", [4], [0], 0))
    np.testing.assert_array_equal(out, [0, 3, 0, 3])
    (out,) = R.run_oracle(*_sc(np.array([1, 2, 3, 4], np.float16), [i32([0, 1, 0, 1])], "add", [2], [0], 0))
    np.testing.assert_array_equal(out, [4, 6])
    for dt, npdt in ((DType.Int32, np.int32), (DType.Uint32, np.uint32)):
        (out,) = R.run_oracle(*_sc(np.array([1, 2, 3], npdt), [i32([1, 1, 3])], "add", [4], [0], 0))
        np.testing.assert_array_equal(out, [0, 3, 0, 3])
    (out,) = R.run_oracle(*_sc(np.array([0, 1, 1], np.int32), [i32([1, 1, 3])], "add", [4], [0], 0, dtype=DType.Bool))
    np.testing.assert_array_equal(out, [0, 1, 0, 1])
    (out,) = R.run_oracle(*_sc(np.array([10, 20, 30], F32), [i32([3, 0, 2])], "add", [4], [0], 0, True))
    np.testing.assert_array_equal(out, [20, 0, 30, 10])
    (out,) = R.run_oracle(*_sc(np.array([[1, 2, 3], [4, 5, 6]], F32), [i32([[0], [2]]), i32([[0, 1, 1]])], "add", [3, 4], [0, 1], 0))
    np.testing.assert_array_equal(out, [[1, 5, 0, 0], [0, 0, 0, 0], [4, 11, 0, 0]])


def _sc(updates, indices, op, shape, axis, out_dim, unique=False, dtype=None):
    return R.scatter(updates, indices, op, shape, axis, out_dim, unique, dtype), [updates] + list(indices)


def scatter_brute(updates, indices, op, shape, axis, out_dim, unique):
    """The reference's loop (src/routine.ts:226-296), one update element at a time."""
    out = np.zeros(shape, updates.dtype)
    index_rank = max(i.ndim for i in indices)
    free_dims = [d for d in range(updates.ndim) if d < out_dim or d >= out_dim + index_rank]
    for coord in itertools.product(*[range(s) for s in updates.shape]):
        dest, free = [], iter(free_dims)
        for ax in range(len(shape)):
            if ax in axis:
                ia = indices[axis.index(ax)]
                first = out_dim + index_rank - ia.ndim
                dest.append(int(ia[tuple(coord[first + j] if ia.shape[j] != 1 else 0 for j in range(ia.ndim))]))
            else:
                dest.append(coord[next(free)])
        if any(c < 0 or c >= s for c, s in zip(dest, shape)):
            continue
        if op == "add" and not unique:
            out[tuple(dest)] += updates[coord]
        else:
            out[tuple(dest)] = updates[coord]
    return out


SCATTER_CASES = [
    # (update shape, index shapes, output shape, indexed axes, outDim)
    ((7,), [(7,)], (5,), [0], 0),
    ((6, 3), [(6,)], (4, 3), [0], 0),
    ((3, 6), [(6,)], (3, 4), [1], 1),
    ((2, 5, 3), [(5,), (5,)], (2, 4, 6, 3), [1, 2], 1),
    ((4, 3, 2), [(4, 1), (1, 3)], (5, 2, 5), [2, 0], 0),
    ((2, 2, 3, 2), [(2, 3)], (2, 6, 2), [1], 1),
]


@pytest.mark.parametrize("case", SCATTER_CASES, ids=lambda c: "x".join(map(str, c[0])))
@pytest.mark.parametrize("op", ["add", "update"])
def test_scatter_matches_brute_force(case, op):
    ushape, ishapes, oshape, axis, out_dim = case
    upd = RNG.integers(-9, 10, ushape).astype(F32)
    idx = [RNG.integers(-1, oshape[a] + 1, s).astype(np.int32) for s, a in zip(ishapes, axis)]  # some out of range
    (got,) = R.run_oracle(*_sc(upd, idx, op, list(oshape), axis, out_dim))
    np.testing.assert_array_equal(got, scatter_brute(upd, idx, op, list(oshape), axis, out_dim, False))


def spd(batch, n):
    a = RNG.standard_normal(batch + (n, n))
    return (a @ np.swapaxes(a, -1, -2) + n * np.eye(n)).astype(F32)


def test_cholesky_tables_and_library():
    for x in (np.array([[2, 1], [1, 2]], F32), np.array([[4, 2, 1], [2, 5, 3], [1, 3, 6]], F32)):
        (L,) = R.run_oracle(R.cholesky(x), [x])
        assert np.all(np.triu(L, 1) == 0)
        np.testing.assert_allclose(L @ L.T, x, rtol=1e-5, atol=1e-6)
    x = spd((3,), 40)
    (L,) = R.run_oracle(R.cholesky(x), [x])
    np.testing.assert_allclose(L, np.linalg.cholesky(x.astype(np.float64)), rtol=2e-5, atol=2e-6)
    # only the lower triangle is read
    junk = x + np.triu(RNG.standard_normal(x.shape), 1).astype(F32)
    (L2,) = R.run_oracle(R.cholesky(junk), [junk])
    assert R.bits_equal(L, L2)
    # not positive definite: NaNs from the first negative pivot on, no exception
    bad = np.array([[1, 2], [2, 1]], F32)
    (L,) = R.run_oracle(R.cholesky(bad), [bad])
    assert L[0, 0] == 1 and L[1, 0] == 2 and np.isnan(L[1, 1]) and L[0, 1] == 0


def test_triangular_solve_tables_and_library():
    a, b = np.array([[2, 1], [0, 3]], F32), np.array([[5, 3]], F32)
    (x,) = R.run_oracle(R.triangular_solve(a, b), [a, b])
    np.testing.assert_allclose(x, [[2, 1]])
    # lower-triangular L x = b of the reference's test, posed as the routine sees it after the front-end's flips:
    # reversing rows and columns of L gives an upper-triangular system in the reversed unknowns.
    L, rhs = np.array([[2, 0], [1, 3]], F32), np.array([4, 7], F32)
    (x,) = R.run_oracle(R.triangular_solve(L[::-1, ::-1].copy(), rhs[::-1].copy()[None]), [L[::-1, ::-1].copy(), rhs[::-1].copy()[None]])
    np.testing.assert_allclose(x[0, ::-1], [2, 5 / 3], rtol=1e-6)
    a = (np.triu(RNG.standard_normal((3, 30, 30))) + 6 * np.eye(30)).astype(F32)
    b = RNG.standard_normal((3, 7, 30)).astype(F32)
    (x,) = R.run_oracle(R.triangular_solve(a, b), [a, b])
    for k in range(3):
        want = scipy.linalg.solve_triangular(a[k].astype(np.float64), b[k].astype(np.float64).T, lower=False).T
        np.testing.assert_allclose(x[k], want, rtol=2e-5, atol=2e-6)
    (xu,) = R.run_oracle(R.triangular_solve(a, b, True), [a, b])
    for k in range(3):
        want = scipy.linalg.solve_triangular(a[k].astype(np.float64), b[k].astype(np.float64).T, lower=False, unit_diagonal=True).T
        np.testing.assert_allclose(xu[k], want, rtol=1e-3, atol=1e-3 * np.abs(want).max())
    # the strictly lower part of `a` is never read
    (x2,) = R.run_oracle(R.triangular_solve(a + np.tril(np.ones_like(a), -1), b), [a + np.tril(np.ones_like(a), -1), b])
    assert R.bits_equal(x, x2)


def test_lu_table_identity_and_library():
    a = np.array([[4, 3], [6, 3]], F32)
    lu, piv, perm = R.run_oracle(R.lu(a), [a])
    np.testing.assert_allclose(lu, [[6, 3], [0.6666667, 1.0]], rtol=1e-6)
    assert piv.tolist() == [1, 1] and perm.tolist() == [1, 0]
    for m, n in ((30, 30), (12, 20), (20, 12), (1, 5), (5, 1)):
        a = RNG.uniform(0, 1, (2, m, n)).astype(F32)
        lu, piv, perm = R.run_oracle(R.lu(a), [a])
        r = min(m, n)
        for k in range(2):
            Lm = np.tril(lu[k], -1)[:, :r] + np.eye(m, r)
            U = np.triu(lu[k])[:r, :]
            np.testing.assert_allclose(Lm @ U, a[k][perm[k]], rtol=1e-5, atol=1e-5)
            assert sorted(perm[k].tolist()) == list(range(m))
            if m == n:
                ref_lu, ref_piv = scipy.linalg.lu_factor(a[k].astype(np.float64))
                assert piv[k].tolist() == ref_piv.tolist()
                np.testing.assert_allclose(lu[k], ref_lu, rtol=1e-3, atol=1e-4)
    # a zero pivot column leaves the rows below untouched (src/routine.ts:406-416)
    z = np.array([[0, 1], [0, 2]], F32)
    lu, piv, perm = R.run_oracle(R.lu(z), [z])
    assert lu.tolist() == [[0, 1], [0, 2]] and piv.tolist() == [0, 1] and perm.tolist() == [0, 1]


def test_jacobi_eigh_tables_and_identities():
    x = np.diag(np.array([3, 1, 2], F32))
    d, v = R.run_oracle(R.jacobi_eigh(x), [x])
    assert np.diagonal(d).tolist() == [3, 1, 2] and R.bits_equal(v, np.eye(3, dtype=F32))
    a = RNG.standard_normal((3, 20, 20))
    sym = (a + np.swapaxes(a, -1, -2)).astype(F32)
    d, v = R.run_oracle(R.jacobi_eigh(sym), [sym])
    for k in range(3):
        w = np.diagonal(d[k]).astype(np.float64)
        np.testing.assert_allclose(np.sort(w), np.linalg.eigvalsh(sym[k].astype(np.float64)), rtol=1e-5, atol=2e-5)
        np.testing.assert_allclose(v[k].T @ v[k], np.eye(20), atol=1e-5)
        np.testing.assert_allclose((v[k] * w) @ v[k].T, sym[k], atol=5e-5)
        assert np.abs(np.tril(d[k], -1)).max() <= 1e-7 * max(1, np.abs(sym[k]).max()) * 1.0001 and np.all(np.triu(d[k], 1) == 0)
    # only the lower triangle is read; zero sweeps return the lower triangle and the identity
    junk = sym + np.triu(RNG.standard_normal(sym.shape), 1).astype(F32)
    d2, v2 = R.run_oracle(R.jacobi_eigh(junk), [junk])
    assert R.bits_equal(d, d2) and R.bits_equal(v, v2)
    d0, v0 = R.run_oracle(R.jacobi_eigh(sym, max_sweeps=0), [sym])
    assert R.bits_equal(d0, np.tril(sym)) and R.bits_equal(v0, np.broadcast_to(np.eye(20, dtype=F32), sym.shape))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 8, 12, 30, 49, 64, 11, 13, 97, 210, 1024])
def test_fft_against_numpy(n):
    assert int(np.prod(R.factor_fft_size(n))) == n
    re, im = RNG.standard_normal((3, n)).astype(F32), RNG.standard_normal((3, n)).astype(F32)
    z = re.astype(np.float64) + 1j * im
    o_re, o_im = R.run_oracle(R.fft(re, im), [re, im])
    want = np.fft.fft(z)
    tol = 2e-6 * np.abs(want).max() * max(1, len(R.factor_fft_size(n)))
    np.testing.assert_allclose(o_re, want.real, atol=tol)
    np.testing.assert_allclose(o_im, want.imag, atol=tol)
    i_re, i_im = R.run_oracle(R.fft(re, im, True), [re, im])
    want = np.fft.ifft(z)
    np.testing.assert_allclose(i_re, want.real, atol=tol / n + 1e-7)
    np.testing.assert_allclose(i_im, want.imag, atol=tol / n + 1e-7)


def test_fft_reference_tables_and_any_factor_order():
    z = lambda *s: np.zeros(s, F32)  # noqa: E731
    re, im = R.run_oracle(R.fft(np.array([0, 1, 2, 3], F32), z(4)), [np.array([0, 1, 2, 3], F32), z(4)])
    np.testing.assert_allclose(re, [6, -2, -2, -2], atol=1e-5)
    np.testing.assert_allclose(im, [0, 2, 0, -2], atol=1e-5)
    a, b = np.array([6, -2, -2, -2], F32), np.array([0, 2, 0, -2], F32)
    re, im = R.run_oracle(R.fft(a, b, True), [a, b])
    np.testing.assert_allclose(re, [0, 1, 2, 3], atol=1e-6)
    np.testing.assert_allclose(im, 0, atol=1e-6)
    x = np.array([[1, 5], [2, 6], [3, 7], [4, 8]], F32)  # the axis-0 example, moved to the last axis by the front-end
    re, im = R.run_oracle(R.fft(x, z(4, 2)), [x, z(4, 2)])
    np.testing.assert_allclose(re, [[6, -4], [8, -4], [10, -4], [12, -4]], atol=1e-5)
    xr, xi = RNG.standard_normal((2, 60)).astype(F32), RNG.standard_normal((2, 60)).astype(F32)
    want = np.fft.fft(xr + 1j * xi)
    for factors in ([4, 3, 5], [5, 3, 4], [2, 2, 15], [60]):
        re, im = R.run_oracle(R.fft(xr, xi, False, factors), [xr, xi])
        np.testing.assert_allclose(re + 1j * im, want, atol=2e-5)


# ---- float64 and float16 elements (the reference's typed arrays: a Float64Array keeps every double, a Float16Array rounds it once)

def test_dense_routines_in_float64_against_the_identities_and_libraries_at_double_precision():
    x = spd((2,), 40).astype(np.float64)
    (L,) = R.run_oracle(R.cholesky(x), [x])
    assert L.dtype == np.float64 and np.all(np.triu(L, 1) == 0)
    np.testing.assert_allclose(L, np.linalg.cholesky(x), rtol=1e-13, atol=1e-14)
    a = np.triu(RNG.standard_normal((2, 30, 30))) + 6 * np.eye(30)
    b = RNG.standard_normal((2, 7, 30))
    for unit in (False, True):
        (sol,) = R.run_oracle(R.triangular_solve(a, b, unit), [a, b])
        for k in range(2):
            want = scipy.linalg.solve_triangular(a[k], b[k].T, lower=False, unit_diagonal=unit).T
            np.testing.assert_allclose(sol[k], want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    m = RNG.uniform(0, 1, (2, 25, 25))
    lu, piv, perm = R.run_oracle(R.lu(m), [m])
    for k in range(2):
        ref_lu, ref_piv = scipy.linalg.lu_factor(m[k])
        assert piv[k].tolist() == ref_piv.tolist()
        np.testing.assert_allclose(lu[k], ref_lu, rtol=1e-10, atol=1e-12)
        np.testing.assert_allclose((np.tril(lu[k], -1) + np.eye(25)) @ np.triu(lu[k]), m[k][perm[k]], rtol=1e-13, atol=1e-14)
    g = RNG.standard_normal((2, 20, 20))
    sym = g + np.swapaxes(g, -1, -2)
    d, v = R.run_oracle(R.jacobi_eigh(sym, 30, 1e-14), [sym])
    for k in range(2):
        w = np.diagonal(d[k])
        np.testing.assert_allclose(np.sort(w), np.linalg.eigvalsh(sym[k]), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(v[k].T @ v[k], np.eye(20), atol=1e-13)
        np.testing.assert_allclose((v[k] * w) @ v[k].T, sym[k], atol=1e-12)
    for n in (12, 49, 64, 97):
        re, im = RNG.standard_normal((2, n)), RNG.standard_normal((2, n))
        o_re, o_im = R.run_oracle(R.fft(re, im), [re, im])
        np.testing.assert_allclose(o_re + 1j * o_im, np.fft.fft(re + 1j * im), atol=1e-12 * n)
        i_re, i_im = R.run_oracle(R.fft(re, im, True), [re, im])
        np.testing.assert_allclose(i_re + 1j * i_im, np.fft.ifft(re + 1j * im), atol=1e-13)


def _once(x):
    """A float64 array rounded once to float16 (numpy's conversion from double is a single rounding)."""
    return np.asarray(x, np.float64).astype(np.float16)


def test_dense_routines_in_float16_round_each_store_once_from_the_double():
    """Small cases worked by hand in Python floats (= the reference's JavaScript numbers) with every store rounded to
    float16: a wrong rounding point (through float32, or keeping a double between stores) changes these bits."""
    H = np.float16
    x = np.array([[4, 2, 1], [2, 5, 3], [1, 3, 6]], H)
    (L,) = R.run_oracle(R.cholesky(x), [x])
    want = np.zeros((3, 3), H)
    for i in range(3):
        for j in range(i + 1):
            s = float(x[i, j])
            for k in range(j):
                s -= float(want[i, k]) * float(want[j, k])
            want[i, j] = _once(np.sqrt(s)) if i == j else _once(s / float(want[j, j]))
    assert L.dtype == H and R.bits_equal(L, want)
    a, b = np.array([[2, 1, 0.3], [0, 3, 0.7], [0, 0, 1.1]], H), np.array([[5, 3, 0.1], [1, 2, 3]], H)
    (sol,) = R.run_oracle(R.triangular_solve(a, b), [a, b])
    want = np.zeros((2, 3), H)
    for t in range(2):
        for i in (2, 1, 0):
            s = float(b[t, i])
            for j in range(i + 1, 3):
                s -= float(a[i, j]) * float(want[t, j])
            want[t, i] = _once(s / float(a[i, i]))
    assert R.bits_equal(sol, want)
    m = np.array([[0.3, 3, 1.7], [6, 3, 0.9], [1.1, -2, 5]], H)
    lu, piv, perm = R.run_oracle(R.lu(m), [m])
    w, pr, pv = m.copy(), [0, 1, 2], []
    for j in range(3):
        r = j + int(np.argmax(np.abs(w[j:, j].astype(np.float64))))
        pv.append(r)
        if r != j:
            w[[j, r]] = w[[r, j]]
            pr[j], pr[r] = pr[r], pr[j]
        for i in range(j + 1, 3):
            f = float(w[i, j]) / float(w[j, j])
            w[i, j] = _once(f)
            for c in range(j + 1, 3):
                w[i, c] = _once(float(w[i, c]) - f * float(w[j, c]))  # the unrounded factor, as the reference keeps it
    assert R.bits_equal(lu, w) and piv.tolist() == pv and perm.tolist() == pr
    # One Jacobi sweep limit and the DFT of four points: identities within float16 resolution.
    g = RNG.standard_normal((8, 8))
    sym = (g + g.T).astype(H)
    d, v = R.run_oracle(R.jacobi_eigh(sym, 30, 1e-3), [sym])
    wv = np.diagonal(d).astype(np.float64)
    np.testing.assert_allclose(np.sort(wv), np.linalg.eigvalsh(np.tril(sym.astype(np.float64)) + np.tril(sym.astype(np.float64), -1).T), atol=3e-2)
    np.testing.assert_allclose(v.astype(np.float64).T @ v.astype(np.float64), np.eye(8), atol=2e-2)
    re, im = np.array([0, 1, 2, 3], H), np.zeros(4, H)
    o_re, o_im = R.run_oracle(R.fft(re, im), [re, im])
    assert o_re.dtype == H and o_re.tolist() == [6, -2, -2, -2]
    np.testing.assert_allclose(o_im.astype(np.float64), [0, 2, 0, -2], atol=1e-3)
    # the float16 store itself: halfway cases straight from the double (1 + 2^-11 + 2^-30 rounds up; through float32 it would tie to even)
    tie = np.array([[1.0 + 2.0 ** -11 + 2.0 ** -30]])
    assert _once(tie)[0, 0] == np.float16(1.0 + 2.0 ** -10)
    x = np.array([[4.0]], H)
    bvec = np.array([[4.0 * (1.0 + 2.0 ** -11) + 2.0 ** -20]], np.float64)
    (sol,) = R.run_oracle(R.triangular_solve(x, bvec.astype(H)), [x, bvec.astype(H)])
    assert sol[0, 0] == _once(float(bvec.astype(H)[0, 0]) / 4.0)[()]


def test_attention_checker_against_reference_tables_and_composition():
    """The fused-attention checker (not a reference routine): the reference's dotProductAttention tables
    (test/nn.test.ts:274-390) and, on random float16 operands, the unfused composition replayed kernel by kernel."""
    import math
    from oracle.routines import attention
    q = np.array([[[[1, 0, 0, 0]], [[0, 1, 0, 0]]]], F32)
    v = np.array([[[[1, 2, 3, 4]], [[5, 6, 7, 8]]]], F32)
    a, b = 0.62245935, 0.37754068
    np.testing.assert_allclose(attention(q, q, v, 0.5, False)[0, 0, 0], [a * 1 + b * 5, a * 2 + b * 6, a * 3 + b * 7, a * 4 + b * 8], atol=1e-6)
    e = np.array([[[[1, 0]], [[0, 1]]]], F32)
    np.testing.assert_allclose(attention(e, e, e, 1.0, False)[0, 0, 0], [0.7310586, 0.26894143], atol=1e-6)
    qc = np.array([[[[1, 0]], [[0.2, 0.2]], [[1, 1]]]], F32)
    kc = np.array([[[[1, 0]], [[0, 1]], [[1, 1]]]], F32)
    vc = np.array([[[[1, 0]], [[0, 1]], [[0, 0]]]], F32)
    y = attention(qc, kc, vc, 1 / math.sqrt(2), True)
    c = 1 / (2 + math.exp(math.sqrt(0.5)))
    np.testing.assert_allclose(y[0, :, 0], [[1, 0], [0.5, 0.5], [c, c]], atol=1e-7)
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    from jaxjs_hip.jit import ShapedArray
    from jit_util import run_program
    from oracle.backend import OracleBackend
    ops = [RNG.standard_normal((2, 128, 2, 64)).astype(np.float16) for _ in range(3)]
    for causal in (False, True):
        outs = []
        for fused in (False, True):
            prog = J.jit(lambda x, y_, z: L.dotProductAttention(x, y_, z, isCausal=causal, fused=fused), [ShapedArray((2, 128, 2, 64), DType.Float16)] * 3)
            assert len(prog.routines) == (1 if fused else 0)
            (o,) = run_program(OracleBackend(), prog, ops)
            outs.append(o.astype(np.float64))
        np.testing.assert_allclose(outs[1], outs[0], rtol=1e-2, atol=4e-3)  # the unfused chain rounds to f16 seven times
