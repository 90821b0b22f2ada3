"""Long-tail cases of the kernel path on the GPU: f64, uint32, data-dependent (gather-style) indexing with
out-of-range indices, empty kernels and empty reductions, masked views under a reduction, multi-view trackers,
many-argument kernels, f16 elementwise, and the device-libm numerics mode.  The checker is the CPU oracle."""
import numpy as np
import pytest

from gpu_util import WARM_ONLY, assert_parity, backend, device_run
from jaxjs_hip import AluExp, AluOp, AluVar, DType, Kernel, Reduction, ShapeTracker
from jaxjs_hip.lowering import mapKernel, reduceKernel
from oracle import oracle

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(77)
F32, F64, I32, U32, F16 = DType.Float32, DType.Float64, DType.Int32, DType.Uint32, DType.Float16


def flat(n):
    return ShapeTracker.fromShape([n])


# ---- f64 ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name,fn", [
    ("add_mul", lambda a, b: AluExp.add(AluExp.mul(a, b), a)),
    ("div_sqrt", lambda a, b: AluExp.mul(AluExp.sqrt(AluExp.mul(a, a)), AluExp.reciprocal(AluExp.add(AluExp.mul(b, b), AluExp.const(DType.Float64, 1.0))))),
    ("idiv_mod", lambda a, b: AluExp.add(AluExp.idiv(a, AluExp.const(DType.Float64, 0.37)), AluExp.mod(b, AluExp.const(DType.Float64, 0.21)))),
    ("minmax", lambda a, b: AluExp.sub(AluExp.max(a, b), AluExp.min(a, b))),
])
def test_f64_maps_are_exact_doubles(name, fn):
    """Native doubles on the device: +,-,*,/,sqrt are correctly rounded on both sides, so bit-exact."""
    n = 1001
    a, b = RNG.normal(0, 3, n), RNG.normal(0, 3, n)
    k = mapKernel([n], [(F64, flat(n)), (F64, flat(n))], fn)
    assert_parity(k, [a, b], exact=True)


def test_f64_transcendentals_are_demoted_like_wasm():
    """src/backend/wasm/translation.ts:113-122: f64 exp/log/sin run the f32 polynomials."""
    n = 257
    x = RNG.uniform(0.1, 5, n)
    for op in (AluExp.exp, AluExp.log, AluExp.sin):
        k = mapKernel([n], [(F64, flat(n))], op)
        got, want, _ = assert_parity(k, [x], rtol=1e-6, atol=1e-7)
        assert got.dtype == np.float64


def test_f64_sum_within_k_scaled_bound():
    rows, L = 37, 5000
    x = RNG.normal(0, 1, (rows, L))
    k = reduceKernel([rows, L], [(F64, ShapeTracker.fromShape([rows, L]))], lambda v: v, AluOp.Add)
    got, _ = device_run(k, [x])
    ref = np.array([float(np.sum(r.astype(np.longdouble))) for r in x])
    assert np.all(np.abs(got - ref) <= 2 * L * np.finfo(np.float64).eps * np.abs(x).sum(-1))


# ---- uint32 ----------------------------------------------------------------------------------------------

U32_OPS = {
    "add_wrap": AluExp.add, "mul_wrap": AluExp.mul, "idiv": AluExp.idiv, "mod": AluExp.mod,
    "min": lambda a, b: AluExp.min(a, b), "max": lambda a, b: AluExp.max(a, b), "cmplt": AluExp.cmplt,
    "shr_logical": lambda a, b: AluExp.bitShift(a, AluExp.mod(b, AluExp.u32(32)), "shr"),
    "shl": lambda a, b: AluExp.bitShift(a, AluExp.mod(b, AluExp.u32(32)), "shl"),
    "xor": lambda a, b: AluExp.bitCombine(a, b, "xor"),
}


@pytest.mark.parametrize("name", sorted(U32_OPS))
def test_uint32_ops_bit_exact(name):
    n = 4099
    a = RNG.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    b = RNG.integers(1, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    a[:4] = [0, 0xffffffff, 0x80000000, 0x7fffffff]
    b[:4] = [0xffffffff, 1, 0x80000001, 0x80000000]
    k = mapKernel([n], [(U32, flat(n)), (U32, flat(n))], U32_OPS[name])
    assert_parity(k, [a, b], exact=True)


@pytest.mark.parametrize("op", [AluOp.Add, AluOp.Min, AluOp.Max])
@pytest.mark.parametrize("shape", [(33, 1000), (1000, 33), (3, 70001)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_uint32_reductions_bit_exact(op, shape):
    rows, L = shape
    x = RNG.integers(0, 1 << 32, (rows, L), dtype=np.uint64).astype(np.uint32)
    k = reduceKernel([rows, L], [(U32, ShapeTracker.fromShape([rows, L]))], lambda v: v, op)
    assert_parity(k, [x], exact=True)
    st = ShapeTracker.fromShape([L, rows]).permute([1, 0])  # same reduce, column orientation in memory
    k = reduceKernel([rows, L], [(U32, st)], lambda v: v, op)
    assert_parity(k, [np.ascontiguousarray(x.T)], exact=True)


# ---- gather-style indexing ---------------------------------------------------------------------------------

def test_gather_with_out_of_range_indices_reads_element_zero():
    """`x[idx]` as the jit's Gather rule builds it (src/frontend/jit.ts:698-752): the index is data.  The Wasm
    backend clamps an out-of-range *index* to 0 (translation.ts:221-228); the device must do the same and must not
    read outside the allocation."""
    n, m = 1000, 5000
    x = RNG.normal(0, 1, n).astype(np.float32)
    idx = RNG.integers(-50, n + 50, m).astype(np.int32)
    idx[:3] = [0, n - 1, n]
    load_idx = AluExp.globalIndex(I32, 1, m, AluVar.gidx)
    k = Kernel(2, m, AluExp.globalIndex(F32, 0, n, load_idx))
    got, want, _ = assert_parity(k, [x, idx], exact=True)
    ok = (idx >= 0) & (idx < n)
    np.testing.assert_array_equal(got[ok], x[idx[ok]])
    np.testing.assert_array_equal(got[~ok], np.full((~ok).sum(), x[0], np.float32))


def test_gather_rows_2d():
    rows, cols, picks = 300, 64, 777
    table = RNG.normal(0, 1, (rows, cols)).astype(np.float32)
    idx = RNG.integers(0, rows, picks).astype(np.int32)
    r, c = AluExp.idiv(AluVar.gidx, AluExp.i32(cols)), AluExp.mod(AluVar.gidx, AluExp.i32(cols))
    row = AluExp.globalIndex(I32, 1, picks, r)
    k = Kernel(2, picks * cols, AluExp.globalIndex(F32, 0, rows * cols, AluExp.add(AluExp.mul(row, AluExp.i32(cols)), c)))
    got, _, _ = assert_parity(k, [table, idx], exact=True)
    np.testing.assert_array_equal(got.reshape(picks, cols), table[idx])


# ---- empty and degenerate shapes ----------------------------------------------------------------------------

def test_empty_kernel_and_empty_reduction():
    if WARM_ONLY:
        pytest.skip("nothing to compile")
    be = backend()
    k0 = mapKernel([0], [(F32, flat(0))], lambda v: v)
    src, dst = be.malloc(0), be.malloc(0)
    be.dispatch(be.prepareKernelSync(k0), [src], [dst])  # no launch, no error
    assert be.readSync(dst) == b""
    be.decRef(src)
    be.decRef(dst)
    # A reduction over an empty axis yields the identity (src/alu.ts:1584-1604) through the epilogue.
    for op, ident in ((AluOp.Add, 0.0), (AluOp.Max, -np.inf), (AluOp.Min, np.inf), (AluOp.Mul, 1.0)):
        k = reduceKernel([5, 0], [(F32, ShapeTracker.fromShape([5, 0]))], lambda v: v, op,
                         epilogue=lambda acc: AluExp.add(acc, AluExp.f32(1)))
        got, _ = device_run(k, [np.zeros(0, np.float32)])
        np.testing.assert_array_equal(got, np.full(5, ident + 1, np.float32))


def test_single_element_and_scalar_reduce():
    k = reduceKernel([1, 1], [(I32, ShapeTracker.fromShape([1, 1]))], lambda v: v, AluOp.Add)
    assert_parity(k, [np.array([41], np.int32)], exact=True)
    n = 100003  # prime: no vector width divides it
    x = RNG.integers(-1000, 1000, n).astype(np.int32)
    k = reduceKernel([1, n], [(I32, ShapeTracker.fromShape([1, n]))], lambda v: v, AluOp.Add)
    got, _, _ = assert_parity(k, [x], exact=True)
    assert got[0] == x.sum()


# ---- views under a reduction ---------------------------------------------------------------------------------

def test_padded_window_sum_like_a_convolution():
    """Sum over a sliding, zero-padded window expressed purely with views (pad -> shrink per tap stacked on a
    new axis is what pooling lowers to); checks masked loads inside a reduce in both orientations."""
    H, Wd = 37, 53
    x = RNG.integers(-9, 10, (H, Wd)).astype(np.float32)
    base = ShapeTracker.fromShape([H, Wd]).pad([(1, 1), (1, 1)])
    taps = [(dy, dx) for dy in range(3) for dx in range(3)]
    exps = []
    idx = None
    shape = [H, Wd]
    from jaxjs_hip.shape import unravelAlu
    idx = unravelAlu(shape, AluVar.gidx)
    total = None
    for dy, dx in taps:
        st = base.shrink([(dy, dy + H), (dx, dx + Wd)])
        term = AluExp.globalView(F32, 0, st, idx)
        total = term if total is None else AluExp.add(total, term)
    k = Kernel(1, H * Wd, total)
    got, _, _ = assert_parity(k, [x], exact=True)
    ref = np.zeros((H, Wd), np.float32)
    xp = np.pad(x, 1)
    for dy, dx in taps:
        ref += xp[dy:dy + H, dx:dx + Wd]
    np.testing.assert_array_equal(got.reshape(H, Wd), ref)
    # the same padded operand under a row reduction
    st = ShapeTracker.fromShape([H, Wd]).pad([(2, 0), (0, 3)])
    k = reduceKernel([H + 2, Wd + 3], [(F32, st)], lambda v: v, AluOp.Add)
    got, _, _ = assert_parity(k, [x], exact=True)
    np.testing.assert_array_equal(got, np.pad(x, [(2, 0), (0, 3)]).sum(-1))


def test_multi_view_tracker_in_map_and_reduce():
    """permute followed by a reshape that cannot merge leaves two views; indices chain through unravel."""
    a, b, c = 6, 10, 14
    x = RNG.integers(-99, 100, (a, b, c)).astype(np.int32)
    st = ShapeTracker.fromShape([a, b, c]).permute([2, 0, 1]).reshape([c * a, b])
    assert len(st.views) == 2
    k = mapKernel([c * a, b], [(I32, st)], lambda v: AluExp.mul(v, AluExp.i32(3)))
    got, _, _ = assert_parity(k, [x], exact=True)
    np.testing.assert_array_equal(got.reshape(c * a, b), x.transpose(2, 0, 1).reshape(c * a, b) * 3)
    k = reduceKernel([c * a, b], [(I32, st)], lambda v: v, AluOp.Max)
    got, _, _ = assert_parity(k, [x], exact=True)
    np.testing.assert_array_equal(got, x.transpose(2, 0, 1).reshape(c * a, b).max(-1))


# ---- many arguments, f16, native numerics ----------------------------------------------------------------------

def test_sixty_four_inputs():
    n, nargs = 1000, 64
    arrays = [RNG.integers(-5, 6, n).astype(np.int32) for _ in range(nargs)]

    def f(*xs):
        acc = xs[0]
        for x in xs[1:]:
            acc = AluExp.add(acc, x)
        return acc
    k = mapKernel([n], [(I32, flat(n))] * nargs, f)
    got, _, _ = assert_parity(k, arrays, exact=True)
    np.testing.assert_array_equal(got, np.sum(arrays, axis=0))


def test_f16_elementwise():
    n = 8 * 1000 + 5
    a = RNG.normal(0, 1, n).astype(np.float16)
    b = RNG.normal(0, 1, n).astype(np.float16)
    k = mapKernel([n], [(F16, flat(n)), (F16, flat(n))], lambda x, y: AluExp.add(AluExp.mul(x, y), x))
    assert_parity(k, [a, b], exact=True)  # each f16 operation rounds once on both sides
    k = mapKernel([n], [(F16, flat(n))], lambda x: AluExp.exp(x))
    assert_parity(k, [a], rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("op", [AluOp.Max, AluOp.Min])
def test_f16_min_max_propagate_nan_and_order_signed_zeros(op):
    """float16 min / max run on v_min_f16 / v_max_f16 with an unordered select: a NaN on either side gives NaN, -0 sorts
    below +0, infinities behave -- elementwise, and as a row reduction whose rows hold those values at every lane and
    batch position (bit patterns compared, so the sign of a zero counts)."""
    special = np.array([np.nan, 0.0, -0.0, np.inf, -np.inf, 1.5, -1.5, 65504.0, 6e-8], np.float16)
    a, b = [x.ravel() for x in np.meshgrid(special, special)]
    pad = 8 * 13 - len(a) % 8
    a, b = np.concatenate([a, special[:pad]]), np.concatenate([b, special[pad - 1::-1][:pad]])
    n = len(a)
    fn = AluExp.max if op == AluOp.Max else AluExp.min
    got, want, _ = assert_parity(mapKernel([n], [(F16, flat(n)), (F16, flat(n))], lambda x, y: fn(x, y)), [a, b], rtol=0, atol=0)
    np.testing.assert_array_equal(got.view(np.uint16)[~np.isnan(want)], want.view(np.uint16)[~np.isnan(want)])
    rows, L = 64, 2048
    x = RNG.normal(0, 1, (rows, L)).astype(np.float16)
    x[::2] = np.abs(x[::2]) * (1 if op == AluOp.Min else -1)      # every other row has one sign only ...
    for r in range(0, rows, 2):
        x[r, (r * 37) % L] = 0.0 if op == AluOp.Min else -0.0      # ... and one zero of the sign that loses ...
        x[r, (r * 91 + 5) % L] = -0.0 if op == AluOp.Min else 0.0  # ... and one of the sign that wins
    x[7, 1000] = np.nan
    x[9, 3] = np.inf if op == AluOp.Max else -np.inf
    got, want, _ = assert_parity(reduceKernel([rows, L], [(F16, ShapeTracker.fromShape([rows, L]))], lambda v: v, op), [x], rtol=0, atol=0)
    assert np.isnan(got[7]) and np.isnan(want[7])
    np.testing.assert_array_equal(np.delete(got, 7).view(np.uint16), np.delete(want, 7).view(np.uint16))
    assert got[0].view(np.uint16) == (0x8000 if op == AluOp.Min else 0x0000)


@pytest.mark.parametrize("name,fn,ref", [("exp", AluExp.exp, np.exp), ("log", AluExp.log, np.log), ("sin", AluExp.sin, np.sin),
                                         ("cos", AluExp.cos, np.cos), ("atan", AluExp.atan, np.arctan)])
def test_native_numerics_track_libm(name, fn, ref):
    """numerics="native" swaps the Wasm polynomials for the device math library: results follow libm to a few ulp
    (and so differ from the Wasm backend by its polynomial error)."""
    from jaxjs_hip.backend import HipBackend
    n = 4096
    x = RNG.uniform(0.05, 6, n).astype(np.float32)
    k = mapKernel([n], [(F32, flat(n))], fn)
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(k, "native").sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    nb = HipBackend.__new__(HipBackend)
    nb.__dict__.update(be.__dict__)
    nb.numerics = "native"
    nb._exes = {}
    exe = nb.prepareKernelSync(k)
    s, o = nb.malloc(x.nbytes, x.tobytes()), nb.malloc(k.bytes)
    nb.dispatch(exe, [s], [o])
    got = np.frombuffer(nb.readSync(o), dtype=np.float32)
    nb.decRef(s)
    nb.decRef(o)
    np.testing.assert_allclose(got, ref(x.astype(np.float64)), rtol=3e-7, atol=1e-7)


# ---- index arithmetic at the top of the int32 range ---------------------------------------------------------

def test_two_billion_elements_through_map_row_and_column_reductions():
    """The IR's indices are int32, so a buffer holds fewer than 2^31 elements; just under that -- float16
    [32768, 65534], 4.3 GB -- a nullary fill, a map and both reduction orientations must still address every element.
    Everything stays on the device; the small integer pattern ((flat index mod 251) - 125, then + 1) makes every
    float32 partial sum an exact integer, so the results are compared with closed forms bit for bit."""
    rows, L = 32768, 65534
    n = rows * L
    assert 2 ** 31 - 2 ** 17 < n < 2 ** 31
    st = ShapeTracker.fromShape([rows, L])
    fill = Kernel(0, n, AluExp.cast(F16, AluExp.sub(AluExp.mod(AluVar.gidx, AluExp.i32(251)), AluExp.i32(125))))
    plus1 = mapKernel([n], [(F16, flat(n))], lambda v: AluExp.add(v, AluExp.const(F16, 1.0)))
    row_sum = reduceKernel([rows, L], [(F16, st)], lambda v: AluExp.cast(F32, v), AluOp.Add)
    col_sum = reduceKernel([L, rows], [(F16, st.permute([1, 0]))], lambda v: AluExp.cast(F32, v), AluOp.Add)
    tail = Kernel(1, 64, AluExp.globalView(F16, 0, flat(n), [AluExp.add(AluVar.gidx, AluExp.i32(n - 64))]))
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for k in (fill, plus1, row_sum, col_sum, tail):
            for src in generate(k, "wasm").sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    a, b = be.malloc(n * 2), be.malloc(n * 2)
    r, c, t = be.malloc(rows * 4), be.malloc(L * 4), be.malloc(64 * 2)
    try:
        be.dispatch(be.prepareKernelSync(fill), [], [a])
        be.dispatch(be.prepareKernelSync(plus1), [a], [b])
        be.dispatch(be.prepareKernelSync(row_sum), [b], [r])
        be.dispatch(be.prepareKernelSync(col_sum), [b], [c])
        be.dispatch(be.prepareKernelSync(tail), [b], [t])
        got_r = np.frombuffer(be.readSync(r), np.float32)
        got_c = np.frombuffer(be.readSync(c), np.float32)
        got_t = np.frombuffer(be.readSync(t), np.float16)
    finally:
        for s_ in (a, b, r, c, t):
            be.decRef(s_)
    # closed forms: value(i) = i % 251 - 124
    period = np.arange(251, dtype=np.int64) - 124
    pre = np.concatenate([[0], np.cumsum(period)])  # pre[m] = sum of the first m values of a period

    def span(lo, count):  # sum of value(i) for i in [lo, lo + count), vectorised over lo
        lo = np.asarray(lo, dtype=np.int64)
        first = lo % 251
        whole, rest = np.divmod(first + count, 251)
        return whole * pre[251] + pre[rest] - pre[first]

    want_r = span(np.arange(rows, dtype=np.int64) * L, L)
    np.testing.assert_array_equal(got_r.astype(np.int64), want_r)
    # column j: rows r contribute value(r * L + j); L % 251 = 23, so the residues walk with step 23: count them
    j = np.arange(L, dtype=np.int64)
    counts = np.bincount((np.arange(rows, dtype=np.int64) * L) % 251, minlength=251)  # residue of r * L
    table = np.array([sum(int(counts[q]) * int(period[(q + s) % 251]) for q in range(251)) for s in range(251)], dtype=np.int64)
    np.testing.assert_array_equal(got_c.astype(np.int64), table[j % 251])
    np.testing.assert_array_equal(got_t.astype(np.int64), (np.arange(n - 64, n, dtype=np.int64) % 251) - 124)
