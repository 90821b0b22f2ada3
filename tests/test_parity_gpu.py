"""HIP path vs the CPU checker on identical seeded inputs, through the C-ABI library.

Bars (stated per test): integer, bool, index and argmax results bit-exact; f32 maps within
rtol 1e-5 / atol 1e-7 of the Wasm-mode checker (in practice a few ulp, asserted where it holds by
construction); f32 reductions within the K-scaled bound |d| <= 2*K*eps*sum|x_i|; f16 within rtol 1e-2.
"""
import math

import numpy as np
import pytest

from jaxjs_hip import AluExp, AluOp, AluVar, DType, Kernel, Reduction, ShapeTracker, unravelAlu
from jaxjs_hip.lowering import mapKernel, matvecKernel, reduceKernel
from gpu_util import assert_parity, device_run
from oracle import oracle

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(20240607)
SPECIAL_F32 = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, 3.5, -3.5, 1e-3, -1e-3, 10.0, -10.0, 88.0, -88.0, 100.0,
                        -100.0, 1e6, -1e6, 1e20, -1e20, 3.4e38, -3.4e38, 1e-38, 1e-45, np.inf, -np.inf, np.nan,
                        0.99999994, 1.9999999, 1.5, 1.75, 6.2831855, 3.1415927, 1.5707964, 7.0, 1e4], dtype=np.float32)


def _vec(n, lo=-4.0, hi=4.0):
    return np.concatenate([SPECIAL_F32, RNG.uniform(lo, hi, n - len(SPECIAL_F32)).astype(np.float32)])


UNARY = {
    "exp": AluExp.exp, "log": AluExp.log, "sin": AluExp.sin, "cos": AluExp.cos, "atan": AluExp.atan,
    "asin": AluExp.asin, "erf": AluExp.erf, "erfc": AluExp.erfc, "sqrt": AluExp.sqrt, "floor": AluExp.floor,
    "ceil": AluExp.ceil, "reciprocal": AluExp.reciprocal,
}


@pytest.mark.parametrize("name", sorted(UNARY))
def test_unary_f32_matches_wasm_numerics(name):
    """The default numerics restate the Wasm backend's own polynomials in the same order of f32
    operations, so results agree to the last bit except where the hardware flushes a subnormal
    intermediate; the assertion is the north-star tolerance plus a 2-ulp cap on normal results."""
    n = 4099  # not a multiple of the vector width: exercises the scalar tail
    x = _vec(n)
    if name in ("sin", "cos"):
        x = np.where(np.abs(x) > 1e5, np.float32(1.0), x)  # range reduction in f32 loses everything beyond
    k = mapKernel([n], [(DType.Float32, ShapeTracker.fromShape([n]))], UNARY[name])
    got, want, _ = assert_parity(k, [x], rtol=1e-5, atol=1e-7)
    normal = np.isfinite(want) & (np.abs(want) > 1e-30)
    from gpu_util import ulp_diff_f32
    assert ulp_diff_f32(got[normal], want[normal]).max() <= 2


BINARY_F32 = {
    "add": AluExp.add, "sub": AluExp.sub, "mul": AluExp.mul, "idiv": AluExp.idiv, "mod": AluExp.mod,
    "min": lambda a, b: AluExp.min(a, b), "max": lambda a, b: AluExp.max(a, b),
    "cmplt": AluExp.cmplt, "cmpne": AluExp.cmpne,
    "div": lambda a, b: AluExp.mul(a, AluExp.reciprocal(b)),  # the front-end's a/b (src/frontend/core.ts:950-955)
}


@pytest.mark.parametrize("name", sorted(BINARY_F32))
def test_binary_f32_bit_exact(name):
    """+,-,*,/,min,max,compare are single IEEE operations: bit-exact, including NaN/-0 handling."""
    s = SPECIAL_F32
    a = np.repeat(s, len(s))
    b = np.tile(s, len(s))
    if name in ("idiv", "mod"):
        keep = np.isfinite(a) & np.isfinite(b) & (np.abs(a) < 1e7) & (np.abs(b) > 1e-3) & (np.abs(b) < 1e7)
        a, b = a[keep], b[keep]
    n = len(a)
    st = ShapeTracker.fromShape([n])
    k = mapKernel([n], [(DType.Float32, st), (DType.Float32, st)], BINARY_F32[name])
    got, want = assert_parity(k, [a, b], exact=False, rtol=0, atol=0)[:2]
    if got.dtype == np.float32:
        np.testing.assert_array_equal(got.view(np.uint32)[~np.isnan(got)], want.view(np.uint32)[~np.isnan(want)])


INT_SPECIAL = np.array([0, 1, -1, 2, -2, 3, 7, -7, 31, 32, 33, 255, 65535, 65536, 65537, 2147483647, -2147483648,
                        -2147483647, 1234567, -7654321, 46341, -46341], dtype=np.int64)


@pytest.mark.parametrize("dtype", [DType.Int32, DType.Uint32])
@pytest.mark.parametrize("name", ["add", "sub", "mul", "idiv", "mod", "min", "max", "cmplt", "cmpne", "and", "or", "xor",
                                  "shl", "shr"])
def test_binary_int_bit_exact(dtype, name):
    nd = np.int32 if dtype == DType.Int32 else np.uint32
    a = np.repeat(INT_SPECIAL, len(INT_SPECIAL)).astype(nd)
    b = np.tile(INT_SPECIAL, len(INT_SPECIAL)).astype(nd)
    fn = {"add": AluExp.add, "sub": AluExp.sub, "mul": AluExp.mul, "idiv": AluExp.idiv, "mod": AluExp.mod,
          "min": lambda x, y: AluExp.min(x, y), "max": lambda x, y: AluExp.max(x, y), "cmplt": AluExp.cmplt,
          "cmpne": AluExp.cmpne, "and": lambda x, y: AluExp.bitCombine(x, y, "and"),
          "or": lambda x, y: AluExp.bitCombine(x, y, "or"), "xor": lambda x, y: AluExp.bitCombine(x, y, "xor"),
          "shl": lambda x, y: AluExp.bitShift(x, y, "shl"), "shr": lambda x, y: AluExp.bitShift(x, y, "shr")}[name]
    n = len(a)
    st = ShapeTracker.fromShape([n])
    assert_parity(mapKernel([n], [(dtype, st), (dtype, st)], fn), [a, b], exact=True)


@pytest.mark.parametrize("dtype", [DType.Int32, DType.Uint32])
def test_constant_multiply_divide_is_folded_as_the_reference_folds_it(dtype):
    """`(x * A) / B` with B | A is rewritten to `x * (A / B)` by the reference's simplifier with no regard to wrap-around
    (src/alu.ts:795-806), and every reference backend runs that simplifier (tuneNullopt, src/tuner.ts:219-240).  So for
    operands whose product overflows, the reference's answer is the folded one, `x * (A / B)` — not `trunc(wrap(x * A) /
    B)`, which is what evaluating the unsimplified expression gives.  The backend follows the reference; the checker, which
    by design evaluates unsimplified expressions, is the one that differs here, and only here."""
    from gpu_util import device_run
    from oracle import oracle
    nd = np.int32 if dtype == DType.Int32 else np.uint32
    x = np.concatenate([INT_SPECIAL, [400000000, -400000000, 1000000007, -1999999973]]).astype(nd)
    n = len(x)
    k = mapKernel([n], [(dtype, ShapeTracker.fromShape([n]))], lambda v: AluExp.idiv(AluExp.mul(v, AluExp.const(dtype, 14)), AluExp.const(dtype, 7)))
    got, _ = device_run(k, [x])
    np.testing.assert_array_equal(got, (x.astype(np.int64) * 2).astype(nd))  # x * 2, wrapped
    unsimplified = oracle.run_kernel(k, [x], oracle.MODE_WASM)
    small = np.abs(x.astype(np.int64)) < (1 << 27)
    np.testing.assert_array_equal(got[small], unsimplified[small])  # no overflow: the two readings agree
    assert (got != unsimplified).any()                               # overflow: they do not


def test_bool_ops_bit_exact():
    a = np.array([0, 0, 1, 1] * 5, dtype=np.int32)
    b = np.array([0, 1, 0, 1] * 5, dtype=np.int32)
    st = ShapeTracker.fromShape([20])
    for fn in (AluExp.add, AluExp.mul, lambda x, y: AluExp.min(x, y), lambda x, y: AluExp.max(x, y), AluExp.cmpne,
               lambda x, y: AluExp.bitCombine(x, y, "xor"), lambda x, y: AluExp.where(x, y, y.not_())):
        assert_parity(mapKernel([20], [(DType.Bool, st), (DType.Bool, st)], fn), [a, b], exact=True)


CASTS = [(DType.Float32, DType.Int32), (DType.Float32, DType.Uint32), (DType.Float32, DType.Bool), (DType.Int32, DType.Float32),
         (DType.Uint32, DType.Float32), (DType.Int32, DType.Uint32), (DType.Uint32, DType.Int32), (DType.Bool, DType.Float32),
         (DType.Int32, DType.Bool), (DType.Float32, DType.Float16), (DType.Float16, DType.Float32), (DType.Float32, DType.Float64),
         (DType.Float64, DType.Float32), (DType.Float64, DType.Int32), (DType.Int32, DType.Float64), (DType.Float16, DType.Int32)]


@pytest.mark.parametrize("src,dst", CASTS, ids=[f"{a.value}-{b.value}" for a, b in CASTS])
def test_casts_bit_exact(src, dst):
    """Saturating float->int with NaN -> 0, int->float round-to-nearest, bool as 0/1."""
    if src in (DType.Float32, DType.Float64, DType.Float16):
        base = np.concatenate([SPECIAL_F32, RNG.uniform(-70000, 70000, 200).astype(np.float32),
                               np.array([2147483520.0, 2147483648.0, 4294967040.0, 4294967296.0, -2147483648.0, -2147483904.0],
                                        dtype=np.float32)])
        with np.errstate(over="ignore"):
            x = base.astype({DType.Float32: np.float32, DType.Float64: np.float64, DType.Float16: np.float16}[src])
    elif src == DType.Bool:
        x = np.array([0, 1, 1, 0, 1], dtype=np.int32)
    else:
        x = INT_SPECIAL.astype(np.int32 if src == DType.Int32 else np.uint32)
    n = len(x)
    k = mapKernel([n], [(src, ShapeTracker.fromShape([n]))], lambda v: AluExp.cast(dst, v))
    assert_parity(k, [x], exact=True)


def test_bitcast_threefry_uniform():
    """random.uniform's bit pipeline (src/library/random.ts:111-136) on device: threefry -> mantissa -> [0,1)."""
    n = 4096
    key = np.array([0, 51], dtype=np.uint32)
    k0 = AluExp.globalIndex(DType.Uint32, 0, 2, AluExp.i32(0))
    k1 = AluExp.globalIndex(DType.Uint32, 0, 2, AluExp.i32(1))
    c1 = AluExp.mod(AluExp.cast(DType.Uint32, AluVar.gidx), AluExp.u32(n))
    bits = AluExp.threefry2x32(k0, k1, AluExp.u32(0), c1, "xor")
    f12 = AluExp.add(AluExp.idiv(bits, AluExp.u32(1 << 9)), AluExp.u32(0x3F800000))
    u = AluExp.sub(AluExp.bitcast(DType.Float32, f12), AluExp.f32(1))
    got, want, _ = assert_parity(Kernel(1, n, u), [key], exact=True)
    assert 0 <= got.min() and got.max() < 1 and abs(got.mean() - 0.5) < 0.02
    # Known answer: uniform(key(51), [4]) (test/random.test.ts:60-71)
    got4, _ = device_run(Kernel(1, 4, u.rewrite(lambda e: AluExp.u32(4) if e is AluExp.u32(n) else None)), [key])
    np.testing.assert_allclose(got4, [0.471269, 0.12344253, 0.17550635, 0.5663593], rtol=0, atol=1e-6)


VIEW_CASES = {
    "flip": lambda st: st.flip([True, False]),
    "permute": lambda st: st.permute([1, 0]),
    "pad": lambda st: st.pad([(1, 2), (3, 0)]),
    "shrink": lambda st: st.shrink([(2, 30), (5, 61)]),
    "pad_reshape": lambda st: st.pad([(1, 1), (2, 2)]).reshape([-1]),
    "flip_reshape": lambda st: st.flip([False, True]).reshape([16, 136]),
    "broadcast": lambda st: st.reshape([34, 1, 64]).expand([34, 3, 64]),
    "shrink_permute_pad": lambda st: st.shrink([(1, 33), (0, 64)]).permute([1, 0]).pad([(0, 1), (4, 4)]),
}


@pytest.mark.parametrize("name", sorted(VIEW_CASES))
def test_views_bit_exact(name):
    """Movement ops are index arithmetic only: results must equal the checker's bit for bit."""
    base = RNG.normal(0, 1, 34 * 64).astype(np.float32)
    st0 = ShapeTracker.fromShape([34, 64])
    fn = VIEW_CASES[name]
    try:
        st = fn(st0)
    except ValueError:
        shape = list(st0.pad([(1, 1), (2, 2)]).shape)
        st = st0.pad([(1, 1), (2, 2)]).reshape([shape[0] * shape[1]])
    shape = st.shape
    k = mapKernel(shape, [(DType.Float32, st)], lambda x: AluExp.add(x, AluExp.f32(1)))
    assert_parity(k, [base], exact=True, rtol=0, atol=0)


REDUCE_SHAPES = [(1, 7), (5, 1), (3, 2), (37, 1000), (1000, 37), (8, 4096), (64, 65), (4, 100003), (1, 1 << 20), (513, 129),
                 (2048, 16), (100, 8)]


@pytest.mark.parametrize("shape", REDUCE_SHAPES, ids=[f"{a}x{b}" for a, b in REDUCE_SHAPES])
@pytest.mark.parametrize("op", [AluOp.Add, AluOp.Max, AluOp.Min, AluOp.Mul])
def test_int_reductions_bit_exact_both_orientations(shape, op):
    """Integer folds are exact modulo 2^32 in any order: row form, column form and the two-stage
    split must all reproduce the checker's sequential fold."""
    rows, cols = shape
    x = RNG.integers(-50, 50, size=rows * cols).astype(np.int32)
    if op == AluOp.Mul:
        x = RNG.choice(np.array([1, 1, 1, -1, 2, 3], dtype=np.int32), size=rows * cols)
    st = ShapeTracker.fromShape([rows, cols])
    assert_parity(reduceKernel([rows, cols], [(DType.Int32, st)], lambda v: v, op), [x], exact=True)
    stT = ShapeTracker.fromShape([cols, rows]).permute([1, 0])  # reduce over the strided axis
    assert_parity(reduceKernel([rows, cols], [(DType.Int32, stT)], lambda v: v, op), [x], exact=True)


@pytest.mark.parametrize("shape", [(37, 1000), (1000, 37), (8, 4096), (4, 100003), (1, 1 << 20), (513, 129)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_f32_sum_within_k_scaled_bound(shape):
    """|gpu - f64 sum| <= 2*K*eps32*sum|x|; max/min of floats are order independent, hence exact."""
    rows, cols = shape
    x = RNG.normal(0, 1, rows * cols).astype(np.float32)
    for st in (ShapeTracker.fromShape([rows, cols]), ShapeTracker.fromShape([cols, rows]).permute([1, 0])):
        k = reduceKernel([rows, cols], [(DType.Float32, st)], lambda v: v, AluOp.Add)
        got, _ = device_run(k, [x])
        xs = x.reshape(rows, cols) if st.contiguous else x.reshape(cols, rows).T
        ref = xs.astype(np.float64).sum(axis=1)
        bound = 2 * cols * np.finfo(np.float32).eps * np.abs(xs.astype(np.float64)).sum(axis=1)
        assert np.all(np.abs(got - ref) <= bound)
        want = oracle.run_kernel(k, [x], oracle.MODE_WASM)
        assert np.all(np.abs(want - ref) <= bound)  # the checker's sequential f32 sum obeys the same bound
        for op in (AluOp.Max, AluOp.Min):
            assert_parity(reduceKernel([rows, cols], [(DType.Float32, st)], lambda v: v, op), [x], exact=True, rtol=0, atol=0)


def test_reduction_nan_propagates_and_signed_zero():
    x = np.array([[1.0, np.nan, 3.0, 2.0], [-0.0, 0.0, -0.0, 0.0], [0.0, -0.0, 0.0, -0.0], [-np.inf, 5.0, np.inf, 1.0]],
                 dtype=np.float32)
    st = ShapeTracker.fromShape([4, 4])
    for op in (AluOp.Max, AluOp.Min, AluOp.Add):
        got, want, _ = assert_parity(reduceKernel([4, 4], [(DType.Float32, st)], lambda v: v, op), [x], exact=False)
        np.testing.assert_array_equal(np.signbit(got), np.signbit(want))


def test_bool_reductions():
    x = (RNG.uniform(size=(64, 300)) < 0.01).astype(np.int32)
    x[3] = 0
    x[5] = 1
    st = ShapeTracker.fromShape([64, 300])
    for op in (AluOp.Add, AluOp.Max, AluOp.Mul, AluOp.Min):
        assert_parity(reduceKernel([64, 300], [(DType.Bool, st)], lambda v: v, op), [x], exact=True)


def test_flat_sum_of_ones_100m():
    """src/frontend/array.test.ts:365-374: int32 ones [100,1000,1000] .sum() == 100_000_000 -- one output,
    a 10^8-long fold: exercises the split-over-blocks two-stage path."""
    n = 100_000_000
    k = reduceKernel([1, n], [(DType.Int32, ShapeTracker.fromShape([1]).reshape([1, 1]).expand([1, n]))],
                     lambda v: v, AluOp.Add)
    got, ks = device_run(k, [np.ones(1, dtype=np.int32)])
    assert got[0] == n
    x = RNG.integers(-3, 4, size=10_000_001).astype(np.int32)
    k = reduceKernel([1, len(x)], [(DType.Int32, ShapeTracker.fromShape([1, len(x)]))], lambda v: v, AluOp.Add)
    got, ks = device_run(k, [x])
    assert "fold" in ks.klass
    assert got[0] == int(x.astype(np.int64).sum())


def test_reduce_epilogue_with_buffer_loads():
    """A fused epilogue may read other buffers at the output position (src/frontend/jit.ts:861-883)."""
    rows, cols = 300, 257
    x = RNG.normal(0, 1, rows * cols).astype(np.float32)
    bias = RNG.normal(0, 1, rows).astype(np.float32)
    idx = unravelAlu([rows], AluVar.gidx) + [AluVar.ridx]
    exp = AluExp.globalView(DType.Float32, 0, ShapeTracker.fromShape([rows, cols]), idx)
    acc = AluVar.acc(DType.Float32)
    b = AluExp.globalView(DType.Float32, 1, ShapeTracker.fromShape([rows]), [AluVar.gidx])
    epi = AluExp.max(AluExp.add(AluExp.mul(acc, AluExp.f32(1.0 / cols)), b), AluExp.f32(0))
    for st_perm in (False, True):
        e = exp if not st_perm else AluExp.globalView(
            DType.Float32, 0, ShapeTracker.fromShape([cols, rows]).permute([1, 0]), idx)
        k = Kernel(2, rows, e, Reduction(DType.Float32, AluOp.Add, cols, epi))
        assert_parity(k, [x, bias], rtol=1e-4, atol=1e-5)


def _c2_kernels(rows, L):
    """The four row-reduce kernels config 2 issues (no jaxpr-level CSE, src/frontend/jaxpr.ts:659-715):
    m = max(x); y = sum(exp(x-m)*sigmoid(x)); m' = max(x) inside argmax (src/library/numpy.ts:546);
    idx = L - max(where(x == m', L - i, 0)) (numpy.ts:547-555)."""
    st = ShapeTracker.fromShape([rows, L])
    stm = ShapeTracker.fromShape([rows]).reshape([rows, 1]).expand([rows, L])
    f = DType.Float32
    kmax = reduceKernel([rows, L], [(f, st)], lambda x: x, AluOp.Max)

    def body(x, m):
        xm = AluExp.add(x, AluExp.sub(AluExp.f32(0), m))                 # x - m as add(x, 0 - m)
        sig = AluExp.reciprocal(AluExp.add(AluExp.exp(AluExp.sub(AluExp.f32(0), x)), AluExp.f32(1)))
        return AluExp.mul(AluExp.exp(xm), sig)

    ksum = reduceKernel([rows, L], [(f, st), (f, stm)], body, AluOp.Add)
    star = ShapeTracker.fromShape([L]).reshape([1, L]).expand([rows, L])

    def arg_body(x, m, rev):
        is_max = AluExp.cmpne(x, m).not_()
        return AluExp.mul(AluExp.cast(DType.Int32, is_max), rev)

    karg = reduceKernel([rows, L], [(f, st), (f, stm), (DType.Int32, star)], arg_body, AluOp.Max,
                        epilogue=lambda acc: AluExp.sub(AluExp.i32(L), acc))
    return kmax, ksum, karg


@pytest.mark.parametrize("rows,L", [(64, 4096), (33, 1000)])
def test_config2_small_matches_checker(rows, L):
    x = RNG.normal(0, 1, rows * L).astype(np.float32)
    rev = np.arange(L, 0, -1, dtype=np.int32)
    kmax, ksum, karg = _c2_kernels(rows, L)
    m, _, _ = assert_parity(kmax, [x], exact=True, rtol=0, atol=0)
    got, ks = device_run(ksum, [x, m])
    want = oracle.run_kernel(ksum, [x, m], oracle.MODE_WASM)
    xs = x.reshape(rows, L).astype(np.float64)
    terms = np.exp(xs - m[:, None]) / (1 + np.exp(-xs))
    bound = 2 * L * np.finfo(np.float32).eps * terms.sum(axis=1) + 1e-5 * terms.sum(axis=1)
    assert np.all(np.abs(got - terms.sum(axis=1)) <= bound) and np.all(np.abs(want - terms.sum(axis=1)) <= bound)
    idx, widx, _ = assert_parity(karg, [x, m, rev], exact=True)
    np.testing.assert_array_equal(idx, np.argmax(x.reshape(rows, L), axis=1).astype(np.int32))


def test_config2_full_size_properties():
    """x f32 [8192, 4096]: argmax bit-exact against numpy's first-index rule; the fused sum against an f64
    evaluation under the K-scaled bound; rows are independent, so a spot-check of 16 rows through the
    checker covers the rest of the path."""
    rows, L = 8192, 4096
    x = RNG.normal(0, 1, rows * L).astype(np.float32)
    x[5 * L + 17] = x[5 * L + 900] = 9.5  # a tie: the first index must win (test/argreduce.test.ts:14-70)
    rev = np.arange(L, 0, -1, dtype=np.int32)
    kmax, ksum, karg = _c2_kernels(rows, L)
    m, _ = device_run(kmax, [x])
    np.testing.assert_array_equal(m, x.reshape(rows, L).max(axis=1))
    y, _ = device_run(ksum, [x, m])
    idx, _ = device_run(karg, [x, m, rev])
    np.testing.assert_array_equal(idx, np.argmax(x.reshape(rows, L), axis=1).astype(np.int32))
    assert idx[5] == 17
    sel = list(range(0, rows, rows // 16))
    want = oracle.run_kernel(ksum, [x, m], oracle.MODE_WASM, gidx=sel)
    xs = x.reshape(rows, L)[sel].astype(np.float64)
    terms = (np.exp(xs - m[sel, None]) / (1 + np.exp(-xs))).sum(axis=1)
    assert np.all(np.abs(y[sel] - terms) <= (2 * L * np.finfo(np.float32).eps + 1e-5) * terms)
    np.testing.assert_allclose(y[sel], want, rtol=1e-5)


@pytest.mark.parametrize("M,K", [(64, 256), (130, 264), (11008, 4096)], ids=lambda v: str(v))
@pytest.mark.parametrize("transposed", [False, True], ids=["W[M,K]", "W[K,M]"])
def test_matvec_f16(M, K, transposed):
    """Config 3.  f16 operands, f32 accumulation, f16 result: rtol 1e-2 on outputs, and the f32 accumulator
    (before the final rounding) inside the K-scaled bound of an exact f64 dot product."""
    W = RNG.normal(0, 0.02, (M, K)).astype(np.float16)
    x = RNG.normal(0, 1, K).astype(np.float16)
    k = matvecKernel(M, K, DType.Float16, w_transposed=transposed)
    Wbuf = np.ascontiguousarray(W.T) if transposed else W
    got, ks = device_run(k, [Wbuf, x])
    ref = W.astype(np.float64) @ x.astype(np.float64)
    mag = np.abs(W.astype(np.float64)) @ np.abs(x.astype(np.float64))
    half_ulp = np.abs(ref) * 2.0**-11 + 2.0**-25
    assert np.all(np.abs(got.astype(np.float64) - ref) <= 2 * K * np.finfo(np.float32).eps * mag + half_ulp)
    if M * K <= 1 << 16:
        want = oracle.run_kernel(k, [Wbuf, x], oracle.MODE_CPU)
        np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-2, atol=1e-4)


# ---- rows and views off the vector grid: wide loads from addresses aligned to one element only ----------------

def _sum_kernel(dt, rows, L, over_rows):
    st = ShapeTracker.fromShape([rows, L])
    if over_rows:  # reduce axis 0: outputs are the L columns
        return reduceKernel([L, rows], [(dt, st.permute([1, 0]))], lambda v: AluExp.cast(DType.Float32 if dt != DType.Int32 else dt, v), AluOp.Add)
    return reduceKernel([rows, L], [(dt, st)], lambda v: AluExp.cast(DType.Float32 if dt != DType.Int32 else dt, v), AluOp.Add)


@pytest.mark.parametrize("dt,rows,L,over_rows", [
    (DType.Float16, 257, 4095, False), (DType.Float32, 300, 1001, False), (DType.Int32, 64, 4099, False),
    (DType.Float16, 1000, 1007, True), (DType.Float16, 4096, 1003, True), (DType.Int32, 4096, 1003, True), (DType.Float32, 33, 70001, True),
], ids=str)
def test_sums_over_rows_of_odd_length_use_wide_loads_and_stay_exact(dt, rows, L, over_rows):
    """Small integer data (every partial sum exact in float32): the results must equal numpy's bit for bit whatever
    lane layout the tuner picks; the plan must show the wide (`V` > 1) loads, which used to need aligned rows, and a
    column sum whose width is not a multiple of V runs its leftover columns through the shared tail."""
    from jaxjs_hip.tuner import tuneHip
    k = _sum_kernel(dt, rows, L, over_rows)
    t = tuneHip(k)
    assert t.params["V"] > 1 and "vector_u" in t.vector_loads.values(), (t.klass, t.params)
    npdt = {DType.Float16: np.float16, DType.Float32: np.float32, DType.Int32: np.int32}[dt]
    x = RNG.integers(-3, 4, (rows, L)).astype(npdt)
    got, ks = device_run(k, [x])
    want = x.astype(np.int64).sum(0 if over_rows else 1)
    np.testing.assert_array_equal(got.astype(np.int64), want, err_msg=f"{ks.klass} {ks.info}")
    if over_rows:
        assert L % t.params["V"] != 0  # leftover columns exist


def test_shifted_views_in_a_map_use_wide_loads():
    """x[1:] - x[:-1] and x[3:] * x[:-3] over float16 and float32: the shifted operand starts off the vector grid."""
    from jaxjs_hip.tuner import tuneHip
    for dt, npdt, n, shift in ((DType.Float16, np.float16, 100001, 1), (DType.Float32, np.float32, 65539, 3)):
        st = ShapeTracker.fromShape([n + shift])
        k = mapKernel([n], [(dt, st.shrink([(shift, n + shift)])), (dt, st.shrink([(0, n)]))], lambda a, b: AluExp.sub(AluExp.mul(a, b), b))
        assert "vector_u" in tuneHip(k).vector_loads.values()
        x = RNG.integers(-5, 6, n + shift).astype(npdt)
        got, _ = device_run(k, [x, x])
        np.testing.assert_array_equal(got, x[shift:] * x[:-shift] - x[:-shift])


# ---- materialised transposes / axis permutations: 64 x 64 tiles through LDS -------------------------------------

TRANSPOSED_MAPS = [
    # buffer shape, permutation, dtype
    ((1000, 4096), (1, 0), DType.Float16), ((777, 333), (1, 0), DType.Float32), ((4096, 1000), (1, 0), DType.Int32),
    ((5, 300, 200), (0, 2, 1), DType.Float16), ((300, 7, 200), (2, 1, 0), DType.Float32), ((64, 3, 5, 100), (3, 1, 2, 0), DType.Uint32),
]


@pytest.mark.parametrize("shape,perm,dt", TRANSPOSED_MAPS, ids=str)
def test_materialised_permutations_go_through_lds_tiles_and_are_exact(shape, perm, dt):
    """`x.transpose(perm)` written out, bare and under an elementwise expression with a cast: the tile class must be
    picked, every element must land where numpy puts it, ragged tile edges and the remaining axes included."""
    from jaxjs_hip.tuner import tuneHip
    npdt = {DType.Float16: np.float16, DType.Float32: np.float32, DType.Int32: np.int32, DType.Uint32: np.uint32}[dt]
    st = ShapeTracker.fromShape(list(shape)).permute(list(perm))
    x = RNG.integers(0, 100, shape).astype(npdt)
    want = np.ascontiguousarray(x.transpose(perm))
    k = mapKernel(list(st.shape), [(dt, st)], lambda v: v)
    assert tuneHip(k).klass == "map_t"
    got, ks = device_run(k, [x])
    assert ks.klass == "map_t"
    np.testing.assert_array_equal(got.reshape(want.shape), want)
    if dt in (DType.Float16, DType.Float32):
        k2 = mapKernel(list(st.shape), [(dt, st)], lambda v: AluExp.cast(DType.Float32, AluExp.add(AluExp.mul(v, AluExp.const(dt, 2.0)), AluExp.const(dt, 1.0))))
        got, ks = device_run(k2, [x])
        assert ks.klass == "map_t" and got.dtype == np.float32
        np.testing.assert_array_equal(got.reshape(want.shape), want.astype(np.float32) * 2 + 1)


def test_transposed_view_with_an_offset_and_the_cases_that_stay_plain_maps():
    from jaxjs_hip.tuner import tuneHip
    R, C = 300, 500
    buf = RNG.integers(0, 100, R * C + 7).astype(np.float32)
    st = ShapeTracker.fromShape([R * C + 7]).shrink([(7, R * C + 7)]).reshape([R, C]).permute([1, 0])
    k = mapKernel([C, R], [(DType.Float32, st)], lambda v: v)
    got, ks = device_run(k, [buf])
    assert ks.klass == "map_t"
    np.testing.assert_array_equal(got.reshape(C, R), buf[7:].reshape(R, C).T)
    # two operands, a position-dependent expression, an innermost axis kept in place, a small array: the plain map
    t2 = ShapeTracker.fromShape([512, 512]).permute([1, 0])
    assert tuneHip(mapKernel([512, 512], [(DType.Float32, t2), (DType.Float32, ShapeTracker.fromShape([512, 512]))], lambda a, b: AluExp.add(a, b))).klass == "map"
    assert tuneHip(mapKernel([512, 512], [(DType.Float32, t2)], lambda a: AluExp.add(a, AluExp.cast(DType.Float32, AluVar.gidx)))).klass == "map"
    assert tuneHip(mapKernel([8, 64, 12, 64], [(DType.Float16, ShapeTracker.fromShape([8, 12, 64, 64]).permute([0, 2, 1, 3]))], lambda a: a)).klass == "map"
    assert tuneHip(mapKernel([100, 100], [(DType.Float32, ShapeTracker.fromShape([100, 100]).permute([1, 0]))], lambda a: a)).klass == "map"
