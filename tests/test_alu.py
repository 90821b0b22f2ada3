"""IR host logic: evaluation semantics, range analysis and the simplifier.

Vectors are the ones the reference's own IR tests assert (src/alu.test.ts); the simplifier is
additionally checked by brute force on random index expressions.
"""
import math
import random

import pytest

from jaxjs_hip.alu import AluExp, AluOp, AluVar, DType, Kernel, Reduction, erf, erfc, threefry2x32


def test_evaluate_basic():  # src/alu.test.ts:5-18
    assert AluExp.i32(3).evaluate({}) == 3
    e2 = AluExp.add(AluExp.i32(3), AluExp.i32(4))
    assert e2.evaluate({}) == 7
    assert AluExp.add(AluExp.i32(3), e2).evaluate({}) == 10
    e4 = AluExp.mul(AluExp.special(DType.Int32, "idx", 10), AluExp.i32(50))
    assert e4.evaluate({"idx": 10}) == 500


def test_ternary():  # src/alu.test.ts:20-35
    x = AluExp.special(DType.Int32, "x", 100)
    e = AluExp.where(AluExp.cmplt(x, AluExp.i32(70)), AluExp.i32(0), AluExp.i32(1))
    assert e.dtype == DType.Int32 and len(e.src) == 3 and e.src[0].dtype == DType.Bool
    assert [e.evaluate({"x": v}) for v in (50, 69, 70, 80)] == [0, 0, 1, 1]


def test_bool_ops():  # src/alu.test.ts:37-48: Add is OR, Mul is AND
    t, f = AluExp.bool(True), AluExp.bool(False)
    assert [AluExp.mul(a, b).evaluate({}) for a, b in ((t, t), (t, f), (f, f))] == [1, 0, 0]
    assert [AluExp.add(a, b).evaluate({}) for a, b in ((t, t), (t, f), (f, f))] == [1, 1, 0]


def test_min_max_range():  # src/alu.test.ts:50-61
    e = AluExp.add(AluExp.i32(3), AluExp.i32(4))
    assert (e.min, e.max) == (7, 7)
    e2 = AluExp.add(AluExp.special(DType.Int32, "x", 10), AluExp.special(DType.Int32, "y", 20))
    assert (e2.min, e2.max) == (0, 28)


def test_type_errors():  # src/alu.test.ts:63-67
    for f in (AluExp.sin, AluExp.cos, AluExp.reciprocal):
        with pytest.raises(TypeError):
            f(AluExp.bool(True))


def test_cmpne_nan():  # src/alu.test.ts:86-94
    assert AluExp.cmpne(AluExp.i32(3), AluExp.i32(4)).evaluate({}) == 1
    assert AluExp.cmpne(AluExp.i32(5), AluExp.i32(5)).evaluate({}) == 0
    assert AluExp.cmpne(AluExp.f32(2.5), AluExp.f32(2.5)).evaluate({}) == 0
    assert AluExp.cmpne(AluExp.f32(math.nan), AluExp.f32(math.nan)).evaluate({}) == 1


def test_transcendentals():  # src/alu.test.ts:96-143
    assert AluExp.exp(AluExp.f32(3)).evaluate({}) == pytest.approx(math.e**3)
    assert AluExp.log(AluExp.f32(8)).evaluate({}) == pytest.approx(math.log(8))
    assert math.isnan(AluExp.log(AluExp.f32(-1)).evaluate({}))
    assert AluExp.erf(AluExp.f32(1)).evaluate({}) == pytest.approx(0.84270079, abs=1e-5)
    assert AluExp.erf(AluExp.f32(0)).evaluate({}) == pytest.approx(0.0, abs=1e-5)
    assert AluExp.erf(AluExp.f32(-1)).evaluate({}) == pytest.approx(-0.84270079, abs=1e-5)
    assert AluExp.erfc(AluExp.f32(1)).evaluate({}) == pytest.approx(0.15729921, abs=1e-5)
    assert AluExp.erfc(AluExp.f32(100)).evaluate({}) == pytest.approx(0.0, abs=1e-5)
    assert AluExp.erfc(AluExp.f32(-1)).evaluate({}) == pytest.approx(1.84270079, abs=1e-5)
    assert AluExp.sqrt(AluExp.f32(16)).evaluate({}) == 4
    # The IR's erf is the A&S approximation, which differs measurably from libm's.
    assert abs(erf(0.5) - math.erf(0.5)) < 2e-7 and erf(0.5) != math.erf(0.5)
    assert abs(erfc(0.5) - math.erfc(0.5)) < 2e-7


def test_cast():  # src/alu.test.ts:145-172
    assert AluExp.cast(DType.Float32, AluExp.i32(42)).evaluate({}) == 42
    assert AluExp.cast(DType.Int32, AluExp.f32(3.14)).evaluate({}) == 3
    assert AluExp.cast(DType.Int32, AluExp.bool(True)).evaluate({}) == 1
    assert AluExp.cast(DType.Bool, AluExp.i32(5)).evaluate({}) == 1
    assert AluExp.cast(DType.Bool, AluExp.i32(0)).evaluate({}) == 0
    e6 = AluExp.cast(DType.Uint32, AluExp.variable(DType.Int32, "x"))
    assert e6.min == 0 and e6.max >= 4294967295
    # Saturating float->int casts, NaN -> 0 (src/frontend/array.test.ts:415-432).
    big = AluExp.variable(DType.Float32, "v")
    assert AluExp.cast(DType.Int32, big).evaluate({"v": 1e20}) == 2147483647
    assert AluExp.cast(DType.Int32, big).evaluate({"v": -1e20}) == -2147483648
    assert AluExp.cast(DType.Uint32, big).evaluate({"v": 1e20}) == 4294967295
    assert AluExp.cast(DType.Uint32, big).evaluate({"v": -1e20}) == 0
    assert AluExp.cast(DType.Int32, big).evaluate({"v": math.nan}) == 0


def test_bitcast():  # src/alu.test.ts:174-200
    assert AluExp.bitcast(DType.Float32, AluExp.i32(0x3F800000)).evaluate({}) == 1.0
    assert AluExp.bitcast(DType.Int32, AluExp.f32(math.inf)).evaluate({}) == 0x7F800000
    assert AluExp.bitcast(DType.Int32, AluExp.f32(math.nan)).evaluate({}) == 0x7FC00000
    assert AluExp.bitcast(DType.Uint32, AluExp.i32(-1)).evaluate({}) == 0xFFFFFFFF
    for dt, src in ((DType.Bool, AluExp.i32(1)), (DType.Float32, AluExp.bool(True)), (DType.Int32, AluExp.bool(False)),
                    (DType.Uint32, AluExp.bool(True)), (DType.Bool, AluExp.f32(1.0))):
        with pytest.raises(TypeError):
            AluExp.bitcast(dt, src)


def test_threefry_kat():  # src/alu.test.ts:202-209, src/backend/wasm/builtins.test.ts:222-232
    assert threefry2x32(0, 0, 0, 0) == (1797259609, 2579123966)
    z = AluExp.u32(0)
    assert AluExp.threefry2x32(z, z, z, z).evaluate({}) == (1797259609 ^ 2579123966)
    assert AluExp.threefry2x32(z, z, z, z, 0).evaluate({}) == 1797259609
    assert AluExp.threefry2x32(z, z, z, z, 1).evaluate({}) == 2579123966


def test_idiv_mod_signs():  # src/alu.test.ts:211-272
    assert AluExp.idiv(AluExp.i32(7), AluExp.i32(3)).evaluate({}) == 2
    e2 = AluExp.idiv(AluExp.i32(-7), AluExp.i32(3))
    assert e2.evaluate({}) == -2 and (e2.min, e2.max) == (-2, -2)
    assert AluExp.mod(AluExp.i32(7), AluExp.i32(3)).evaluate({}) == 1
    assert AluExp.mod(AluExp.i32(-7), AluExp.i32(3)).evaluate({}) == -1
    assert AluExp.mod(AluExp.i32(7), AluExp.i32(-3)).evaluate({}) == 1
    assert AluExp.mod(AluExp.f32(5.5), AluExp.f32(-1.7)).evaluate({}) == pytest.approx(0.4)


@pytest.mark.parametrize("mulc,addc,div", [(2, -1, 2), (-2, 1, -2)])
def test_idiv_simplify_negative(mulc, addc, div):  # src/alu.test.ts:222-252
    i = AluExp.special(DType.Int32, "i", 3)
    e = AluExp.idiv(AluExp.add(AluExp.mul(i, AluExp.i32(mulc)), AluExp.i32(addc)), AluExp.i32(div))
    vals = [e.evaluate({"i": v}) for v in range(3)]
    assert vals == [0, 0, 1]
    assert [e.simplify().evaluate({"i": v}) for v in range(3)] == vals


def test_floor_ceil():  # src/alu.test.ts:274-302
    assert AluExp.floor(AluExp.f32(3.7)).evaluate({}) == 3
    assert AluExp.floor(AluExp.f32(-2.3)).evaluate({}) == -3
    assert AluExp.floor(AluExp.i32(0)).op == AluOp.Const
    assert AluExp.floor(AluExp.f32(math.inf)).evaluate({}) == math.inf
    assert AluExp.ceil(AluExp.f32(3.2)).evaluate({}) == 4
    assert AluExp.ceil(AluExp.f32(-2.8)).evaluate({}) == -2


def test_shr_is_logical_and_int_wraps():  # src/alu.ts:1088-1091; wasm/translation.ts:101-103
    a = AluExp.variable(DType.Int32, "a")
    assert AluExp.bitShift(a, AluExp.i32(28), "shr").evaluate({"a": -1}) == 15
    assert AluExp.add(a, AluExp.i32(1)).evaluate({"a": 2147483647}) == -2147483648
    assert AluExp.mul(a, AluExp.i32(65536)).evaluate({"a": 65536}) == 0


def test_interning_gives_structural_identity():
    g = AluVar.gidx
    a = AluExp.add(AluExp.mul(g, AluExp.i32(3)), AluExp.i32(1))
    b = AluExp.add(AluExp.mul(g, AluExp.i32(3)), AluExp.i32(1))
    assert a is b
    assert AluExp.f32(0.0) is not AluExp.f32(-0.0)
    assert AluExp.f32(math.nan) is AluExp.f32(math.nan)


def test_reduction_f16_add_accumulates_in_f32():  # src/alu.ts:1560-1568
    r = Reduction(DType.Float16, AluOp.Add, 8)
    assert r.dtype == DType.Float32 and r.epilogue.dtype == DType.Float16
    assert r.epilogue.op == AluOp.Cast and r.epilogue.src[0] is AluVar.acc(DType.Float32)
    r2 = Reduction(DType.Float16, AluOp.Max, 8)
    assert r2.dtype == DType.Float16


def test_reduction_identities():  # src/alu.ts:1584-1604
    ident = lambda d, o: Reduction(d, o, 1).identity  # noqa: E731
    assert ident(DType.Int32, AluOp.Min) == 0x7FFFFFFF and ident(DType.Int32, AluOp.Max) == -(1 << 31)
    assert ident(DType.Uint32, AluOp.Min) == 0xFFFFFFFF and ident(DType.Uint32, AluOp.Max) == 0
    assert ident(DType.Float32, AluOp.Min) == math.inf and ident(DType.Float32, AluOp.Max) == -math.inf
    assert ident(DType.Bool, AluOp.Add) == 0 and ident(DType.Bool, AluOp.Mul) == 1
    assert ident(DType.Bool, AluOp.Max) == 0 and ident(DType.Bool, AluOp.Min) == 1


def test_kernel_dtype_and_bytes():
    k = Kernel(0, 200, AluExp.cast(DType.Float32, AluVar.gidx))
    assert k.dtype == DType.Float32 and k.bytes == 800
    r = Reduction(DType.Float16, AluOp.Add, 4)
    k2 = Kernel(0, 10, AluExp.cast(DType.Float16, AluVar.ridx), r)
    assert k2.dtype == DType.Float16 and k2.bytes == 20


def _random_index_exp(rng, leaves, depth):
    if depth == 0 or rng.random() < 0.2:
        return rng.choice(leaves) if rng.random() < 0.7 else AluExp.i32(rng.choice([0, 1, 2, 3, 4, 6, 8, 12, 16, -1, -3]))
    a = _random_index_exp(rng, leaves, depth - 1)
    kind = rng.random()
    c = AluExp.i32(rng.choice([1, 2, 3, 4, 5, 6, 8, 12, 16, 24, 32]))
    if kind < 0.25:
        return AluExp.add(a, _random_index_exp(rng, leaves, depth - 1))
    if kind < 0.45:
        return AluExp.mul(a, c) if rng.random() < 0.7 else AluExp.mul(c, a)
    if kind < 0.65:
        return AluExp.idiv(a, c)
    if kind < 0.85:
        return AluExp.mod(a, c)
    if kind < 0.9:
        return AluExp.sub(a, _random_index_exp(rng, leaves, depth - 1))
    if kind < 0.95:
        return AluExp.where(AluExp.cmplt(a, c), a, _random_index_exp(rng, leaves, depth - 1))
    return AluExp.max(a, AluExp.min(_random_index_exp(rng, leaves, depth - 1), c))


def test_simplify_preserves_values_brute_force():
    rng = random.Random(1234)
    x = AluExp.special(DType.Int32, "x", 7)
    y = AluExp.special(DType.Int32, "y", 12)
    z = AluExp.special(DType.Int32, "z", 5)
    changed = 0
    for _ in range(1500):
        e = _random_index_exp(rng, [x, y, z], 4)
        s = e.simplify()
        changed += s is not e
        for xv in range(7):
            for yv in (0, 1, 5, 11):
                for zv in (0, 2, 4):
                    ctx = {"x": xv, "y": yv, "z": zv}
                    v = e.evaluate(ctx)
                    assert s.evaluate(ctx) == v, (e, s, ctx)
                    assert e.min <= v <= e.max, (e, ctx)
    assert changed > 300


def test_simplify_unravel_roundtrip():  # src/shape.test.ts:401-417
    from jaxjs_hip.shape import ShapeTracker, unravelAlu

    idx = AluExp.special(DType.Int32, "idx", 200)
    for shape in ([10, 20], [5, 2, 20]):
        st = ShapeTracker.fromShape(shape)
        iexpr, vexpr = st.toAluExp(unravelAlu(st.shape, idx))
        assert vexpr.resolve() == 1
        assert iexpr is idx


def test_unsigned_and_signed_wraparound_is_not_folded_away():
    """`0 - x` on uint32 wraps to 2^32 - x: its range is unknown, not [0, 0]; same for int32 products that overflow.
    (Found by differential fuzzing: min(c, (0 - u) * (u * u) / 7) had been folded to the constant 0.)"""
    u = AluExp.special(DType.Uint32, "u", 1 << 20)
    neg = AluExp.sub(AluExp.u32(0), u)
    assert neg.max > 0 and neg.simplify().op != AluOp.Const
    e = AluExp.min(AluExp.u32(12345), AluExp.idiv(AluExp.mul(neg, AluExp.mul(u, u)), AluExp.u32(7))).simplify()
    assert e.op != AluOp.Const
    assert e.evaluate({"u": 3}) == min(12345, (((0 - 3) % 2**32) * 9 % 2**32) // 7)
    i = AluExp.special(DType.Int32, "i", 1 << 20)
    sq = AluExp.mul(AluExp.mul(i, i), AluExp.i32(4096))  # up to 2^52 mathematically: wraps in int32
    assert AluExp.cmplt(sq, AluExp.i32(0)).simplify().op != AluOp.Const
