"""View / ShapeTracker algebra against the vectors of the reference's shape tests (src/shape.test.ts)
plus a brute-force check of every movement op against numpy on small arrays."""
import itertools
import random

import numpy as np
import pytest

from jaxjs_hip.alu import AluExp, DType
from jaxjs_hip.shape import ShapeTracker, View, unravelAlu


def test_create():  # src/shape.test.ts:6-50
    v = View.create([10, 2, 3])
    assert v.shape == (10, 2, 3) and v.strides == (6, 3, 1) and v.offset == 0 and v.mask is None
    with pytest.raises(ValueError, match="non-negative"):
        View.create([-1, 3])
    assert View.create([0, 5]).strides == (0, 0)
    assert View.create([2, 3], [1, 2], 40).strides == (1, 2)
    assert View.create([3, 10], [10, 1], 0, [(0, 3), (0, 10)]).mask is None
    assert View.create([3, 10], [10, 1], 0, [(0, 0), (0, 10)]).mask == ((0, 0), (0, 0))


def test_size_contiguous():  # src/shape.test.ts:52-72
    assert View.create([2, 3, 4]).size == 24
    assert View.create([]).size == 1
    assert View.create([2, 3]).contiguous
    assert not View.create([2, 3]).flip([True, False]).contiguous


def test_pad_shrink_expand_permute_flip():  # src/shape.test.ts:74-197
    v = View.create([3, 3])
    assert v.pad([(0, 0), (0, 0)]) is v
    p = v.pad([(1, 2), (3, 4)])
    assert p.shape == (6, 10) and p.offset == -6 and p.mask == ((1, 4), (3, 6))
    with pytest.raises(ValueError):
        v.pad([(0, -1), (0, 0)])
    s = View.create([5, 5]).shrink([(1, 4), (2, 5)])
    assert s.shape == (3, 3) and s.offset == 7
    with pytest.raises(ValueError):
        View.create([5, 5]).shrink([(4, 1), (0, 5)])
    e = View.create([10, 1, 3]).expand([10, 4, 3])
    assert e.shape == (10, 4, 3) and e.strides == (3, 0, 1)
    with pytest.raises(ValueError, match="Can't expand"):
        View.create([2, 3]).expand([3, 3])
    v3 = View.create([2, 3, 4])
    pm = v3.permute([2, 0, 1])
    assert pm.shape == (4, 2, 3) and pm.strides == (v3.strides[2], v3.strides[0], v3.strides[1])
    with pytest.raises(ValueError, match="Invalid permutation"):
        View.create([2, 3]).permute([0, 0])
    f = View.create([2, 3]).flip([True, False])
    assert f.offset == 3 and f.strides == (-3, 1)
    with pytest.raises(ValueError):
        View.create([2, 3]).flip([True])


def test_reshape():  # src/shape.test.ts:199-262
    v = View.create([2, 3])
    assert v.reshape([3, 2]).shape == (3, 2)
    assert v.reshape([2, 3]) is v
    with pytest.raises(ValueError, match="Reshape size"):
        v.reshape([4, 2])
    r = (
        View.create([240])
        .reshape([2, 2, 6, 1, 10])
        .permute([1, 0, 2, 3, 4])
        .pad([(1, 1), (2, 3), (0, 0), (0, 0), (0, 0)])
        .reshape([4, 7, 3, 2, 10])
    )
    assert r.mask == ((1, 3), (2, 4), (0, 3), (0, 2), (0, 10))
    assert r.offset == -300 and r.shape == (4, 7, 3, 2, 10) and r.strides == (60, 120, 20, 10, 1)


def test_minify_compose():  # src/shape.test.ts:264-327
    assert View.create([1, 3, 1, 4]).minify().shape == (12,)
    vf = View.create([2, 3]).flip([True, False])
    assert vf.minify().shape == vf.shape
    v1, v2 = View.create([2, 3]), View.create([2, 3])
    assert v2.compose(v1) is v1
    assert View.create([2, 3]).compose(vf) is vf
    bad = v1.flip([True, False]).shrink([(0, 2), (0, 2)])
    assert bad.compose(v1) is None
    a = View.create([1, 10, 784], [0, 0, 1])
    b = View.create([1, 10, 196, 4])
    assert b.strides == (0, 784, 4, 1)
    for c in (a.compose(b), a.reshape(b.shape)):
        assert c is not None and c.shape == (1, 10, 196, 4) and c.strides == (0, 0, 4, 1)


def test_shapetracker_views():  # src/shape.test.ts:329-345
    base = ShapeTracker.fromShape([2, 3])
    assert base.reshape([6]).compose(base) == base
    flipped = base.flip([True, False])
    assert len(flipped.views) == 1
    assert flipped.reshape([3, 2]).views == (flipped.views[0], View.create([3, 2]))


def test_to_alu_exp():  # src/shape.test.ts:347-399
    v = View.create([200])
    exp, vexp = v.toAluExp([AluExp.special(DType.Int32, "x", 200)])
    assert vexp.resolve() == 1 and exp.evaluate({"x": 42}) == 42
    v = View.create([20, 10])
    sp = [AluExp.special(DType.Int32, "x", 20), AluExp.special(DType.Int32, "y", 10)]
    exp, vexp = v.toAluExp(sp)
    assert vexp.resolve() == 1
    assert exp.evaluate({"x": 5, "y": 3}) == 53 and exp.evaluate({"x": 15, "y": 3}) == 153
    exp, vexp = v.flip([True, False]).toAluExp(sp)
    assert vexp.resolve() == 1
    assert exp.evaluate({"x": 5, "y": 3}) == 143 and exp.evaluate({"x": 15, "y": 3}) == 43

    v = View.create([3, 3]).pad([(1, 1), (2, 3)])
    assert v.shape == (5, 8)
    _, vexp = v.toAluExp([AluExp.special(DType.Int32, "x", 5), AluExp.special(DType.Int32, "y", 8)])
    got = [vexp.evaluate({"x": x, "y": y}) for x, y in ((0, 0), (1, 0), (1, 2), (3, 4), (4, 4), (3, 5))]
    assert got == [0, 0, 1, 1, 0, 0]

    st = ShapeTracker.fromShape([2, 2]).pad([(1, 1), (1, 1)]).flip([False, True]).reshape([16])
    exp, vexp = st.toAluExp([AluExp.special(DType.Int32, "x", 16)])
    assert [exp.evaluate({"x": x}) for x in (5, 6, 9, 10)] == [1, 0, 3, 2]
    assert [vexp.evaluate({"x": i}) for i in range(16)] == [int(i in (5, 6, 9, 10)) for i in range(16)]


def _materialize(st: ShapeTracker, base: np.ndarray) -> np.ndarray:
    """Evaluate a tracker element by element through toAluExp."""
    shape = st.shape
    sp = [AluExp.special(DType.Int32, f"i{k}", max(s, 1)) for k, s in enumerate(shape)]
    iexpr, vexpr = st.toAluExp(sp)
    out = np.zeros(shape, dtype=base.dtype)
    for pos in itertools.product(*[range(s) for s in shape]):
        ctx = {f"i{k}": p for k, p in enumerate(pos)}
        if vexpr.evaluate(ctx):
            out[pos] = base[iexpr.evaluate(ctx)]
    return out


def test_movement_ops_match_numpy_brute_force():
    rng = random.Random(7)
    for trial in range(120):
        shape = [rng.choice([1, 2, 3, 4]) for _ in range(rng.choice([1, 2, 3]))]
        base = np.arange(1, int(np.prod(shape)) + 1, dtype=np.int64)
        ref = base.reshape(shape)
        st = ShapeTracker.fromShape(shape)
        for _ in range(rng.choice([1, 2, 3, 4])):
            op = rng.choice(["permute", "flip", "pad", "shrink", "reshape", "expand"])
            nd = ref.ndim
            if op == "permute":
                perm = list(range(nd))
                rng.shuffle(perm)
                st, ref = st.permute(perm), ref.transpose(perm)
            elif op == "flip":
                fl = [rng.random() < 0.5 for _ in range(nd)]
                st = st.flip(fl)
                ref = ref[tuple(slice(None, None, -1) if f else slice(None) for f in fl)]
            elif op == "pad":
                pads = [(rng.choice([0, 1, 2]), rng.choice([0, 1])) for _ in range(nd)]
                st, ref = st.pad(pads), np.pad(ref, pads)
            elif op == "shrink":
                arg = []
                for s in ref.shape:
                    b = rng.randrange(0, s)
                    arg.append((b, rng.randrange(b + 1, s + 1)))
                st = st.shrink(arg)
                ref = ref[tuple(slice(b, e) for b, e in arg)]
            elif op == "reshape":
                n = ref.size
                divs = [d for d in range(1, n + 1) if n % d == 0]
                a = rng.choice(divs)
                new = [a, n // a] if rng.random() < 0.7 else [n]
                st, ref = st.reshape(new), ref.reshape(new)
            elif op == "expand":
                st = st.reshape([1] + list(ref.shape))
                k = rng.choice([1, 2, 3])
                st = st.expand([k] + list(ref.shape))
                ref = np.broadcast_to(ref.reshape((1,) + ref.shape), (k,) + ref.shape)
        assert list(ref.shape) == st.shape
        np.testing.assert_array_equal(_materialize(st, base), ref, err_msg=f"trial {trial}: {st}")
        # A simplified tracker must describe the same array.
        np.testing.assert_array_equal(_materialize(st.simplify(), base), ref, err_msg=f"simplify {trial}: {st}")
