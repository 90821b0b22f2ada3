"""Convolution and pooling through the restated view algebra (src/frontend/convolution.ts) and jit rule
(src/frontend/jit.ts:622-635): the reference's tables (test/conv.test.ts:24-58, 71-80), brute-force window
extraction, and random convolutions against a direct numpy loop -- replayed on the CPU oracle here, and on the GPU
in the `gpu`-marked tests."""
import itertools

import numpy as np
import pytest

from jaxjs_hip import jit as J
from jaxjs_hip import library as L
from jaxjs_hip.alu import AluExp, AluOp, DType
from jaxjs_hip.convolution import ConvParams, checkConvShape, pool, prepareConv
from jaxjs_hip.jit import ShapedArray
from jaxjs_hip.shape import ShapeTracker
from jit_util import run_program
from oracle.backend import OracleBackend

F32 = DType.Float32


def f32(x):
    return np.asarray(x, dtype=np.float32)


def run_on(backend, fn, *arrays, dtype=F32):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), dtype) for a in arrays])
    return prog, run_program(backend, prog, arrays)


def run(fn, *arrays):
    return run_on(OracleBackend(), fn, *arrays)


def conv_reference(x, w, strides, padding, lhs_dilation=None, rhs_dilation=None):
    """Direct loops in float64: x [N,C,*xs], w [O,C,*ks]."""
    n = x.ndim - 2
    ld = lhs_dilation or [1] * n
    rd = rhs_dilation or [1] * n
    xs = x.shape[2:]
    dil = np.zeros(x.shape[:2] + tuple((s - 1) * d + 1 for s, d in zip(xs, ld)), np.float64)
    dil[(slice(None), slice(None)) + tuple(slice(None, None, d) for d in ld)] = x
    pads = [(max(p0, 0), max(p1, 0)) for p0, p1 in padding]
    dil = np.pad(dil, [(0, 0), (0, 0)] + pads)
    crop = tuple(slice(max(-p0, 0), dil.shape[2 + i] - max(-p1, 0)) for i, (p0, p1) in enumerate(padding))
    dil = dil[(slice(None), slice(None)) + crop]
    ks = w.shape[2:]
    out_sp = [-(-(dil.shape[2 + i] - ((ks[i] - 1) * rd[i] + 1) + 1) // strides[i]) for i in range(n)]
    out = np.zeros((x.shape[0], w.shape[0]) + tuple(out_sp), np.float64)
    for o in itertools.product(*[range(s) for s in out_sp]):
        for k in itertools.product(*[range(s) for s in ks]):
            pos = tuple(o[i] * strides[i] + k[i] * rd[i] for i in range(n))
            patch = dil[(slice(None), slice(None)) + pos]          # [N, C]
            out[(slice(None), slice(None)) + o] += patch @ w[(slice(None), slice(None)) + k].astype(np.float64).T
    return out


# ---- the reference's tables ------------------------------------------------------------------------------

def test_1d_convolution_tables():
    x, y = f32([[[1, 2, 3, 4, 5]]]), f32([[[2, 0.5, -1]]])
    _, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "VALID"), x, y)
    np.testing.assert_array_equal(r, [0, 1.5, 3])
    prog, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "SAME"), x, y)
    np.testing.assert_array_equal(r, [-1.5, 0, 1.5, 3, 10.5])
    assert len(prog.kernels) == 1 and prog.kernels[0].reduction.size == 3


def test_same_and_same_lower_padding():
    x, y = np.ones((1, 1, 5), np.float32), np.ones((1, 1, 4), np.float32)
    _, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "SAME"), x, y)
    np.testing.assert_array_equal(r, [3, 4, 4, 3, 2])
    _, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "SAME_LOWER"), x, y)
    np.testing.assert_array_equal(r, [2, 3, 4, 4, 3])


def test_2d_convolution_table():
    x = f32([[3, 1, 5], [2, 2, 9]]).reshape(1, 1, 2, 3)
    y = f32([[1, 2], [3, 4]]).reshape(1, 1, 2, 2)
    _, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1, 1], "VALID"), x, y)
    np.testing.assert_array_equal(r, [19, 53])


def test_transposed_convolution_table():
    """lhsDilation 2 with padding [2,2] (test/conv.test.ts:71-91): lowered to a Dot plus shifted adds, no Conv left."""
    x, k = f32([[[1, 2, 3]]]), f32([[[1, 10, 100]]])
    fn = lambda a, b: L.convGeneralDilated(a, b, [1], [(2, 2)], lhsDilation=[2])
    _, (r,) = run(fn, x, k)
    np.testing.assert_array_equal(r, [100, 10, 201, 20, 302, 30, 3])
    jaxpr, _ = J.trace(fn, [ShapedArray((1, 1, 3), F32), ShapedArray((1, 1, 3), F32)])
    prims = [e.primitive for e in jaxpr.eqns]
    assert "Conv" not in prims and "Dot" in prims and "Shrink" in prims and "Add" in prims


TRANSPOSED_1D = [  # test/conv.test.ts:93-146 and :205-243: dilation, padding, kernel (None = the 3-output, 2-channel one)
    (2, (2, 1), None), (3, (0, 2), None), (2, (-1, 2), None), (2, (4, 3), [[[1, -1, 2, 0, 3]]]), (4, (1, 2), [[[2, -1]]]),
]


@pytest.mark.parametrize("dilation,padding,kernel", TRANSPOSED_1D)
def test_transposed_1d_convolution_lowering_matches_direct_loops(dilation, padding, kernel):
    if kernel is None:
        x = f32([[[1, 2, 3, 4], [5, 6, 7, 8]], [[2, 4, 6, 8], [1, 3, 5, 7]]])
        k = f32([[[1, 0, -1], [2, 1, 0]], [[0, 1, 2], [-1, 0, 1]], [[2, -1, 1], [1, 1, -2]]])
    else:
        x, k = f32([[[1, 2, 3, 4]]]), f32(kernel)
    _, (r,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], [padding], lhsDilation=[dilation]), x, k)
    want = conv_reference(x, k, [1], [padding], [dilation])
    np.testing.assert_array_equal(r.reshape(want.shape), want)


def test_transposed_convolution_downstream_ops_and_integer_dtype():
    """test/conv.test.ts:148-203: the lowered result feeds an add and a split; int32 operands stay int32."""
    x, k = f32([[[1, 2, 3], [4, 5, 6]]]), f32([[[1, 0, -1], [2, 1, 0]], [[0, 1, 2], [-1, 0, 1]]])
    want = conv_reference(x, k, [1], [(2, 1)], [2]) + 1
    _, (a, b) = run(lambda p, q: L.split(L.convGeneralDilated(p, q, [1], [(2, 1)], lhsDilation=[2]).add(1), [3], 2), x, k)
    np.testing.assert_array_equal(a.reshape(1, 2, 3), want[:, :, :3])
    np.testing.assert_array_equal(b.reshape(1, 2, -1), want[:, :, 3:])
    prog = J.jit(lambda p, q: L.convGeneralDilated(p, q, [1], [(2, 1)], lhsDilation=[2]), [ShapedArray((1, 2, 3), DType.Int32), ShapedArray((2, 2, 3), DType.Int32)])
    (ri,) = run_program(OracleBackend(), prog, [x.astype(np.int32), k.astype(np.int32)])
    assert ri.dtype == np.int32
    np.testing.assert_array_equal(ri.reshape(want.shape), want - 1)


def test_zero_dimensional_grouped_and_conv_transpose_tables():
    """test/conv.test.ts:245-262 (a convolution without spatial axes is x @ y^T), :352-398 (feature groups: shapes and
    values), :400-432 (depthwise), :545-618 (convTranspose output shapes for SAME / VALID, 1-D 2x upscale)."""
    _, (z,) = run(lambda a, b: L.convGeneralDilated(a, b, [], "VALID"), f32([[1, 2], [3, 4], [5, 8]]), f32([[6, 4], [3, 2]]))
    assert z.tolist() == [14, 7, 34, 17, 62, 31]
    seen = {}
    for xs, ws, pad, G, want in (((2, 4, 8, 8), (6, 2, 3, 3), "VALID", 2, (2, 6, 6, 6)), ((1, 4, 5, 5), (8, 1, 3, 3), "SAME", 4, (1, 8, 5, 5))):
        J.jit(lambda a, b: seen.__setitem__("g", L.convGeneralDilated(a, b, [1, 1], pad, featureGroupCount=G)) or seen["g"], [ShapedArray(xs, F32), ShapedArray(ws, F32)])
        assert tuple(seen["g"].shape) == want
    x = f32([[1, 2, 3, 4], [5, 6, 7, 8]]).reshape(1, 2, 4)
    y = f32([[1, 0, -1], [1, 1, 1]]).reshape(2, 1, 3)
    _, (g,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "VALID", featureGroupCount=2), x, y)
    assert g.tolist() == [-2, -2, 18, 21]
    xd = f32([[1, 2, 3, 4, 5], [2, 3, 4, 5, 6], [3, 4, 5, 6, 7]]).reshape(1, 3, 5)
    yd = f32([[1, -1], [1, 0], [0, 1]]).reshape(3, 1, 2)
    _, (dw,) = run(lambda a, b: L.convGeneralDilated(a, b, [1], "VALID", featureGroupCount=3), xd, yd)
    assert dw.tolist() == [-1, -1, -1, -1, 2, 3, 4, 5, 4, 5, 6, 7]
    rng = np.random.default_rng(2)
    xg, wg = rng.integers(-3, 4, (2, 6, 7, 5)).astype(np.float32), rng.integers(-3, 4, (4, 3, 3, 2)).astype(np.float32)
    _, (gg,) = run(lambda a, b: L.convGeneralDilated(a, b, [2, 1], [(1, 1), (0, 1)], featureGroupCount=2), xg, wg)
    halves = [conv_reference(xg[:, 3 * i:3 * i + 3], wg[2 * i:2 * i + 2], [2, 1], [(1, 1), (0, 1)]) for i in range(2)]
    np.testing.assert_array_equal(gg.reshape(2, 4, *halves[0].shape[2:]), np.concatenate(halves, 1))
    for bad in ((2, 5, 4), (4, 2, 3)), ((2, 4, 4), (3, 2, 3)), ((2, 4, 4), (4, 1, 3)):
        with pytest.raises(ValueError):
            J.jit(lambda a, b: L.convGeneralDilated(a, b, [1], "VALID", featureGroupCount=2), [ShapedArray(bad[0], F32), ShapedArray(bad[1], F32)])
    shapes = [((1, 1, 4), (1, 1, 3), [2], "SAME", (1, 1, 8)), ((1, 1, 5), (1, 1, 3), [2], "SAME", (1, 1, 10)), ((2, 3, 6), (5, 3, 4), [3], "SAME", (2, 5, 18)),
              ((1, 1, 4), (1, 1, 3), [2], "VALID", (1, 1, 9)), ((1, 1, 5), (1, 1, 3), [2], "VALID", (1, 1, 11)), ((2, 3, 6), (5, 3, 4), [3], "VALID", (2, 5, 19)),
              ((1, 1, 4, 4), (1, 1, 3, 3), [2, 2], "SAME", (1, 1, 8, 8)), ((2, 3, 8, 8), (5, 3, 3, 3), [2, 2], "SAME", (2, 5, 16, 16)),
              ((1, 2, 5, 7), (4, 2, 4, 4), [2, 3], "SAME", (1, 4, 10, 21)), ((1, 1, 4, 4), (1, 1, 3, 3), [2, 2], "VALID", (1, 1, 9, 9)),
              ((1, 2, 5, 5), (4, 2, 4, 4), [2, 2], "VALID", (1, 4, 12, 12))]
    for xs, ks, st, pad, want in shapes:
        J.jit(lambda a, b: seen.__setitem__("t", L.convTranspose(a, b, st, pad)) or seen["t"], [ShapedArray(xs, F32), ShapedArray(ks, F32)])
        assert tuple(seen["t"].shape) == want, (xs, ks, st, pad)
    _, (up,) = run(lambda a, b: L.convTranspose(a, b, [2], "SAME"), f32([[[1, 2, 3]]]), f32([[[1, 1]]]))
    assert up.tolist() == [1, 1, 2, 2, 3, 3]
    xt, kt = rng.integers(-3, 4, (1, 2, 4, 3)).astype(np.float32), rng.integers(-3, 4, (3, 2, 3, 2)).astype(np.float32)
    _, (t2,) = run(lambda a, b: L.convTranspose(a, b, [2, 3], "SAME"), xt, kt)
    pads = [L._conv_transpose_padding(3, 2, "SAME"), L._conv_transpose_padding(2, 3, "SAME")]
    want = conv_reference(xt, kt, [1, 1], pads, [2, 3])
    np.testing.assert_array_equal(t2.reshape(want.shape), want)
    _, (t3,) = run(lambda a, b: L.convTranspose(a, b, [2, 3], "SAME", transposeKernel=True), xt, np.ascontiguousarray(np.flip(kt, (2, 3)).transpose(1, 0, 2, 3)))
    np.testing.assert_array_equal(t3, t2)


# ---- brute force --------------------------------------------------------------------------------------------

CONV_CASES = [
    dict(x=(2, 3, 9), w=(4, 3, 3), strides=[1], padding=[(0, 0)]),
    dict(x=(2, 3, 9), w=(4, 3, 3), strides=[2], padding=[(1, 2)]),
    dict(x=(1, 2, 10), w=(3, 2, 3), strides=[1], padding=[(2, 2)], rd=[2]),
    dict(x=(1, 2, 5), w=(3, 2, 3), strides=[1], padding=[(2, 1)], ld=[2]),
    dict(x=(1, 2, 6), w=(2, 2, 3), strides=[1], padding=[(-1, 2)], ld=[2]),
    dict(x=(2, 3, 8, 7), w=(5, 3, 3, 3), strides=[1, 1], padding=[(1, 1), (1, 1)]),
    dict(x=(2, 3, 8, 7), w=(5, 3, 3, 2), strides=[2, 1], padding=[(0, 1), (1, 0)]),
    dict(x=(1, 4, 9, 9), w=(2, 4, 3, 3), strides=[2, 2], padding=[(1, 1), (1, 1)], rd=[2, 1]),
    dict(x=(1, 2, 5, 4, 3), w=(2, 2, 2, 2, 2), strides=[1, 1, 1], padding=[(0, 0), (1, 0), (0, 1)]),
    dict(x=(3, 8, 6, 6), w=(16, 8, 1, 1), strides=[1, 1], padding=[(0, 0), (0, 0)]),
    # k = C * kh * kw is not a multiple of the loaders' groups (147, 27, 900): still implicit GEMMs on the GPU
    dict(x=(2, 3, 30, 30), w=(32, 3, 7, 7), strides=[2, 2], padding=[(2, 3), (2, 3)]),
    dict(x=(2, 3, 16, 16), w=(32, 3, 3, 3), strides=[1, 1], padding=[(1, 1), (1, 1)]),
    dict(x=(1, 100, 12, 12), w=(40, 100, 3, 3), strides=[1, 1], padding=[(1, 1), (1, 1)]),
]


def _conv_case(c, backend):
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, c["x"]).astype(np.float32)
    w = rng.integers(-3, 4, c["w"]).astype(np.float32)
    prog, (r,) = run_on(backend, lambda a, b: L.convGeneralDilated(a, b, c["strides"], c["padding"], lhsDilation=c.get("ld"),
                                                                  rhsDilation=c.get("rd")), x, w)
    want = conv_reference(x, w, c["strides"], c["padding"], c.get("ld"), c.get("rd"))
    np.testing.assert_array_equal(r.reshape(want.shape), want)  # small integers: exact in f32
    return prog


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_convolution_matches_direct_loops(case):
    prog = _conv_case(case, OracleBackend())
    lowered = len(case["x"]) == 3 and case.get("ld") and min(case["padding"][0]) >= 0  # 1-D transposed: overlap-add lowering
    if lowered:
        assert sum(1 for k in prog.kernels if k.reduction is not None) == 1 and len(prog.kernels) > 1  # one Dot, then shifts and adds
    else:
        assert len(prog.kernels) == 1  # one reduce kernel over C * prod(ks)


def test_pooling_and_window_reductions():
    x = np.random.default_rng(4).integers(-9, 10, (2, 3, 8, 9)).astype(np.float32)
    _, (r,) = run(lambda a: L.reduceWindow(a, AluOp.Max, [2, 2], [2, 2]), x)
    want = x[:, :, :8, :8].reshape(2, 3, 4, 2, 4, 2).max(axis=(3, 5))
    np.testing.assert_array_equal(r.reshape(want.shape), want)
    _, (r,) = run(lambda a: L.reduceWindow(a, AluOp.Add, [3, 3], [1, 1]).mul(1 / 9), x)
    want = sum(x[:, :, dy:dy + 6, dx:dx + 7] for dy in range(3) for dx in range(3)) / 9
    np.testing.assert_allclose(r.reshape(want.shape), want, rtol=1e-6)
    _, (r,) = run(lambda a: L.reduceWindow(a, AluOp.Min, [3], [2]), x)  # window on the last axis only
    want = np.stack([x[..., 2 * o:2 * o + 3].min(-1) for o in range(4)], -1)
    np.testing.assert_array_equal(r.reshape(want.shape), want)


def test_conv_consumer_materialises_a_computed_operand():
    """An activation feeding a convolution is computed once, not once per output channel (jit.ts:891-950)."""
    x = f32(np.arange(2 * 3 * 6).reshape(2, 3, 6) / 10)
    w = f32(np.ones((4, 3, 3)))
    prog, (r,) = run(lambda a, b: L.convGeneralDilated(J.exp(a), b, [1], "VALID"), x, w)
    assert len(prog.kernels) == 2 and prog.kernels[0].reduction is None
    np.testing.assert_allclose(r.reshape(2, 4, 4), conv_reference(np.exp(x), w, [1], [(0, 0)]), rtol=1e-5)


def test_shape_errors():
    p = ConvParams(0, [1], [(0, 0)], [1], [1])
    with pytest.raises(ValueError):
        checkConvShape([1, 2, 5], [3, 4, 3], p)  # channel mismatch
    with pytest.raises(ValueError):
        checkConvShape([1, 2, 2], [3, 2, 3], p)  # kernel larger than input


# ---- GPU --------------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_convolution_on_gpu(case):
    from gpu_util import WARM_ONLY, backend
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"], lhsDilation=case.get("ld"),
                                                       rhsDilation=case.get("rd")), [ShapedArray(case["x"], F32), ShapedArray(case["w"], F32)])
        for k in prog.kernels:
            for src in generate(k).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    _conv_case(case, backend())


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [DType.Float16, F32], ids=lambda d: d.value)
@pytest.mark.parametrize("case", CONV_CASES[-3:], ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_convolutions_with_a_ragged_k_axis_are_implicit_gemms(case, dt):
    """3 input channels under a 7x7 or 3x3 window, 100 channels under 3x3: C * kh * kw = 147, 27, 900.  The kernel class
    must be the matrix-core one (the gathered operand's loaders check every k) and small integers come out exact."""
    from gpu_util import device_run
    from jaxjs_hip.alu import numpyDtype
    prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"]), [ShapedArray(case["x"], dt), ShapedArray(case["w"], dt)])
    assert len(prog.kernels) == 1
    rng = np.random.default_rng(5)
    x = rng.integers(-2, 3, case["x"]).astype(numpyDtype(dt))
    w = rng.integers(-1, 2, case["w"]).astype(numpyDtype(dt))
    got, ks = device_run(prog.kernels[0], [x, w])
    assert ks.klass.startswith("gemm"), (ks.klass, ks.info)
    want = conv_reference(x.astype(np.float32), w.astype(np.float32), case["strides"], case["padding"], None, None)
    np.testing.assert_array_equal(got.astype(np.float32).reshape(want.shape), want, err_msg=str(ks.info))


@pytest.mark.gpu
def test_resnet_shaped_convolution_and_pooling_on_gpu():
    """3x3 stride-1 'SAME' convolution [8,64,28,28] * [64,64,3,3] in f32 against float64 loops on a sample of the
    outputs (K-scaled bound), and a 2x2 max pool, both on the GPU."""
    from gpu_util import WARM_ONLY, backend
    rng = np.random.default_rng(8)
    x = rng.standard_normal((8, 64, 28, 28)).astype(np.float32)
    w = (rng.standard_normal((64, 64, 3, 3)) * 0.05).astype(np.float32)
    conv_prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, [1, 1], "SAME"), [ShapedArray(x.shape, F32), ShapedArray(w.shape, F32)])
    pool_prog = J.jit(lambda a: L.reduceWindow(a, AluOp.Max, [2, 2], [2, 2]), [ShapedArray(x.shape, F32)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        conv16 = J.jit(lambda a, b: L.convGeneralDilated(a, b, [1, 1], "SAME"),
                       [ShapedArray(x.shape, DType.Float16), ShapedArray(w.shape, DType.Float16)])
        for k in conv_prog.kernels + pool_prog.kernels + conv16.kernels:
            for src in generate(k).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    # The patches operand is a masked three-view tracker: the kernel must take the MFMA class through its
    # element-gather loader, not the generic row reduction.
    assert be.prepareKernelSync(conv_prog.kernels[0]).data.ks.klass.startswith("gemm")
    conv16 = J.jit(lambda a, b: L.convGeneralDilated(a, b, [1, 1], "SAME"),
                   [ShapedArray(x.shape, DType.Float16), ShapedArray(w.shape, DType.Float16)])
    assert be.prepareKernelSync(conv16.kernels[0]).data.ks.klass.startswith("gemm")
    x16, w16 = x.astype(np.float16), w.astype(np.float16)
    (r16,) = run_program(be, conv16, [x16, w16])
    r16 = r16.reshape(8, 64, 28, 28).astype(np.float64)
    xp16 = np.pad(x16.astype(np.float64), [(0, 0), (0, 0), (1, 1), (1, 1)])
    for (n, o, i, j) in rng.integers(0, [8, 64, 28, 28], (200, 4)):
        want = float((xp16[n, :, i:i + 3, j:j + 3] * w16[o].astype(np.float64)).sum())
        assert abs(r16[n, o, i, j] - want) <= 1e-2 * abs(want) + 2e-2
    (r,) = run_program(be, conv_prog, [x, w])
    r = r.reshape(8, 64, 28, 28)
    xp = np.pad(x.astype(np.float64), [(0, 0), (0, 0), (1, 1), (1, 1)])
    for (n, o, i, j) in rng.integers(0, [8, 64, 28, 28], (200, 4)):
        patch = xp[n, :, i:i + 3, j:j + 3]
        want = float((patch * w[o].astype(np.float64)).sum())
        mag = float((np.abs(patch) * np.abs(w[o])).sum())
        assert abs(r[n, o, i, j] - want) <= 2 * 576 * np.finfo(np.float32).eps * mag + 1e-6
    (p,) = run_program(be, pool_prog, [x])
    np.testing.assert_array_equal(p.reshape(8, 64, 14, 14), x.reshape(8, 64, 14, 2, 14, 2).max(axis=(3, 5)))


# f16 convolutions whose image operand is (or is not) eligible for the row-vector gather loader: image widths that are
# a multiple of 8 or of 4 only (shorter vectors), other widths and strides (element loader), padding on every
# side, dilation, one to three spatial dims, ragged pixel counts.
F16_CONV_CASES = [
    dict(x=(2, 8, 16, 16), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="rows8"),
    dict(x=(3, 16, 8, 24), w=(32, 16, 3, 3), strides=[1, 1], padding="SAME", loader="rows8"),
    dict(x=(2, 8, 28, 28), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="rows4"),
    dict(x=(2, 8, 14, 14), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="element"),
    dict(x=(2, 8, 30, 30), w=(32, 8, 3, 3), strides=[1, 1], padding="VALID", loader="rows4"),
    dict(x=(1, 8, 20, 40), w=(32, 8, 5, 5), strides=[1, 1], padding=[(3, 1), (0, 4)], loader="rows8"),
    dict(x=(2, 8, 24, 24), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", rd=[2, 2], loader="rows8"),
    dict(x=(2, 16, 64), w=(32, 16, 3), strides=[1], padding="SAME", loader="rows8"),
    dict(x=(1, 8, 6, 8, 16), w=(32, 8, 3, 3, 3), strides=[1, 1, 1], padding="SAME", loader="rows8"),
    dict(x=(2, 8, 7, 7), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="element"),
    dict(x=(2, 8, 32, 32), w=(32, 8, 3, 3), strides=[2, 2], padding="SAME", loader="element"),
    dict(x=(2, 8, 16, 16), w=(32, 8, 1, 1), strides=[1, 1], padding="VALID", loader=None),
    # stride-1 window walks with at least 16 input and 64 output channels and an output width that is a multiple of 4:
    # the patch-in-LDS convolution template (image rows resident in LDS, one copy per window column)
    dict(x=(2, 16, 16, 16), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(3, 32, 8, 24), w=(64, 32, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(2, 16, 28, 28), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),      # 4-element fill vectors
    dict(x=(2, 16, 30, 30), w=(64, 16, 3, 3), strides=[1, 1], padding="VALID", loader="patch"),     # output narrower than the image
    dict(x=(1, 32, 20, 40), w=(64, 32, 5, 5), strides=[1, 1], padding=[(3, 1), (0, 4)], loader="patch"),
    dict(x=(2, 64, 12, 12), w=(128, 64, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),     # two channel tiles, ragged last position tile
    dict(x=(1, 16, 56, 56), w=(256, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),     # 128-channel tiles
    dict(x=(2, 128, 14, 12), w=(64, 128, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),    # several channel slabs
    dict(x=(2, 16, 64), w=(64, 16, 3), strides=[1], padding="SAME", loader="patch"),                # one spatial dim
    dict(x=(1, 16, 16, 16), w=(64, 16, 7, 7), strides=[1, 1], padding="SAME", loader="patch"),      # shifts of 3: two dwords from each neighbour
    dict(x=(2, 16, 12, 16), w=(64, 16, 1, 3), strides=[1, 1], padding="SAME", loader="patch"),      # one window row
    dict(x=(2, 16, 12, 16), w=(64, 16, 3, 1), strides=[1, 1], padding="SAME", loader="patch"),      # one window column: no shifted copies
    dict(x=(1, 48, 8, 8), w=(64, 48, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),        # three slabs; one fill vector per row
    dict(x=(1, 256, 8, 8), w=(64, 256, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),      # sixteen slabs: the paired loop
    dict(x=(1, 16, 8, 112), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),      # 14 fill vectors per row, 4 rows per wave
    dict(x=(8, 16, 8, 4), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),        # one tile per image, mostly padding
    dict(x=(1, 16, 12, 32), w=(64, 16, 5, 5), strides=[1, 1], padding="SAME", loader="patch"),      # shifts of 2 to either side
    dict(x=(2, 16, 16, 16), w=(32, 16, 3, 3), strides=[1, 1], padding="SAME", loader="rows8"),      # 32 output channels: generic loaders
    # output widths that are not a multiple of 4: rows are walked at the next multiple, the extra columns dropped
    dict(x=(2, 16, 14, 14), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(3, 32, 7, 7), w=(64, 32, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(2, 16, 10, 10), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(2, 16, 15, 15), w=(64, 16, 3, 3), strides=[1, 1], padding="VALID", loader="patch"),
    dict(x=(2, 16, 9, 6), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="patch"),
    dict(x=(2, 16, 9, 5), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="element"),       # overhang of a whole vector: generic loaders
    dict(x=(1, 16, 33, 21), w=(64, 16, 5, 5), strides=[1, 1], padding="SAME", loader="patch"),
    # strided window walks: copies pick every second column, rows live in planes by parity
    dict(x=(2, 16, 32, 32), w=(64, 16, 3, 3), strides=[2, 2], padding="SAME", loader="patch"),
    dict(x=(2, 16, 32, 32), w=(64, 16, 3, 3), strides=[2, 2], padding=[(1, 1), (1, 1)], loader="patch"),  # left and top padding
    dict(x=(2, 16, 16, 32), w=(64, 16, 3, 3), strides=[1, 2], padding="SAME", loader="patch"),
    dict(x=(2, 16, 32, 16), w=(64, 16, 3, 3), strides=[2, 1], padding="SAME", loader="patch"),
    dict(x=(1, 32, 32, 32), w=(64, 32, 5, 5), strides=[2, 2], padding="SAME", loader="patch"),            # a dword from the right neighbour
    dict(x=(3, 32, 56, 56), w=(128, 32, 3, 3), strides=[2, 2], padding="SAME", loader="patch"),           # several position tiles per image
    dict(x=(2, 16, 24, 24), w=(64, 16, 3, 3), strides=[3, 3], padding="SAME", loader="element"),          # other strides: generic loaders
    # strided and not whole vectors: unaligned loads, every second element kept
    dict(x=(2, 16, 33, 32), w=(64, 16, 3, 3), strides=[2, 2], padding="VALID", loader="patch"),
    dict(x=(2, 32, 28, 28), w=(64, 32, 3, 3), strides=[2, 2], padding="SAME", loader="patch"),            # 28 -> 14
    dict(x=(3, 16, 14, 14), w=(128, 16, 3, 3), strides=[2, 2], padding=[(1, 1), (1, 1)], loader="patch"), # 14 -> 7
    dict(x=(2, 16, 20, 12), w=(64, 16, 3, 3), strides=[2, 1], padding="SAME", loader="patch"),
]


def _f16_conv_program(c):
    return J.jit(lambda a, b: L.convGeneralDilated(a, b, c["strides"], c["padding"], rhsDilation=c.get("rd")),
                 [ShapedArray(c["x"], DType.Float16), ShapedArray(c["w"], DType.Float16)])


@pytest.mark.parametrize("case", F16_CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_f16_convolution_loader_choice(case):
    """Which loader the generator picks is decided on the host: check it without a GPU."""
    from jaxjs_hip.kernelgen import generate
    ks = generate(_f16_conv_program(case).kernels[0])
    if case["loader"] is None:
        assert "gather" not in ks.info or set(ks.info["gather"].values()) == {"none"}
    else:
        assert ks.klass.startswith("gemm") and case["loader"] in ks.info["gather"].values(), ks.info
        if case["loader"] == "patch":
            cv = ks.info["conv"]
            assert (cv["KH"] * cv["KW"], cv["C"]) == (int(np.prod(case["w"][2:])), case["w"][1]) and len(ks.steps) == 2
        # the optional tap-major k order (k' = tap * C + c) applies to every one of them
        tm = generate(_f16_conv_program(case).kernels[0], gemm_tile=(("TAPMAJOR", 1),))
        assert tm.info["tap_major"]["T"] == int(np.prod(case["w"][2:])) and any(v.startswith("tap-major rows") for v in tm.info["gather"].values())


# ---- the layer shapes the bench measures, at full size --------------------------------------------------------------

LAYER_CONVS = [((32, 64, 56, 56), (64, 64, 3, 3), 1), ((32, 256, 28, 28), (256, 256, 3, 3), 1), ((32, 256, 14, 14), (256, 256, 3, 3), 1),
               ((32, 64, 56, 56), (128, 64, 3, 3), 2),
               ((1, 64, 256, 256), (128, 64, 3, 3), 1)]  # the reference's conv2d bench (website/src/routes/bench/conv2d/strategies.ts:13-19)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(DType.Float16, np.float16), (DType.Float32, np.float32)], ids=["f16", "f32"])
@pytest.mark.parametrize("cx,cw,st", LAYER_CONVS, ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else f"s{v}")
def test_layer_sized_convolutions_are_exact(cx, cw, st, dt, npdt):
    """3x3 SAME convolutions of ResNet-sized layers (batch 32), stride 1 and 2, with entries in {-1, 0, 1}: every output is
    an integer below 2048, exact in float16 and float32, and must equal a tap-by-tap host convolution everywhere."""
    from gpu_util import WARM_ONLY, backend
    prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, [st, st], "SAME"), [ShapedArray(cx, dt), ShapedArray(cw, dt)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(prog.kernels[0]).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(21)
    x = rng.integers(-1, 2, cx).astype(npdt)
    w = rng.integers(-1, 2, cw).astype(npdt)
    be = backend()
    exe = be.prepareKernelSync(prog.kernels[0])
    assert exe.data.ks.klass.startswith("gemm"), exe.data.ks.klass
    sx, sw, so = be.malloc(x.nbytes, x.tobytes()), be.malloc(w.nbytes, w.tobytes()), be.malloc(prog.kernels[0].bytes)
    be.dispatch(exe, [sx, sw], [so])
    r = np.frombuffer(be.readSync(so), npdt).astype(np.float32)
    for s_ in (sx, sw, so):
        be.decRef(s_)
    (pt, pb), (pl, pr) = L.padtypeToPads(cx[2:], cw[2:], [st, st], [1, 1], "SAME")
    xp = np.pad(x.astype(np.float32), [(0, 0), (0, 0), (pt, pb), (pl, pr)])
    OH, OW = -(-cx[2] // st), -(-cx[3] // st)
    want = np.zeros((cx[0], cw[0], OH, OW), np.float32)
    for ky in range(3):
        for kx in range(3):
            win = xp[:, :, ky:ky + (OH - 1) * st + 1:st, kx:kx + (OW - 1) * st + 1:st]
            want += np.einsum("nchw,oc->nohw", win, w[:, :, ky, kx].astype(np.float32), optimize=True)
    assert np.abs(want).max() < 2048
    np.testing.assert_array_equal(r.reshape(want.shape), want, err_msg=str(exe.data.ks.info))


# float32 convolutions on the gather loaders: stride-1 windows whose output width is a multiple of 4 read four consecutive
# output positions with one 128-bit load (masked lanes zeroed), everything else element by element.
F32_CONV_CASES = [
    dict(x=(2, 8, 16, 16), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="rows4"),
    dict(x=(2, 8, 30, 30), w=(32, 8, 3, 3), strides=[1, 1], padding="VALID", loader="rows4"),
    dict(x=(1, 8, 20, 40), w=(32, 8, 5, 5), strides=[1, 1], padding=[(3, 1), (0, 4)], loader="rows4"),
    dict(x=(2, 8, 24, 24), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", rd=[2, 2], loader="rows4"),
    dict(x=(2, 16, 64), w=(32, 16, 3), strides=[1], padding="SAME", loader="rows4"),
    dict(x=(2, 8, 14, 14), w=(32, 8, 3, 3), strides=[1, 1], padding="SAME", loader="element"),
    dict(x=(2, 8, 32, 32), w=(32, 8, 3, 3), strides=[2, 2], padding="SAME", loader="element"),
    dict(x=(4, 16, 28, 28), w=(64, 16, 3, 3), strides=[1, 1], padding="SAME", loader="rows4"),
]


def _f32_conv_program(c):
    return J.jit(lambda a, b: L.convGeneralDilated(a, b, c["strides"], c["padding"], rhsDilation=c.get("rd")),
                 [ShapedArray(c["x"], DType.Float32), ShapedArray(c["w"], DType.Float32)])


@pytest.mark.parametrize("case", F32_CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_f32_convolution_loader_choice(case):
    from jaxjs_hip.kernelgen import generate
    ks = generate(_f32_conv_program(case).kernels[0])
    assert ks.klass.startswith("gemm") and case["loader"] in ks.info["gather"].values(), ks.info


@pytest.mark.gpu
@pytest.mark.parametrize("case", F32_CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_f32_convolution_on_gpu_is_exact_on_small_integers(case):
    from gpu_util import WARM_ONLY, backend
    prog = _f32_conv_program(case)
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(prog.kernels[0]).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(13)
    x = rng.integers(-2, 3, case["x"]).astype(np.float32)
    w = rng.integers(-2, 3, case["w"]).astype(np.float32)
    be = backend()
    exe = be.prepareKernelSync(prog.kernels[0])
    sx, sw, so = be.malloc(x.nbytes, x.tobytes()), be.malloc(w.nbytes, w.tobytes()), be.malloc(prog.kernels[0].bytes)
    be.dispatch(exe, [sx, sw], [so])
    r = np.frombuffer(be.readSync(so), np.float32).copy()
    for s_ in (sx, sw, so):
        be.decRef(s_)
    pads = case["padding"]
    if isinstance(pads, str):
        pads = L.padtypeToPads(case["x"][2:], case["w"][2:], case["strides"], case.get("rd") or [1] * len(case["strides"]), pads)
    want = conv_reference(x, w, case["strides"], pads, None, case.get("rd"))
    np.testing.assert_array_equal(r.reshape(want.shape).astype(np.float64), want)


@pytest.mark.gpu
@pytest.mark.parametrize("tap_major", [0, 1], ids=["k-order", "tap-major"])
@pytest.mark.parametrize("case", F16_CONV_CASES, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_f16_convolution_on_gpu_is_exact_on_small_integers(case, tap_major):
    from gpu_util import WARM_ONLY, backend
    prog = _f16_conv_program(case)
    opts = dict(gemm_tile=(("TAPMAJOR", 1),)) if tap_major else {}
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(prog.kernels[0], **opts).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(12)
    x = rng.integers(-2, 3, case["x"]).astype(np.float16)
    w = rng.integers(-2, 3, case["w"]).astype(np.float16)
    be = backend()
    exe = be.prepareKernelSync(prog.kernels[0], **opts)
    sx, sw, so = be.malloc(x.nbytes, x.tobytes()), be.malloc(w.nbytes, w.tobytes()), be.malloc(prog.kernels[0].bytes)
    be.dispatch(exe, [sx, sw], [so])
    r = np.frombuffer(be.readSync(so), np.float16).copy()
    for s_ in (sx, sw, so):
        be.decRef(s_)
    pads = case["padding"]
    if isinstance(pads, str):
        pads = L.padtypeToPads(case["x"][2:], case["w"][2:], case["strides"], case.get("rd") or [1] * len(case["strides"]), pads)
    want = conv_reference(x.astype(np.float32), w.astype(np.float32), case["strides"], pads, None, case.get("rd"))
    np.testing.assert_array_equal(r.reshape(want.shape).astype(np.float64), want)  # |sums| < 2048: exact in f16


# First layers of small CNNs: one (or three) input channels, a handful of taps per output, millions of outputs.  Too few
# k for the matrix cores; the fold is short and its only stream along the reduce axis is the filter, so one lane per output
# walks the taps (column class, unrolled whole) instead of a few lanes sharing each output's taps.
FIRST_LAYER_CONVS = [
    dict(x=(128, 1, 28, 28), w=(32, 1, 3, 3), strides=[1, 1], padding="VALID"),
    dict(x=(256, 1, 28, 28), w=(8, 1, 5, 5), strides=[1, 1], padding="SAME"),
    dict(x=(64, 1, 28, 28), w=(16, 1, 3, 3), strides=[2, 2], padding="SAME"),
    dict(x=(96, 2, 20, 24), w=(24, 2, 3, 3), strides=[1, 1], padding="SAME", rd=[2, 2]),
]


@pytest.mark.parametrize("case", FIRST_LAYER_CONVS, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_first_layer_convolutions_take_one_lane_per_output(case):
    from jaxjs_hip.kernelgen import generate
    for dt in (F32, DType.Float16):
        prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"], rhsDilation=case.get("rd")),
                     [ShapedArray(case["x"], dt), ShapedArray(case["w"], dt)])
        ks = generate(prog.kernels[0])
        assert ks.klass == "reduce_col" and ks.info["T"] == 1 and ks.info["split"] == 1, (ks.klass, ks.info)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(DType.Float16, np.float16), (DType.Float32, np.float32)], ids=["f16", "f32"])
@pytest.mark.parametrize("case", FIRST_LAYER_CONVS, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_first_layer_convolutions_on_gpu_are_exact_on_small_integers(case, dt, npdt):
    from gpu_util import WARM_ONLY, backend
    prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"], rhsDilation=case.get("rd")),
                 [ShapedArray(case["x"], dt), ShapedArray(case["w"], dt)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(prog.kernels[0]).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(17)
    x = rng.integers(-2, 3, case["x"]).astype(npdt)
    w = rng.integers(-2, 3, case["w"]).astype(npdt)
    be = backend()
    exe = be.prepareKernelSync(prog.kernels[0])
    sx, sw, so = be.malloc(x.nbytes, x.tobytes()), be.malloc(w.nbytes, w.tobytes()), be.malloc(prog.kernels[0].bytes)
    be.dispatch(exe, [sx, sw], [so])
    r = np.frombuffer(be.readSync(so), npdt).copy()
    for s_ in (sx, sw, so):
        be.decRef(s_)
    pads = case["padding"]
    if isinstance(pads, str):
        pads = L.padtypeToPads(case["x"][2:], case["w"][2:], case["strides"], case.get("rd") or [1] * len(case["strides"]), pads)
    want = conv_reference(x.astype(np.float32), w.astype(np.float32), case["strides"], pads, None, case.get("rd"))
    np.testing.assert_array_equal(r.reshape(want.shape).astype(np.float64), want, err_msg=str(exe.data.ks.info))


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(DType.Float16, np.float16), (DType.Float32, np.float32)], ids=["f16", "f32"])
@pytest.mark.parametrize("cx,cw,groups", [((8, 64, 56, 56), (64, 8, 3, 3), 8), ((4, 32, 40, 40), (32, 1, 3, 3), 32), ((2, 16, 64, 64), (16, 4, 5, 5), 4)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else f"g{v}")
def test_grouped_and_depthwise_convolutions_on_gpu_are_exact_on_small_integers(cx, cw, groups, dt, npdt):
    """Feature groups (lax.ts:252-343): a leading batch axis of the Conv primitive, k = C/G x taps per output -- too few rows
    per group for the matrix cores.  One lane per output, the fold of up to 256 steps unrolled whole; checked group by group
    against the host convolution."""
    from gpu_util import WARM_ONLY, backend
    from jit_util import run_program
    prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, [1, 1], "SAME", featureGroupCount=groups), [ShapedArray(cx, dt), ShapedArray(cw, dt)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for k in prog.kernels:
            for src in generate(k).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(19)
    x = rng.integers(-2, 3, cx).astype(npdt)
    w = rng.integers(-2, 3, cw).astype(npdt)
    (got,) = run_program(backend(), prog, [x, w])
    pads = L.padtypeToPads(cx[2:], cw[2:], [1, 1], [1, 1], "SAME")
    cg, og = cx[1] // groups, cw[0] // groups
    want = np.concatenate([conv_reference(x[:, g * cg:(g + 1) * cg].astype(np.float32), w[g * og:(g + 1) * og].astype(np.float32), [1, 1], pads)
                           for g in range(groups)], axis=1)
    np.testing.assert_array_equal(np.asarray(got).reshape(want.shape).astype(np.float64), want)


# Convolutions of audio models: a few hundred channels against one long row of a few thousand positions.
LONG_ROW_CONVS = [
    dict(x=(1, 80, 3000), w=(384, 80, 3), strides=[1], padding="SAME"),
    dict(x=(1, 384, 3000), w=(384, 384, 3), strides=[2], padding="SAME"),
    dict(x=(1, 512, 1500), w=(512, 512, 3), strides=[1], padding="SAME"),
]


def test_long_row_convolutions_keep_off_the_patch_template_and_cover_the_chip():
    """The patch-in-LDS template holds whole image rows, so a row several times as wide as its tile would be filled again by
    every tile along it ([1,384,3000] stride 2 took 500 us that way); such shapes run on the gather loaders, in tiles small
    enough that the launch has at least half as many workgroups as the chip has CUs."""
    from jaxjs_hip.kernelgen import generate
    from jaxjs_hip import tuner
    for case in LONG_ROW_CONVS:
        prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"]),
                     [ShapedArray(case["x"], DType.Float16), ShapedArray(case["w"], DType.Float16)])
        ks = generate(prog.kernels[0])
        assert ks.klass == "gemm" and ks.info["gather"]["b"] != "patch" and ks.info["tiles"] * 2 >= tuner.CU_COUNT, ks.info


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(DType.Float16, np.float16), (DType.Float32, np.float32)], ids=["f16", "f32"])
@pytest.mark.parametrize("case", LONG_ROW_CONVS, ids=lambda c: "x".join(map(str, c["x"])) + "*" + "x".join(map(str, c["w"])))
def test_long_row_convolutions_on_gpu_are_exact_on_small_integers(case, dt, npdt):
    from gpu_util import WARM_ONLY, backend
    prog = J.jit(lambda a, b: L.convGeneralDilated(a, b, case["strides"], case["padding"]), [ShapedArray(case["x"], dt), ShapedArray(case["w"], dt)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for src in generate(prog.kernels[0]).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    rng = np.random.default_rng(23)
    x = rng.integers(-1, 2, case["x"]).astype(npdt)
    w = rng.integers(-1, 2, case["w"]).astype(npdt)
    be = backend()
    exe = be.prepareKernelSync(prog.kernels[0])
    sx, sw, so = be.malloc(x.nbytes, x.tobytes()), be.malloc(w.nbytes, w.tobytes()), be.malloc(prog.kernels[0].bytes)
    be.dispatch(exe, [sx, sw], [so])
    r = np.frombuffer(be.readSync(so), npdt).copy()
    for s_ in (sx, sw, so):
        be.decRef(s_)
    pads = L.padtypeToPads(case["x"][2:], case["w"][2:], case["strides"], [1], case["padding"])
    want = conv_reference(x.astype(np.float32), w.astype(np.float32), case["strides"], pads)
    assert np.abs(want).max() < 2048
    np.testing.assert_array_equal(r.reshape(want.shape).astype(np.float64), want, err_msg=str(exe.data.ks.info))
