"""Kernels that only the reference's transforms hand to a backend, built by hand (no autodiff here).

`grad`, `jvp` and `vmap` live above the Backend interface, but what they bind reaches `dispatch` as Kernels that no
forward library call produces:

* `Primitive.PoolTranspose` -- the transpose rule of `Pool` (src/frontend/linearize.ts:755-762), lowered by
  src/frontend/jit.ts:623-638 through `poolTranspose` (src/frontend/convolution.ts:274-378);
* the two convolutions the transpose rule of `Conv` binds (src/frontend/linearize.ts:775-838): towards the activations
  (flipped, channel-swapped filter; strides and input dilation trade places) and towards the filter (batch and channel
  axes swapped on both operands; strides and filter dilation trade places);
* `transposeDot`'s contractions over the other operand's axes (src/frontend/linearize.ts:767-774);
* the `Scatter` add that transposes `Gather` (src/frontend/linearize.ts:868-882).

The functions below bind exactly what those rules bind, with the parameters their formulas give; expected values are
the reference's own tables (test/conv.test.ts:271-300, 341-354, 407-455; src/frontend/convolution.test.ts:22-58) and
brute-force adjoints in numpy.  CPU tests run on the checker, the `gpu` ones on the device against both."""
import itertools

import numpy as np
import pytest

from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker
from jaxjs_hip import jit as J
from jaxjs_hip import library as L
from jaxjs_hip.convolution import ConvParams, pool, poolTranspose
from jaxjs_hip.jit import ShapedArray
from jit_util import run_program
from oracle.backend import OracleBackend

F32, F16 = DType.Float32, DType.Float16


# ---- what the transpose rules bind -----------------------------------------------------------------------------------

# (restated in the package beside the other primitives that only transforms bind: src/frontend/linearize.ts:783-837)
conv_transposed_to_lhs = J.convTransposeLhs
conv_transposed_to_rhs = J.convTransposeRhs


# ---- numpy references ------------------------------------------------------------------------------------------------

def conv_forward(x, w, strides, padding, lhs_dil, rhs_dil):
    """Direct loops: x [N, C, *xs], w [O, C, *ks] -> [N, O, *ys] in float64."""
    n = x.ndim - 2
    xs = [(d - 1) * ld + 1 for d, ld in zip(x.shape[2:], lhs_dil)]
    xd = np.zeros(x.shape[:2] + tuple(xs))
    xd[(slice(None), slice(None)) + tuple(slice(None, None, ld) for ld in lhs_dil)] = x
    lo = [max(pl, 0) for pl, _ in padding]
    hi = [max(pr, 0) for _, pr in padding]
    xd = np.pad(xd, [(0, 0), (0, 0)] + list(zip(lo, hi)))
    xd = xd[(slice(None), slice(None)) + tuple(slice(max(-pl, 0), xd.shape[2 + i] - max(-pr, 0)) for i, (pl, pr) in enumerate(padding))]
    ks = w.shape[2:]
    ys = [-(-(xd.shape[2 + i] - ((ks[i] - 1) * rhs_dil[i] + 1) + 1) // strides[i]) for i in range(n)]
    out = np.zeros((x.shape[0], w.shape[0]) + tuple(ys))
    for o in itertools.product(*[range(y) for y in ys]):
        for k in itertools.product(*[range(kk) for kk in ks]):
            pos = tuple(o[i] * strides[i] + k[i] * rhs_dil[i] for i in range(n))
            out[(slice(None), slice(None)) + o] += np.einsum("nc,oc->no", xd[(slice(None), slice(None)) + pos], w[(slice(None), slice(None)) + k])
    return out


def conv_vjp_numeric(x, w, ct, strides, padding, lhs_dil, rhs_dil):
    """Exact adjoints of the (bilinear) convolution by probing: d<ct, conv(x, w)>/dx and /dw."""
    dx, dw = np.zeros(x.shape), np.zeros(w.shape)
    for idx in np.ndindex(*x.shape):
        e = np.zeros(x.shape)
        e[idx] = 1.0
        dx[idx] = np.sum(ct * conv_forward(e, w, strides, padding, lhs_dil, rhs_dil))
    for idx in np.ndindex(*w.shape):
        e = np.zeros(w.shape)
        e[idx] = 1.0
        dw[idx] = np.sum(ct * conv_forward(x, e, strides, padding, lhs_dil, rhs_dil))
    return dx, dw


def pool_transpose_numpy(g, in_shape, window, strides):
    """g [..., *out, *window] scattered back onto in_shape: position o*s + k receives g[o, k]."""
    nk = len(window)
    out = np.zeros(in_shape)
    o_shape = g.shape[-2 * nk:-nk]
    for o in itertools.product(*[range(d) for d in o_shape]):
        for k in itertools.product(*[range(d) for d in window]):
            pos = tuple(oo * s + kk for oo, s, kk in zip(o, strides, k))
            out[(Ellipsis,) + pos] += g[(Ellipsis,) + o + k]
    return out


def on_checker(fn, arrays, dtype=F32):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), dtype) for a in arrays])
    be = OracleBackend()
    outs = run_program(be, prog, arrays)
    assert be.live_slots() == 0
    return prog, outs


def f32(x):
    return np.asarray(x, dtype=np.float32)


# ---- CPU: view algebra and the reference's tables --------------------------------------------------------------------

def test_pool_transpose_view_returns_every_pooled_element_to_its_origin():
    """src/frontend/convolution.test.ts:22-58: pool [7, 12] with window [2, 2], strides [1, 2]; the transposed view has
    shape [7, 12, 3, 5] and wherever it is valid it addresses the pooled element that was read from that input position."""
    from jaxjs_hip.alu import AluVar  # noqa: F401
    st = ShapeTracker.fromShape([7, 12])
    pooled = pool(st, [2, 2], [1, 2])
    assert list(pooled.shape) == [6, 6, 2, 2]
    unpooled = poolTranspose(pooled, [7, 12], [2, 2], [1, 2])
    assert list(unpooled.shape) == [7, 12, 3, 5]
    vars_ = [AluExp.variable(DType.Int32, f"i{i}") for i in range(4)]
    iexpr, vexpr = unpooled.toAluExp(vars_)
    hits = 0
    for i, j, a, b in itertools.product(range(7), range(12), range(3), range(5)):
        env = {"i0": i, "i1": j, "i2": a, "i3": b}
        if vexpr.evaluate(env):
            assert iexpr.evaluate(env) == i * 12 + j
            hits += 1
    assert hits == 6 * 6 * 2 * 2  # every pooled element is returned exactly once


@pytest.mark.parametrize("in_shape,window,strides", [
    ([2, 4], [2, 2], [2, 2]),        # non-overlapping windows (the k <= s form)
    ([7, 12], [2, 2], [1, 2]),       # mixed
    ([3, 9], [3], [1]),              # overlapping windows along one axis
    ([2, 3, 10, 11], [3, 4], [2, 3]),  # overlap, strides > 1, leading axes
    ([5, 8], [2, 3], [3, 4]),        # windows smaller than the stride: some inputs receive nothing
])
def test_pool_transpose_kernel_is_the_adjoint_of_pool(in_shape, window, strides):
    rng = np.random.default_rng(4)
    from jaxjs_hip.convolution import checkPoolShape
    g = rng.integers(-4, 5, checkPoolShape(in_shape, window, strides)).astype(np.float32)
    prog, (y,) = on_checker(lambda ct: J.poolTransposeWindows(ct, in_shape, window, strides), [g])
    assert len(prog.kernels) == 1 and prog.kernels[0].reduction is not None and prog.kernels[0].reduction.op == AluOp.Add
    want = pool_transpose_numpy(g.astype(np.float64), in_shape, window, strides)
    np.testing.assert_array_equal(y.reshape(in_shape), want.astype(np.float32))
    # <pool(x), g> == <x, poolTranspose(g)>
    x = rng.integers(-3, 4, in_shape).astype(np.float32)
    _, (px,) = on_checker(lambda a: J.poolWindows(a, window, strides), [x])
    assert float(np.sum(px.astype(np.float64) * g.ravel())) == float(np.sum(x.astype(np.float64) * want))


def test_grad_of_max_pool_table():
    """test/conv.test.ts:341-354: d/dx sum(maxpool 2x2 / 2) of [[1,5,3,4],[1,2,3,4]] = [[0,1,0,.5],[0,0,0,.5]].  The
    transform's chain: pool view, compare with the window maximum, divide by the number of maxima, PoolTranspose."""
    x = f32([[1, 5, 3, 4], [1, 2, 3, 4]])

    def fn(a):
        w = J.poolWindows(a, [2, 2], [2, 2])                      # [1, 2, 2, 2]
        m = J.reduce(w, AluOp.Max, [2, 3], keepdims=True)
        hit = J.where(J.equal(w, J.broadcast(m.reshape([1, 2]), [1, 2, 2, 2], [2, 3])), 1.0, 0.0)
        cnt = J.reduce(hit, AluOp.Add, [2, 3])
        ct = hit.mul(J.reciprocal(J.broadcast(cnt, [1, 2, 2, 2], [2, 3])))
        return J.poolTransposeWindows(ct, [2, 4], [2, 2], [2, 2])
    _, (dx,) = on_checker(fn, [x])
    np.testing.assert_array_equal(dx.reshape(2, 4), f32([[0, 1, 0, 0.5], [0, 0, 0, 0.5]]))


def test_grad_of_0d_convolution_table():
    """test/conv.test.ts:271-288: x [3, 2], y [2, 2], cotangent of ones: dx = [[9, 6]] * 3."""
    y = f32([[6, 4], [3, 2]])
    p = ConvParams(0, [], [], [], [])
    _, (dx,) = on_checker(lambda ct, w: conv_transposed_to_lhs(ct, w, [3, 2], p), [np.ones((3, 2), np.float32), y])
    np.testing.assert_array_equal(dx.reshape(3, 2), f32([[9, 6]] * 3))


def test_grad_of_1d_convolution_tables():
    """test/conv.test.ts:290-300: f = conv(x, y, SAME)[0, 0, 3]; dx = [0,0,2,.5,-1,0,0], dy = [3,4,5]."""
    x = f32([[[1, 2, 3, 4, 5, 6, 7]]])
    y = f32([[[2, 0.5, -1]]])
    ct = np.zeros((1, 1, 7), np.float32)
    ct[0, 0, 3] = 1
    p = ConvParams(0, [1], [(1, 1)], [1], [1])
    _, (dx,) = on_checker(lambda c, w: conv_transposed_to_lhs(c, w, [1, 1, 7], p), [ct, y])
    np.testing.assert_array_equal(dx, f32([0, 0, 2, 0.5, -1, 0, 0]))
    _, (dy,) = on_checker(lambda a, c: conv_transposed_to_rhs(a, c, [1, 1, 3], p), [x, ct])
    np.testing.assert_array_equal(dy, f32([3, 4, 5]))


def test_grad_of_depthwise_conv1d_table():
    """test/conv.test.ts:407-455: three groups of one channel; the filter's cotangent under a cotangent of ones is the sum
    of each channel's windows: [[10, 14]], [[14, 18]], [[18, 22]].  The groups are a leading batch axis of the primitive
    (vmapDims = 1), which both transposed convolutions keep in front."""
    x = f32([[[1, 2, 3, 4, 5]], [[2, 3, 4, 5, 6]], [[3, 4, 5, 6, 7]]]).reshape(3, 1, 1, 5)   # [G, N, C/G, W]
    p = ConvParams(1, [1], [(0, 0)], [1], [1])
    ct = np.ones((3, 1, 1, 4), np.float32)                                                   # [G, N, O/G, W']
    _, (dy,) = on_checker(lambda a, c: conv_transposed_to_rhs(a, c, [3, 1, 1, 2], p), [x, ct])
    np.testing.assert_array_equal(dy.reshape(3, 1, 2), f32([[[10, 14]], [[14, 18]], [[18, 22]]]))
    y = f32([[[1, -1]], [[1, 0]], [[0, 1]]]).reshape(3, 1, 1, 2)
    _, (dx,) = on_checker(lambda c, w: conv_transposed_to_lhs(c, w, [3, 1, 1, 5], p), [ct, y])
    np.testing.assert_array_equal(dx.reshape(3, 5), f32([[1, 0, 0, 0, -1], [1, 1, 1, 1, 0], [0, 1, 1, 1, 1]]))


STRIDED = [(x, k) for x in (1, 3, 8, 12, 15) for k in (1, 3, 4) if x >= k]


@pytest.mark.parametrize("xdim,kdim", STRIDED)
def test_grad_shapes_with_stride_2(xdim, kdim):
    """test/conv.test.ts:302-319: 2-d VALID convolution with stride 2 on [3, 1, x, x] and [1, 1, k, k]: both cotangents
    have their operand's shape -- and, beyond the reference's shape check, the values of the exact adjoints."""
    rng = np.random.default_rng(xdim * 10 + kdim)
    x = rng.integers(-3, 4, (3, 1, xdim, xdim)).astype(np.float32)
    w = rng.integers(-3, 4, (1, 1, kdim, kdim)).astype(np.float32)
    p = ConvParams(0, [2, 2], [(0, 0), (0, 0)], [1, 1], [1, 1])
    out = conv_forward(x.astype(np.float64), w.astype(np.float64), [2, 2], p.padding, [1, 1], [1, 1])
    ct = rng.integers(-2, 3, out.shape).astype(np.float32)
    dx_want, dw_want = conv_vjp_numeric(x.astype(np.float64), w.astype(np.float64), ct.astype(np.float64), [2, 2], p.padding, [1, 1], [1, 1])
    _, (dx,) = on_checker(lambda c, f: conv_transposed_to_lhs(c, f, list(x.shape), p), [ct, w])
    _, (dw,) = on_checker(lambda a, c: conv_transposed_to_rhs(a, c, list(w.shape), p), [x, ct])
    np.testing.assert_array_equal(dx.reshape(x.shape), dx_want.astype(np.float32))
    np.testing.assert_array_equal(dw.reshape(w.shape), dw_want.astype(np.float32))


# ---- GPU ---------------------------------------------------------------------------------------------------------------

def on_gpu(fn, arrays, dtype=F32):
    from gpu_util import WARM_ONLY, backend
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), dtype) for a in arrays])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.routinegen import generateRoutine
        from jaxjs_hip.runtime import compile_source
        for k in prog.kernels + [c.kernel() for c in prog.consts]:
            for src in generate(k).sources:
                compile_source(src)
        for r in prog.routines:
            for src in generateRoutine(r).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    outs = run_program(be, prog, arrays)
    classes = [be.prepareKernelSync(k).data.ks.klass for k in prog.kernels]
    return prog, outs, classes


@pytest.mark.gpu
@pytest.mark.parametrize("in_shape,window,strides", [
    ([2, 4], [2, 2], [2, 2]), ([7, 12], [2, 2], [1, 2]), ([2, 3, 10, 11], [3, 4], [2, 3]), ([5, 8], [2, 3], [3, 4]),
    ([8, 16, 56, 56], [3, 3], [2, 2]),   # the cotangent of a 3x3 / 2 max pool over a ResNet-sized activation
    ([4, 32, 28, 28], [2, 2], [2, 2]),
])
def test_pool_transpose_kernels_on_the_gpu(in_shape, window, strides):
    from jaxjs_hip.convolution import checkPoolShape
    rng = np.random.default_rng(5)
    g = rng.integers(-4, 5, checkPoolShape(in_shape, window, strides)).astype(np.float32)
    fn = lambda ct: J.poolTransposeWindows(ct, in_shape, window, strides)  # noqa: E731
    prog, (y,), classes = on_gpu(fn, [g])
    assert len(prog.kernels) == 1
    if np.prod(in_shape) <= 4096:
        _, (want,) = on_checker(fn, [g])
        np.testing.assert_array_equal(y, want)
    np.testing.assert_array_equal(y.reshape(in_shape), pool_transpose_numpy(g.astype(np.float64), in_shape, window, strides).astype(np.float32))


@pytest.mark.gpu
def test_reference_grad_tables_on_the_gpu():
    """The tables of the CPU tests above (max-pool, 0-d, 1-d and depthwise convolution cotangents) on the device."""
    x = f32([[1, 5, 3, 4], [1, 2, 3, 4]])

    def maxpool(a):
        w = J.poolWindows(a, [2, 2], [2, 2])
        m = J.reduce(w, AluOp.Max, [2, 3], keepdims=True)
        hit = J.where(J.equal(w, J.broadcast(m.reshape([1, 2]), [1, 2, 2, 2], [2, 3])), 1.0, 0.0)
        cnt = J.reduce(hit, AluOp.Add, [2, 3])
        return J.poolTransposeWindows(hit.mul(J.reciprocal(J.broadcast(cnt, [1, 2, 2, 2], [2, 3]))), [2, 4], [2, 2], [2, 2])
    _, (dx,), _ = on_gpu(maxpool, [x])
    np.testing.assert_array_equal(dx.reshape(2, 4), f32([[0, 1, 0, 0.5], [0, 0, 0, 0.5]]))
    p0 = ConvParams(0, [], [], [], [])
    _, (dx,), _ = on_gpu(lambda ct, w: conv_transposed_to_lhs(ct, w, [3, 2], p0), [np.ones((3, 2), np.float32), f32([[6, 4], [3, 2]])])
    np.testing.assert_array_equal(dx.reshape(3, 2), f32([[9, 6]] * 3))
    ct = np.zeros((1, 1, 7), np.float32)
    ct[0, 0, 3] = 1
    p1 = ConvParams(0, [1], [(1, 1)], [1], [1])
    _, (dx,), _ = on_gpu(lambda c, w: conv_transposed_to_lhs(c, w, [1, 1, 7], p1), [ct, f32([[[2, 0.5, -1]]])])
    np.testing.assert_array_equal(dx, f32([0, 0, 2, 0.5, -1, 0, 0]))
    _, (dy,), _ = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, [1, 1, 3], p1), [f32([[[1, 2, 3, 4, 5, 6, 7]]]), ct])
    np.testing.assert_array_equal(dy, f32([3, 4, 5]))
    xg = f32([[[1, 2, 3, 4, 5]], [[2, 3, 4, 5, 6]], [[3, 4, 5, 6, 7]]]).reshape(3, 1, 1, 5)
    pg = ConvParams(1, [1], [(0, 0)], [1], [1])
    _, (dy,), _ = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, [3, 1, 1, 2], pg), [xg, np.ones((3, 1, 1, 4), np.float32)])
    np.testing.assert_array_equal(dy.reshape(3, 1, 2), f32([[[10, 14]], [[14, 18]], [[18, 22]]]))


@pytest.mark.gpu
@pytest.mark.parametrize("xdim,kdim", [(3, 3), (8, 3), (12, 4), (15, 1), (15, 4)])
def test_strided_convolution_cotangents_on_the_gpu(xdim, kdim):
    rng = np.random.default_rng(xdim * 10 + kdim)
    x = rng.integers(-3, 4, (3, 1, xdim, xdim)).astype(np.float32)
    w = rng.integers(-3, 4, (1, 1, kdim, kdim)).astype(np.float32)
    p = ConvParams(0, [2, 2], [(0, 0), (0, 0)], [1, 1], [1, 1])
    out = conv_forward(x.astype(np.float64), w.astype(np.float64), [2, 2], p.padding, [1, 1], [1, 1])
    ct = rng.integers(-2, 3, out.shape).astype(np.float32)
    dx_want, dw_want = conv_vjp_numeric(x.astype(np.float64), w.astype(np.float64), ct.astype(np.float64), [2, 2], p.padding, [1, 1], [1, 1])
    _, (dx,), _ = on_gpu(lambda c, f: conv_transposed_to_lhs(c, f, list(x.shape), p), [ct, w])
    _, (dw,), _ = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, list(w.shape), p), [x, ct])
    np.testing.assert_array_equal(dx.reshape(x.shape), dx_want.astype(np.float32))
    np.testing.assert_array_equal(dw.reshape(w.shape), dw_want.astype(np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(F32, np.float32), (F16, np.float16)])
def test_layer_sized_convolution_cotangents_run_on_the_matrix_cores(dt, npdt):
    """A 3x3 SAME convolution layer [8, 32, 28, 28] . [64, 32, 3, 3]: both cotangent Kernels are recognised as implicit
    GEMMs (the activations' one gathers the cotangent through the flipped filter; the filter's one contracts over batch
    and positions), and small-integer data makes every sum exact, so the results equal the einsum adjoints bit for bit."""
    rng = np.random.default_rng(12)
    N, C, O, H = 8, 32, 64, 28
    x = rng.integers(-2, 3, (N, C, H, H)).astype(npdt)
    w = rng.integers(-1, 2, (O, C, 3, 3)).astype(npdt)
    ct = rng.integers(-1, 2, (N, O, H, H)).astype(npdt)
    p = ConvParams(0, [1, 1], [(1, 1), (1, 1)], [1, 1], [1, 1])
    _, (dx,), cls_x = on_gpu(lambda c, f: conv_transposed_to_lhs(c, f, [N, C, H, H], p), [ct, w], dt)
    _, (dw,), cls_w = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, [O, C, 3, 3], p), [x, ct], dt)
    xp = np.pad(x.astype(np.float64), [(0, 0), (0, 0), (1, 1), (1, 1)])
    cp = np.pad(ct.astype(np.float64), [(0, 0), (0, 0), (1, 1), (1, 1)])
    dx_want = np.zeros((N, C, H, H))
    dw_want = np.zeros((O, C, 3, 3))
    for ky in range(3):
        for kx in range(3):
            dw_want[:, :, ky, kx] = np.einsum("nchw,nohw->oc", xp[:, :, ky:ky + H, kx:kx + H], ct.astype(np.float64))
            dx_want += np.einsum("nohw,oc->nchw", cp[:, :, 2 - ky:2 - ky + H, 2 - kx:2 - kx + H], w[:, :, ky, kx].astype(np.float64))
    assert np.abs(dx_want).max() < 2048 and (dt == F32 or np.abs(dw_want).max() < 2048 * 16)
    np.testing.assert_array_equal(dx.astype(np.float64).reshape(dx_want.shape), dx_want)
    if dt == F32:
        np.testing.assert_array_equal(dw.astype(np.float64).reshape(dw_want.shape), dw_want)
    else:  # sums of 6272 terms leave the float16 integer range: one rounding of the exact float32 sum
        np.testing.assert_array_equal(dw.reshape(dw_want.shape), dw_want.astype(np.float16))
    assert any(c.startswith("gemm") for c in cls_x) and any(c.startswith("gemm") for c in cls_w), (cls_x, cls_w)


def conv_vjp_by_taps(x, w, ct, strides, padding, rhs_dil):
    """Adjoints of y[n,o,oy,ox] = sum x[n,c,oy*s+ky*d-p, ox*s+kx*d-p] w[o,c,ky,kx] (2-d, no input dilation), one filter tap
    at a time in float64: dx gets ct x w scattered back, dw gets x windows contracted with ct."""
    N, C, H, W = x.shape
    O, _, KH, KW = w.shape
    (sy, sx), (dy, dx_) = strides, rhs_dil
    (pt, pb), (pl, pr) = padding
    xp = np.pad(x.astype(np.float64), [(0, 0), (0, 0), (pt, pb), (pl, pr)])
    OH, OW = ct.shape[2:]
    gx = np.zeros_like(xp)
    gw = np.zeros(w.shape)
    c64, w64 = ct.astype(np.float64), w.astype(np.float64)
    for ky in range(KH):
        for kx in range(KW):
            ys = slice(ky * dy, ky * dy + (OH - 1) * sy + 1, sy)
            xs = slice(kx * dx_, kx * dx_ + (OW - 1) * sx + 1, sx)
            gw[:, :, ky, kx] = np.einsum("nchw,nohw->oc", xp[:, :, ys, xs], c64)
            gx[:, :, ys, xs] += np.einsum("nohw,oc->nchw", c64, w64[:, :, ky, kx])
    return gx[:, :, pt:pt + H, pl:pl + W], gw


RANDOM_CONVS = [
    # N, C, O, H, W, KH, KW, strides, padding, filter dilation
    (4, 32, 32, 12, 12, 3, 3, (1, 1), ((1, 1), (1, 1)), (1, 1)),
    (2, 32, 64, 16, 14, 3, 3, (2, 2), ((1, 1), (1, 1)), (1, 1)),
    (3, 48, 32, 13, 15, 3, 2, (1, 2), ((0, 0), (1, 0)), (1, 1)),
    (2, 32, 32, 17, 17, 3, 3, (1, 1), ((2, 2), (2, 2)), (2, 2)),
    (2, 64, 32, 9, 20, 1, 5, (1, 1), ((0, 0), (2, 2)), (1, 1)),
    (1, 32, 96, 20, 20, 5, 5, (2, 2), ((2, 2), (2, 2)), (1, 1)),
    (5, 40, 40, 8, 8, 2, 2, (2, 2), ((0, 0), (0, 0)), (1, 1)),
    # layer-sized: the filter cotangent's k axis (batch x 56 x 56 positions) is cut into slices of one image each, the
    # cotangent operand read as a plain two-stride view (runs of 3136), the activations through the k-vector loader
    (8, 32, 32, 56, 56, 3, 3, (1, 1), ((1, 1), (1, 1)), (1, 1)),
    (4, 64, 64, 56, 56, 3, 3, (1, 1), ((1, 1), (1, 1)), (1, 1)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt", [(F32, np.float32), (F16, np.float16)])
@pytest.mark.parametrize("cfg", RANDOM_CONVS, ids=lambda c: "x".join(map(str, c[:7])) + "_s%d%d_d%d%d" % (c[7] + c[9]))
def test_convolution_cotangents_over_strides_paddings_and_dilations(cfg, dt, npdt):
    """Both cotangent convolutions for strided, padded, dilated and asymmetric windows, sized so that the matcher hands
    them to the matrix-core templates (gather loaders on both operands, input dilation by the forward stride): exact on
    small-integer data against tap-by-tap adjoints."""
    N, C, O, H, W, KH, KW, strides, padding, rd = cfg
    rng = np.random.default_rng(sum(cfg[:7]))
    x = rng.integers(-2, 3, (N, C, H, W)).astype(npdt)
    w = rng.integers(-1, 2, (O, C, KH, KW)).astype(npdt)
    p = ConvParams(0, list(strides), [tuple(q) for q in padding], [1, 1], list(rd))
    from jaxjs_hip.convolution import checkConvShape
    out_shape = checkConvShape(list(x.shape), list(w.shape), p)
    ct = rng.integers(-1, 2, out_shape).astype(npdt)
    dx_want, dw_want = conv_vjp_by_taps(x, w, ct, strides, padding, rd)
    _, (dx,), cls_x = on_gpu(lambda c, f: conv_transposed_to_lhs(c, f, list(x.shape), p), [ct, w], dt)
    _, (dw,), cls_w = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, list(w.shape), p), [x, ct], dt)
    assert np.abs(dx_want).max() < 2048 and np.abs(dw_want).max() < 2048  # exact in float16 too
    np.testing.assert_array_equal(dx.astype(np.float64).reshape(dx_want.shape), dx_want, err_msg=str(cls_x))
    np.testing.assert_array_equal(dw.astype(np.float64).reshape(dw_want.shape), dw_want, err_msg=str(cls_w))


def _fuzz_conv_cases(count=24, seed=3):
    """Seeded random 2-d convolutions: batch 1..16, 8..64 input and 16..128 output channels, images 7..56 wide, windows up
    to 5x5, strides and filter dilations 1 or 2, asymmetric paddings 0..2."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        N, C, O = int(rng.choice([1, 2, 3, 4, 8, 16])), int(rng.choice([8, 16, 24, 32, 48, 64])), int(rng.choice([16, 32, 64, 96, 128]))
        H, W = int(rng.choice([7, 8, 12, 14, 16, 20, 28, 30, 32, 56])), int(rng.choice([7, 8, 12, 14, 16, 20, 24, 28, 32, 40, 56]))
        KH, KW = int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 2, 3, 5]))
        st = (int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2])))
        rd = (int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2])))
        pad = ((int(rng.integers(0, 3)), int(rng.integers(0, 3))), (int(rng.integers(0, 3)), int(rng.integers(0, 3))))
        if (KH - 1) * rd[0] + 1 > H + sum(pad[0]) or (KW - 1) * rd[1] + 1 > W + sum(pad[1]) or N * C * O * H * W * KH * KW > 2e9:
            continue
        cases.append((N, C, O, H, W, KH, KW, st, pad, rd, F16 if rng.random() < 0.5 else F32))
    return cases


@pytest.mark.gpu
@pytest.mark.parametrize("cfg", _fuzz_conv_cases(), ids=lambda c: "x".join(map(str, c[:7])) + "_s%d%d_d%d%d_" % (c[7] + c[9]) + c[10].value)
def test_random_convolutions_forward_and_both_cotangents(cfg):
    """Whatever class and loader each of the three kernels of a convolution layer gets (patch-in-LDS template, row-vector,
    k-vector or element gather loaders, k slices with a fold, reduction classes for thin shapes): forward output, activation
    cotangent and filter cotangent on small-integer data against tap-by-tap host convolutions, exact where the values
    fit the dtype."""
    N, C, O, H, W, KH, KW, st, pad, rd, dt = cfg
    npdt = np.float16 if dt == F16 else np.float32
    rng = np.random.default_rng(N * 1000 + C * 10 + H)
    x = rng.integers(-2, 3, (N, C, H, W)).astype(npdt)
    w = rng.integers(-1, 2, (O, C, KH, KW)).astype(npdt)
    p = ConvParams(0, list(st), [tuple(q) for q in pad], [1, 1], list(rd))
    from jaxjs_hip.convolution import checkConvShape
    ct = rng.integers(-1, 2, checkConvShape(list(x.shape), list(w.shape), p)).astype(npdt)
    _, (y,), _c = on_gpu(lambda a, b: L.convGeneralDilated(a, b, list(st), [tuple(q) for q in pad], rhsDilation=list(rd)), [x, w], dt)
    _, (dx,), _c = on_gpu(lambda c, f: conv_transposed_to_lhs(c, f, list(x.shape), p), [ct, w], dt)
    _, (dw,), cls_w = on_gpu(lambda a, c: conv_transposed_to_rhs(a, c, list(w.shape), p), [x, ct], dt)
    dx_want, dw_want = conv_vjp_by_taps(x, w, ct, st, pad, rd)
    xp = np.pad(x.astype(np.float64), [(0, 0), (0, 0), pad[0], pad[1]])
    OH, OW = ct.shape[2:]
    y_want = np.zeros(ct.shape)
    for ky in range(KH):
        for kx in range(KW):
            win = xp[:, :, ky * rd[0]:ky * rd[0] + (OH - 1) * st[0] + 1:st[0], kx * rd[1]:kx * rd[1] + (OW - 1) * st[1] + 1:st[1]]
            y_want += np.einsum("nchw,oc->nohw", win, w[:, :, ky, kx].astype(np.float64))
    for got, want, what in ((y, y_want, "forward"), (dx, dx_want, "activation cotangent"), (dw, dw_want, "filter cotangent")):
        if dt == F32 or np.abs(want).max() < 2048:
            np.testing.assert_array_equal(got.astype(np.float64).reshape(want.shape), want, err_msg=f"{what} {cls_w}")
        else:  # float16 cannot hold the sums exactly: half an ulp of the result
            np.testing.assert_allclose(got.astype(np.float64).reshape(want.shape), want, rtol=2.0 ** -10, atol=0, err_msg=what)


def test_layer_sized_cotangent_plans():
    """Which templates and loaders the two cotangent convolutions of a 3x3 layer [8,64,56,56] -> 64 channels get (decided
    on the host): towards the activations the patch-in-LDS convolution template, its flipped and transposed filter read
    through the element loader by the weight pre-pass; towards the filter a GEMM over k = batch x positions in slices of
    a quarter image (whole fractions of the cotangent's runs along k: one run is one image of one channel), the
    activations through the k-vector loader, the cotangent as a plain two-stride view."""
    from jaxjs_hip.kernelgen import generate
    N, C, O, H = 8, 64, 64, 56
    p = ConvParams(0, [1, 1], [(1, 1), (1, 1)], [1, 1], [1, 1])
    for dt in (F16, F32):
        pl = J.jit(lambda c, f: conv_transposed_to_lhs(c, f, [N, C, H, H], p), [ShapedArray((N, O, H, H), dt), ShapedArray((O, C, 3, 3), dt)])
        pr = J.jit(lambda a, c: conv_transposed_to_rhs(a, c, [O, C, 3, 3], p), [ShapedArray((N, C, H, H), dt), ShapedArray((N, O, H, H), dt)])
        kl, kr = generate(pl.kernels[0]), generate(pr.kernels[0])
        assert kl.klass == "gemm" and kr.klass == "gemm+fold" and kr.info["splitk"] == 4 * N, (kl.klass, kr.klass, kr.info)
        if dt == F16:
            assert kl.info["gather"] == {"a": "element (pre-pass)", "b": "patch"} and len(kl.steps) == 2, kl.info
            assert kr.info["gather"] == {"a": "k8", "b": "none"}, kr.info
        else:
            assert kl.info["gather"] == {"a": "element", "b": "rows4"}, kl.info
            assert kr.info["gather"] == {"a": "k4", "b": "none"}, kr.info


@pytest.mark.gpu
def test_transposed_dot_and_gather_cotangents_on_the_gpu():
    """`transposeDot` (src/frontend/linearize.ts:767-774): for c = a @ b the cotangents are ct @ b^T and a^T @ ct -- the
    same contraction Kernels read through transposed views, which must stay on the matrix cores and be exact on integer
    data.  The cotangent of a row gather (an embedding lookup) is the Scatter-add routine with repeated rows."""
    rng = np.random.default_rng(6)
    M, K, N = 256, 384, 512
    a = rng.integers(-2, 3, (M, K)).astype(np.float16)
    b = rng.integers(-2, 3, (K, N)).astype(np.float16)
    ct = rng.integers(-2, 3, (M, N)).astype(np.float16)
    _, (da,), cls_a = on_gpu(lambda c, y: L.matmul(c, J.transpose(y, [1, 0])), [ct, b], F16)
    _, (db,), cls_b = on_gpu(lambda x, c: L.matmul(J.transpose(x, [1, 0]), c), [a, ct], F16)
    np.testing.assert_array_equal(da.reshape(M, K), (ct.astype(np.float32) @ b.astype(np.float32).T).astype(np.float16))
    np.testing.assert_array_equal(db.reshape(K, N), (a.astype(np.float32).T @ ct.astype(np.float32)).astype(np.float16))
    assert cls_a == ["gemm"] and cls_b == ["gemm"]
    V, D, B = 1000, 64, 4096
    idx = rng.integers(0, V, B).astype(np.int32)
    g = rng.integers(-3, 4, (B, D)).astype(np.float32)
    from gpu_util import WARM_ONLY, backend
    from jaxjs_hip.routine import Routine, Routines, RoutineType
    rt = Routine(Routines.Scatter, RoutineType([[B, D], [B]], [F32, DType.Int32], [[V, D]], [F32]),
                 dict(op="add", shape=[V, D], axis=[0], outDim=0, uniqueIndices=False))
    if WARM_ONLY:
        pytest.skip("warm-up run")
    be = backend()
    exe = be.prepareRoutineSync(rt)
    s_g, s_i, s_o = be.malloc(g.nbytes, g.tobytes()), be.malloc(idx.nbytes, idx.tobytes()), be.malloc(V * D * 4)
    be.dispatch(exe, [s_g, s_i], [s_o])
    got = np.frombuffer(be.readSync(s_o), np.float32).reshape(V, D)
    for s in (s_g, s_i, s_o):
        be.decRef(s)
    want = np.zeros((V, D), np.float64)
    np.add.at(want, idx, g.astype(np.float64))
    np.testing.assert_array_equal(got, want.astype(np.float32))  # small integers: exact in any order
