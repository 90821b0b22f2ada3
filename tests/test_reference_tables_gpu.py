"""Tables of the reference's device-parameterised suite, replayed on the hip backend through traced programs
(the suite itself needs a newer Node than this image has): reductions over axes (test/numpy.test.ts:24-43,
3041-3096, 221-257), argmax/argmin (test/argreduce.test.ts:14-70, test/numpy.test.ts:4007-4035), logsumexp
(test/nn.test.ts:166-180), float16 sums and dots accumulating in float32 (test/dtype-f16.test.ts:77-89) and exp
over its whole range (test/numpy.test.ts:2803-2830).  Every case runs under the Wasm-faithful and the fast numerics."""
import math

import numpy as np
import pytest

from gpu_util import WARM_ONLY, backend, fast_backend
from jaxjs_hip import jit as J
from jaxjs_hip import library as L
from jaxjs_hip.alu import DType
from jaxjs_hip.jit import ShapedArray
from jit_util import run_program

pytestmark = pytest.mark.gpu
if WARM_ONLY:  # every comparison below would see the empty placeholder
    pytestmark = [pytest.mark.gpu, pytest.mark.xfail(reason="warm-up run: compiled only", strict=False)]
F32, F16, I32 = DType.Float32, DType.Float16, DType.Int32
NP = {F32: np.float32, F16: np.float16, I32: np.int32}


@pytest.fixture(params=["wasm", "fast"])
def be(request):
    if WARM_ONLY:
        return request.param
    return backend() if request.param == "wasm" else fast_backend()


def run(be, fn, *arrays, dtype=F32):
    arrays = [np.asarray(a, dtype=NP[dtype]) for a in arrays]
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), dtype) for a in arrays])
    if WARM_ONLY:  # compile this program's kernels into the on-disk cache and move on to the next program
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for k in prog.kernels + [c.kernel() for c in prog.consts]:
            for src in generate(k, be).sources:
                compile_source(src)
        return np.zeros(0)
    outs = run_program(be, prog, arrays)
    return outs[0] if len(outs) == 1 else outs


def test_sum_over_several_axes(be):
    x = np.arange(24).reshape(2, 3, 4)
    np.testing.assert_array_equal(run(be, lambda a: a.sum([0, 2]), x), [60, 92, 124])
    np.testing.assert_array_equal(run(be, lambda a: a.sum([0, 2], keepdims=True), x), [60, 92, 124])
    np.testing.assert_array_equal(run(be, lambda a: a.sum([0, 2]), x, dtype=I32), [60, 92, 124])


def test_min_max_tables(be):
    v, m = [3, 1, 4, 2], [[3, 1, 4], [2, 5, 0]]
    assert run(be, lambda a: a.min(), v).tolist() == [1] and run(be, lambda a: a.max(), v).tolist() == [4]
    np.testing.assert_array_equal(run(be, lambda a: a.min(0), m), [2, 1, 0])
    np.testing.assert_array_equal(run(be, lambda a: a.max(0), m), [3, 5, 4])
    assert run(be, lambda a: a.min(), m).tolist() == [0] and run(be, lambda a: a.max(), m).tolist() == [5]


def test_mean_tables(be):
    assert run(be, lambda a: a.mean(), [1, 2, 3, 4], dtype=I32).tolist() == [2.5]
    assert run(be, lambda a: a.mean(), [1, 2, 3, 4]).tolist() == [2.5]
    got = run(be, lambda a: a.mean(1), [[1, 2, 3], [4, 5, 6]], dtype=I32)
    assert got.dtype == np.float32 and got.tolist() == [2, 5]


def test_argmax_argmin_tables(be):
    flat = lambda f: (lambda a: f(a.reshape([a.aval.size]), 0))  # noqa: E731  (np.argmax(x) ravels first, numpy.ts:538-540)
    assert run(be, flat(L.argmax), [3, 5, 5, 2, 5, 1]).tolist() == [1]
    assert run(be, flat(L.argmax), [-10, -5, -20, -5, -15]).tolist() == [1]
    assert run(be, flat(L.argmax), np.ones(5)).tolist() == [0]
    x = [[1, 2, 3], [6, 5, 4], [7, 8, 9]]
    assert run(be, flat(L.argmax), x).tolist() == [8]
    assert run(be, lambda a: L.argmax(a, 0), x).tolist() == [2, 2, 2]
    assert run(be, lambda a: L.argmax(a, 1), x).tolist() == [2, 0, 2]
    assert run(be, flat(L.argmin), [3, 1, 5, 1, 1, 2]).tolist() == [1]
    assert run(be, flat(L.argmin), np.ones(5) * 42).tolist() == [0]
    y = [[9, 8, 7], [4, 5, 6], [3, 2, 1]]
    assert run(be, flat(L.argmin), y).tolist() == [8]
    assert run(be, lambda a: L.argmin(a, 0), y).tolist() == [2, 2, 2]
    assert run(be, lambda a: L.argmin(a, 1), y).tolist() == [2, 0, 2]
    assert run(be, flat(L.argmax), [0.1, 0.2, 0.3, 0.2]).tolist() == [2]
    assert run(be, lambda a: L.argmax(a, 1), [[0.1, -0.2, -0.3, 0.1], [0, 0.1, 0.3, 0.3]]).tolist() == [0, 2]
    assert run(be, flat(L.argmax), [[0.1, -0.2], [0.3, 0.1]]).tolist() == [2]


def test_logsumexp_table(be):
    assert run(be, lambda a: L.logsumexp(a), [-10, -1, 1, 2])[0] == pytest.approx(2.3490167, abs=5e-3)   # toBeCloseTo
    assert run(be, lambda a: L.logsumexp(a), [[1, 2, 3, 4], [5, 6, 7, 8]])[0] == pytest.approx(8.45834, abs=5e-3)
    x = np.random.default_rng(5).normal(0, 3, (64, 1000)).astype(np.float32)
    want = np.log(np.sum(np.exp(x.astype(np.float64) - x.max(1, keepdims=True)), axis=1)) + x.max(1)
    np.testing.assert_allclose(run(be, lambda a: L.logsumexp(a, 1), x), want, rtol=1e-5)


def test_f16_reductions_accumulate_in_f32(be):
    x = [100, 1, 1, 1, 1, 1, 1, 1, 1]
    got = run(be, lambda a: L.lax_dot(a, a, [0], [0]), x, dtype=F16)
    assert got.dtype == np.float16 and got.tolist() == [10008]
    got = run(be, lambda a: a.sum(), [16000, 1, 1, 1, 1, 1, 1, 1, 1], dtype=F16)
    assert got.dtype == np.float16 and got.tolist() == [16008]


def test_exp_small_and_large(be):
    got = run(be, lambda a: J.exp(a), [-math.inf, 0, 1, 2, 3])
    np.testing.assert_allclose(got, [0, 1, math.e, math.e ** 2, math.e ** 3], rtol=1e-5, atol=1e-7)
    got = run(be, lambda a: J.exp(a), [-1000, -100, -50, -10, 0, 10, 50, 100, 1000])
    want = [0, 3.720075976020836e-44, 1.9287498479639178e-22, 4.5399929762484854e-5, 1, 22026.465794806718,
            5.184705528587072e21, 2.6881171418161356e43, math.inf]
    with np.errstate(over="ignore"):
        want32 = np.array(want, np.float64).astype(np.float32)  # exp(100) is beyond float32: Inf
    np.testing.assert_allclose(got, want32, rtol=1e-5, atol=1e-7)
    assert got[0] == 0 and got[-1] == math.inf and got[4] == 1
