"""Programs on which the device compiler has aborted the process, compiled afresh in a child process (no GPU needed:
hiprtc cross-compiles), so that a compiler abort fails a test here instead of ending a user's process on the GPU box.
The cases are the float16 programs whose unrolled lanes round a float32 intermediate and negate or subtract it."""
import multiprocessing as mp

import pytest

from jaxjs_hip import DType


def _cases():
    from jaxjs_hip import jit as J, library as Lb
    mm = [(256, 256), (256, 256)]
    return {
        "logSoftmax_rows_of_50257": (lambda x: Lb.logSoftmax(x, -1), [(8, 50257)]),
        "logSigmoid": (lambda x: Lb.logSigmoid(x), [(16, 1001)]),
        "acos": (lambda x: Lb.acos(x), [(3, 5, 77)]),
        "var_axis0": (lambda x: Lb.var_(x, 0), [(3, 5, 77)]),
        "negated_product": (lambda a, b: J.neg(Lb.matmul(a, b)), mm),
        "logSigmoid_behind_a_product": (lambda a, b: Lb.logSigmoid(Lb.matmul(a, b)), mm),
    }


def _compile(name, numerics, out):
    from jaxjs_hip import jit as J
    from jaxjs_hip.jit import ShapedArray
    from jaxjs_hip.kernelgen import generate
    from jaxjs_hip.runtime import compile_source
    fn, shapes = _cases()[name]
    prog = J.jit(fn, [ShapedArray(s, DType.Float16) for s in shapes])
    n = 0
    for k in prog.kernels:
        for src in generate(k, numerics).sources:
            n += len(compile_source(src, use_cache=False)) > 1000
    out.put(n)


@pytest.mark.parametrize("numerics", ["fast", "wasm"])
@pytest.mark.parametrize("name", list(_cases()))
def test_device_compiler_survives(name, numerics):
    ctx = mp.get_context("fork")
    out = ctx.Queue()
    child = ctx.Process(target=_compile, args=(name, numerics, out))
    child.start()
    child.join(300)
    assert child.exitcode == 0, f"the compiler process ended with {child.exitcode}"
    assert out.get(timeout=5) >= 1
