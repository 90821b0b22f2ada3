"""Whole traced programs on the hip backend: the row softmax/argmax pair and the GPT-2-small block.

Every Kernel of a program is checked on its own (inputs taken from the oracle's replay of the program, so
an error cannot hide behind a later kernel), then the program is replayed end to end on the GPU."""
import math

import numpy as np
import pytest

import gpu_util
from gpu_util import WARM_ONLY, backend
from jaxjs_hip import workloads as W
from jaxjs_hip.alu import DType, numpyDtype
from jit_util import run_program
from oracle import oracle
from oracle.backend import OracleBackend
from test_jit import block_inputs, block_reference

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["wasm", "fast"])
def numerics_mode(request):
    """Every program test runs on the Wasm-faithful numerics and again on the backend's default ("fast")."""
    gpu_util.set_numerics(request.param)
    yield request.param
    gpu_util.set_numerics("wasm")


def warm(prog):
    from jaxjs_hip.kernelgen import generate
    from jaxjs_hip.runtime import compile_source
    from jaxjs_hip.routinegen import generateRoutine
    for k in prog.kernels + [c.kernel() for c in prog.consts]:
        for src in generate(k, gpu_util.NUMERICS).sources:
            compile_source(src)
    for r in prog.routines:
        for src in generateRoutine(r, gpu_util.NUMERICS).sources:
            compile_source(src)
    pytest.skip("warm-up run: compiled only")


def replay_on_oracle(prog, arrays):
    """id -> host array for every buffer of the program (constants, inputs, intermediates)."""
    bufs = {}
    for i, c in enumerate(prog.consts):
        bufs[i] = oracle.run_kernel(c.kernel(), [], oracle.MODE_WASM)
    for j, a in enumerate(arrays):
        bufs[len(prog.consts) + j] = np.ascontiguousarray(a)
    for s in prog.steps:
        if s.kind == "execute":
            bufs[s.output] = oracle.run_kernel(s.kernel, [bufs[i] for i in s.inputs], oracle.MODE_WASM)
    return bufs


def check_each_kernel(prog, bufs, f16_rtol=1e-2):
    be = backend()
    classes = []
    for s in prog.steps:
        if s.kind != "execute":
            continue
        k = s.kernel
        exe = be.prepareKernelSync(k)
        slots = [be.malloc(bufs[i].nbytes, bufs[i].tobytes()) for i in s.inputs]
        out = be.malloc(k.bytes)
        be.dispatch(exe, slots, [out])
        got = np.frombuffer(be.readSync(out), dtype=numpyDtype(k.dtype))
        for x in slots + [out]:
            be.decRef(x)
        want = bufs[s.output]
        classes.append(exe.data.ks.klass)
        msg = f"kernel -> buffer {s.output}, class {exe.data.ks.klass}, {exe.data.ks.info}"
        if k.dtype in (DType.Int32, DType.Uint32, DType.Bool):
            np.testing.assert_array_equal(got, want, err_msg=msg)
        elif k.dtype == DType.Float16:
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=f16_rtol, atol=2e-3, equal_nan=True, err_msg=msg)
        elif k.exp.collect(lambda e: e.dtype == DType.Float16):
            # float32 statistics of float16 data (sum of x*x): a float16 product feeding a wider accumulator is formed
            # exactly on the GPU (as an MFMA forms it) where the checker rounds it to float16 first: float16 tolerance
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=2e-3, atol=2e-3, equal_nan=True, err_msg=msg)
        else:
            R = k.reduction.size if k.reduction is not None else 1
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-5 * max(1, math.sqrt(R)), atol=1e-6, equal_nan=True, err_msg=msg)
    return classes


def test_row_softmax_argmax_program():
    prog = W.rowSoftmaxArgmaxProgram(256, 1000)
    if WARM_ONLY:
        warm(prog)
    x = np.random.default_rng(3).standard_normal((256, 1000)).astype(np.float32)
    x[5, 100] = x[5, 900] = 7.0
    bufs = replay_on_oracle(prog, [x])
    assert check_each_kernel(prog, bufs) == ["reduce_row"] * 4
    y, idx = run_program(backend(), prog, [x])
    np.testing.assert_array_equal(idx, np.argmax(x, -1).astype(np.int32))  # bit-exact, first index on ties
    np.testing.assert_allclose(y, bufs[prog.outputs[0]], rtol=1e-5 * math.sqrt(1000))


@pytest.mark.parametrize("rows,cols", [(64, 1001), (16, 50257)], ids=str)
def test_float16_log_softmax_over_rows_off_the_pack_width(rows, cols):
    """`x - log(sum)` in float16 with rows that are not whole packs of eight: every lane of a pack reads its own row's
    statistic, rounds the logarithm to float16 and negates it (the first form on which the device compiler was seen
    to abort; see the test of such programs below); each kernel against the checker."""
    from jaxjs_hip import jit as J, library as Lb
    from jaxjs_hip.jit import ShapedArray
    prog = J.jit(lambda x: Lb.logSoftmax(x, -1), [ShapedArray((rows, cols), DType.Float16)])
    if WARM_ONLY:
        warm(prog)
    x = np.random.default_rng(rows).standard_normal((rows, cols)).astype(np.float16)
    bufs = replay_on_oracle(prog, [x])
    assert check_each_kernel(prog, bufs)[-1] == "map"
    (y,) = run_program(backend(), prog, [x])
    want = x.astype(np.float64) - np.log(np.exp(x.astype(np.float64)).sum(-1, keepdims=True))
    np.testing.assert_allclose(y.astype(np.float64).reshape(rows, cols), want, rtol=1e-2, atol=2e-2)


def _float16_cases():
    from jaxjs_hip import jit as J, library as Lb
    return {
        "logSigmoid": (lambda x: Lb.logSigmoid(x), [(16, 1001)]),
        "acos": (lambda x: Lb.acos(Lb.tanh(x)), [(16, 1001)]),
        "var_axis0": (lambda x: Lb.var_(x, 0), [(3, 5, 77)]),
        "negated_product": (lambda a, b: J.neg(Lb.matmul(a, b)), [(256, 256), (256, 256)]),
        "logSigmoid_behind_a_product": (lambda a, b: Lb.logSigmoid(Lb.matmul(a, b)), [(256, 256), (256, 256)]),
    }


@pytest.mark.parametrize("name", list(_float16_cases()))
def test_float16_programs_the_device_compiler_used_to_abort_on(name):
    """Float16 kernels whose unrolled lanes round a float32 intermediate and then negate or subtract it: the device
    compiler's SLP vectorizer paired those lanes and instruction selection aborted the process (such sources now ask
    for compilation without that pass).  Every kernel against the checker."""
    from jaxjs_hip import jit as J
    from jaxjs_hip.jit import ShapedArray
    fn, shapes = _float16_cases()[name]
    prog = J.jit(fn, [ShapedArray(s, DType.Float16) for s in shapes])
    if WARM_ONLY:
        warm(prog)
    rng = np.random.default_rng(len(name))
    arrs = [(rng.standard_normal(s) * (0.1 if len(shapes) == 2 else 1.0)).astype(np.float16) for s in shapes]
    bufs = replay_on_oracle(prog, arrs)
    check_each_kernel(prog, bufs, f16_rtol=2e-2)


@pytest.mark.parametrize("dtype", [DType.Float16, DType.Float32], ids=lambda d: d.value)
@pytest.mark.parametrize("rows,width,wide", [(1000, 768, True), (77, 64, True), (1000, 61, False)], ids=str)
def test_table_rows_by_loaded_ids_including_ids_outside_the_table(rows, width, wide, dtype):
    """`take` along axis 0: a row of whole lane groups is fetched with one wide load per group.  Ids outside the table
    go the way the lowered index arithmetic takes them (wrap modulo the table, then the guard's element 0): bit-exact
    against the checker for ids -1, rows, -rows, 2^31 - 1, -2^31 and a multiple of rows beyond the table."""
    from jaxjs_hip import jit as J, library as Lb
    from jaxjs_hip.jit import ShapedArray
    from jaxjs_hip.kernelgen import generate
    n = 4096
    prog = J.jit(lambda t, i: Lb.take(t, i, 0), [ShapedArray((rows, width), dtype), ShapedArray((n,), DType.Int32)])
    (k,) = prog.kernels
    assert ("_in ? " in generate(k, gpu_util.NUMERICS).sources[0]) == wide
    if WARM_ONLY:
        warm(prog)
    rng = np.random.default_rng(rows + width)
    table = rng.standard_normal((rows, width)).astype(numpyDtype(dtype))
    ids = rng.integers(0, rows, n).astype(np.int32)
    ids[:8] = [-1, rows, -rows, 2**31 - 1, -2**31, 3 * rows, -3 * rows, rows - 1]
    want = oracle.run_kernel(k, [table, ids], oracle.MODE_WASM)
    np.testing.assert_array_equal(want.reshape(n, width)[8:], table[ids[8:]])
    (y,) = run_program(backend(), prog, [table, ids])
    np.testing.assert_array_equal(y.ravel(), want.ravel())


def test_attention_scores_over_ragged_lengths_take_the_shallow_plan_and_are_exact():
    """q.k^T over a head size of 64 with 300 positions (not a multiple of any tile): the plan for short k axes under
    many tiles applies through clamped edge loads.  Small integers, so the float16 result is exact."""
    from jaxjs_hip import jit as J, library as Lb
    from jaxjs_hip.jit import ShapedArray
    from jaxjs_hip.kernelgen import generate
    B, L, N, H = 12, 300, 12, 64
    prog = J.jit(lambda q, k: Lb.einsum("BLNH,BSNH->BNLS", q, k), [ShapedArray((B, L, N, H), DType.Float16)] * 2)
    info = generate(prog.kernels[0], gpu_util.NUMERICS).info
    assert (info["BM"], info["BN"], info["direct_lds"], info["stages"]) == (128, 128, True, 2), info
    if WARM_ONLY:
        warm(prog)
    rng = np.random.default_rng(9)
    q, k = [rng.integers(-2, 3, (B, L, N, H)).astype(np.float16) for _ in range(2)]
    (y,) = run_program(backend(), prog, [q, k])
    want = np.einsum("blnh,bsnh->bnls", q.astype(np.float32), k.astype(np.float32))
    np.testing.assert_array_equal(y.astype(np.float32).reshape(want.shape), want)


def _piece_cases():
    from jaxjs_hip import library as Lb
    cat = lambda axis: (lambda *xs: Lb.concatenate(list(xs), axis), lambda *xs: np.concatenate(xs, axis))  # noqa: E731
    pad = lambda w: (lambda x: Lb.pad(x, w), lambda x: np.pad(x, w))  # noqa: E731
    return {
        "kv_append": (cat(1), [(2, 255, 4, 64), (2, 1, 4, 64)], True),
        "three_pieces_axis0": (cat(0), [(100, 264), (3, 264), (50, 264)], True),
        "last_axis_40_24": (cat(1), [(512, 40), (512, 24)], True),
        "last_axis_5_7": (cat(1), [(512, 5), (512, 7)], False),  # pieces that are not whole lane groups: element loads
        "pad_channels": (pad([(0, 0), (8, 8), (0, 0), (0, 0)]), [(2, 16, 12, 12)], True),
        "pad_rows": (pad([(3, 73), (0, 0)]), [(128, 768)], True),
        "pad_image": (pad([(0, 0), (0, 0), (1, 1), (1, 1)]), [(2, 16, 12, 12)], False),
    }


@pytest.mark.parametrize("dtype", [DType.Float16, DType.Float32], ids=lambda d: d.value)
@pytest.mark.parametrize("name", list(_piece_cases()))
def test_concatenations_and_paddings_move_whole_lane_groups(name, dtype):
    """Pieces of a concatenation or a padding read their operand under a bounds guard; when every lane group lies
    inside or outside the operand as a whole the group is one wide load.  Bit-exact against numpy, and the plan is the
    one expected (a guarded wide load in the source, or none)."""
    from jaxjs_hip import jit as J
    from jaxjs_hip.jit import ShapedArray
    from jaxjs_hip.kernelgen import generate
    (fn, ref), shapes, wide = _piece_cases()[name]
    prog = J.jit(fn, [ShapedArray(s, dtype) for s in shapes])
    (k,) = prog.kernels
    assert ("_in ? " in generate(k, gpu_util.NUMERICS).sources[0]) == wide
    if WARM_ONLY:
        warm(prog)
    rng = np.random.default_rng(len(name))
    arrs = [rng.standard_normal(s).astype(numpyDtype(dtype)) for s in shapes]
    (y,) = run_program(backend(), prog, arrs)
    np.testing.assert_array_equal(y.reshape(ref(*arrs).shape), ref(*arrs))


@pytest.mark.parametrize("heads,expect_out_proj", [(4, "gemm"), (2, "gemm")])
def test_gpt2_block_small_f16(heads, expect_out_proj):
    """d=128: with 2 heads (H=64) the out-projection reads the attention output through a two-level k axis whose runs
    hold whole MFMA slabs (vector loads); with 4 heads (H=32) the runs are too short for that and the operand is
    loaded element by element -- still on the matrix cores."""
    batch, seq, d, d_ff = 2, 64, 128, 512
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff)
    if WARM_ONLY:
        warm(prog)
    arrs = block_inputs(batch, seq, d, d_ff, np.float16)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    arrays = [arrs[n] for n in order]
    bufs = replay_on_oracle(prog, arrays)
    classes = check_each_kernel(prog, bufs)
    assert classes.count("gemm") == (6 if expect_out_proj == "gemm" else 5) and classes[11] == expect_out_proj
    (y,) = run_program(backend(), prog, arrays)
    np.testing.assert_allclose(y.astype(np.float64), bufs[prog.outputs[0]].astype(np.float64), rtol=2e-2, atol=2e-2)
    want = block_reference(arrs["x"].astype(np.float64), {n: arrs[n].astype(np.float64) for n in order[1:]}, heads)
    np.testing.assert_allclose(y.astype(np.float64).reshape(batch, seq, d), want, rtol=3e-2, atol=3e-2)


def check_each_kernel_on_a_sample(be, prog, arrays, per_kernel=1500, seed=0):
    """Run the program step by step on the GPU and check every Kernel on its own: its inputs are the buffers the GPU
    itself produced (an error cannot hide behind, or be blamed on, an earlier kernel), its output is compared with the
    checker evaluated at `per_kernel` sampled output positions (the first and last ones included).  Tolerances are the
    contract's: integers exact, float16 outputs rel 1e-2, float32 statistics of float16 data at the float16-product
    tolerance, float32 within the K-scaled bound.  Returns the program's outputs and the worst relative error seen beyond the
    absolute floor."""
    rng = np.random.default_rng(seed)
    scope, host = {}, {}
    for i, c in enumerate(prog.consts):
        k = c.kernel()
        scope[i] = be.malloc(k.bytes)
        be.dispatch(be.prepareKernelSync(k), [], [scope[i]])
        host[i] = np.frombuffer(be.readSync(scope[i]), dtype=numpyDtype(k.dtype))
    for j, a in enumerate(arrays):
        a = np.ascontiguousarray(a)
        scope[len(prog.consts) + j] = be.malloc(a.nbytes, a.tobytes())
        host[len(prog.consts) + j] = a
    worst = 0.0
    for step in prog.steps:
        if step.kind == "malloc":
            scope[step.output] = be.malloc(step.size)
        elif step.kind == "free":
            be.decRef(scope.pop(step.output))
            host.pop(step.output, None)
        elif step.kind == "incref":
            be.incRef(scope[step.output])
        elif step.kind == "execute":
            assert step.routine is None
            k = step.kernel
            exe = be.prepareKernelSync(k)
            be.dispatch(exe, [scope[i] for i in step.inputs], [scope[step.output]])
            got_all = np.frombuffer(be.readSync(scope[step.output]), dtype=numpyDtype(k.dtype))
            host[step.output] = got_all
            idx = np.unique(np.concatenate([rng.integers(0, k.size, per_kernel), [0, k.size - 1]]))
            want = oracle.run_kernel(k, [host[i] for i in step.inputs], oracle.MODE_WASM, gidx=idx)
            got = got_all[idx]
            msg = f"kernel -> buffer {step.output}, class {exe.data.ks.klass}, {exe.data.ks.info}"
            if k.dtype in (DType.Int32, DType.Uint32, DType.Bool):
                np.testing.assert_array_equal(got, want, err_msg=msg)
                continue
            g, w = got.astype(np.float64), want.astype(np.float64)
            R = k.reduction.size if k.reduction is not None else 1
            if k.dtype == DType.Float16:
                # a sum of R float16 products: the checker rounds each product to float16 before it adds, the GPU adds
                # exact products; both round the result to float16 once (rel 1e-2 covers it with an absolute floor)
                rtol, atol = 1e-2, 2e-3
            elif k.exp.collect(lambda e: e.dtype == DType.Float16):
                rtol, atol = 2e-3, 2e-3
            else:
                rtol, atol = 1e-5 * max(1, math.sqrt(R)), 1e-6
            np.testing.assert_allclose(g, w, rtol=rtol, atol=atol, equal_nan=True, err_msg=msg)
            fin = np.isfinite(w) & np.isfinite(g)
            worst = max(worst, float(np.max(np.maximum(np.abs(g[fin] - w[fin]) - atol, 0.0) / np.maximum(np.abs(w[fin]), atol), initial=0.0)))
    outs = [host[o] for o in prog.outputs]
    for s in scope.values():
        be.decRef(s)
    return outs, worst


def test_gpt2_block_full_size_f16_every_kernel_against_the_checker():
    """The benchmark shape (batch 8, seq 1024, d 768, 12 heads, d_ff 3072).  The whole program runs on the GPU and
    every one of its kernels is held to the contract on a sample of its outputs (float16: rel 1e-2), each fed the
    buffers the GPU produced before it.  The end result of batch elements 0 and 7 is then also compared with a float64
    restatement of the block: eighteen float16 roundings apart, so this last bound is a sanity check on the composition
    (a few float16 ulps of values of order 1), not the parity bar."""
    batch, seq, d, heads, d_ff = 8, 1024, 768, 12, 3072
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff)
    if WARM_ONLY:
        warm(prog)
    arrs = block_inputs(batch, seq, d, d_ff, np.float16, seed=11)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    be = backend()
    (y,), worst = check_each_kernel_on_a_sample(be, prog, [arrs[n] for n in order])
    assert worst <= 1e-2, worst
    y = y.reshape(batch, seq, d).astype(np.float64)
    assert np.isfinite(y).all()
    P = {n: arrs[n].astype(np.float64) for n in order[1:]}
    for b in (0, 7):
        want = block_reference(arrs["x"][b:b + 1].astype(np.float64), P, heads)[0]
        err = np.abs(y[b] - want)
        assert err.max() < 6e-2 and err.mean() < 4e-3, (b, err.max(), err.mean())


def _routine_program_cases():
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    rng = np.random.default_rng(9)
    f = np.float32
    a = (rng.standard_normal((4, 40, 40)) + 6 * np.eye(40)).astype(f)
    b = rng.standard_normal((4, 40, 3)).astype(f)
    g = rng.standard_normal((3, 24, 24))
    spd = (g @ g.transpose(0, 2, 1) + 24 * np.eye(24)).astype(f)
    x = rng.standard_normal((33, 50)).astype(f)
    re, im = rng.standard_normal((48, 7)).astype(f), rng.standard_normal((48, 7)).astype(f)
    return {
        # name: (function, inputs, exact?)
        "solve": (lambda a, b: L.solve(a, b), [a, b], True),
        "cholesky_then_reconstruct": (lambda s: L.matmul(L.cholesky(s), L.cholesky(s, upper=True)), [spd], False),
        "sort_argsort_axis0": (lambda x: (L.sort(J.exp(x), 0), L.argsort(x, 0)), [x], False),
        "eigh_unsorted": (lambda s: L.eigh_unsorted(s), [spd], True),
        "fft_axis0_roundtrip": (lambda r, i: L.fft(*L.fft(r, i, 0), 0, inverse=True), [re, im], False),
        "lower_triangular_solve": (lambda s, b: L.triangularSolve(L.cholesky(s), b, leftSide=True, lower=True), [spd, rng.standard_normal((3, 24, 5)).astype(f)], True),
    }


@pytest.mark.parametrize("name", ["solve", "cholesky_then_reconstruct", "sort_argsort_axis0", "eigh_unsorted", "fft_axis0_roundtrip",
                                  "lower_triangular_solve"])
def test_programs_with_routines(name):
    """Kernels and routines interleaved in one traced program (LU + triangular solves + the permutation product,
    Cholesky feeding a GEMM, sort of a computed operand along axis 0 ...): hip backend against the oracle backend.
    Programs whose kernels are maps, copies and small exact products around bit-exact routines must agree bit for bit;
    the others within the float32 map tolerance scaled by the contraction length."""
    from jaxjs_hip import jit as J
    from jaxjs_hip.jit import ShapedArray
    fn, arrays, exact = _routine_program_cases()[name]
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), DType.Float32) for a in arrays])
    assert prog.routines
    if WARM_ONLY:
        warm(prog)
    want = run_program(OracleBackend(), prog, arrays)
    got = run_program(backend(), prog, arrays)
    for g, w in zip(got, want):
        if g.dtype.kind != "f":
            np.testing.assert_array_equal(g, w)
        elif exact and name != "solve":
            np.testing.assert_array_equal(g, w)
        else:
            np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-5 * np.abs(w).max())


@pytest.mark.parametrize("shape", [(3, 200, 24), (2, 16, 130), (1, 512, 64)], ids=str)
def test_svd_program(shape):
    """`svd` as the reference composes it (Gram product, Jacobi eigendecomposition routine, argsort + gathers, one more
    product scaled by 1/s; src/library/lax-linalg.ts:102-163) traced and run on the GPU: singular values against
    numpy's float64 SVD, reconstruction and orthogonality of the factors.  (The factors themselves are not compared
    with the CPU run element by element: the Gram matrices of the two differ in the last place and near-degenerate
    eigenvectors may rotate.)"""
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    from jaxjs_hip.jit import ShapedArray
    a = np.random.default_rng(21).standard_normal(shape).astype(np.float32)
    prog = J.jit(lambda x: L.svd(x), [ShapedArray(shape, DType.Float32)])
    assert [r.name.value for r in prog.routines] == ["JacobiEigh", "Argsort"]
    if WARM_ONLY:
        warm(prog)
    u, sv, vh = run_program(backend(), prog, [a])
    m, n = shape[-2:]
    k = min(m, n)
    u, sv, vh = u.reshape(shape[0], m, k).astype(np.float64), sv.reshape(shape[0], k).astype(np.float64), vh.reshape(shape[0], k, n).astype(np.float64)
    want = np.linalg.svd(a.astype(np.float64), compute_uv=False)
    # the Gram matrix squares the condition number: singular values are good to ~eps * s_max^2 / s
    np.testing.assert_allclose(sv, want, rtol=2e-3, atol=2e-4 * want.max())
    np.testing.assert_allclose((u * sv[:, None, :]) @ vh, a, atol=2e-3 * np.abs(a).max())
    eye = np.broadcast_to(np.eye(k), (shape[0], k, k))
    np.testing.assert_allclose(vh @ vh.transpose(0, 2, 1) if m >= n else u.transpose(0, 2, 1) @ u, eye, atol=2e-4)


def _indexing_and_random_cases():
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    F, I, U = DType.Float32, DType.Int32, DType.Uint32
    rng = np.random.default_rng(13)
    table = rng.standard_normal((5000, 96)).astype(np.float32)
    tokens = rng.integers(0, 5000, (8, 128)).astype(np.int32)
    x = rng.standard_normal((64, 300)).astype(np.float32)
    order = np.argsort(x, axis=1).astype(np.int32)
    key = np.array([0, 2024], np.uint32)
    return {
        # name: (function, inputs, dtypes)
        "embedding_lookup": (lambda t, i: L.take(t, i, 0), [table, tokens], [F, I]),
        "take_along_axis": (lambda a, i: L.takeAlongAxis(a, i, 1), [x, order], [F, I]),
        "concat_split_roundtrip": (lambda a: J.concatenate(list(reversed(J.split(a.mul(3.0), 1, [100, 150, 50]))), 1), [x], [F]),
        "random_bits": (lambda k: L.random_bits(k, [1000, 257]), [key], [U]),
        "random_split": (lambda k: L.random_split(k, [7, 3]), [key], [U]),
        "random_uniform": (lambda k: L.random_uniform(k, [300000], -2.0, 3.0), [key], [U]),
        "random_normal": (lambda k: L.random_normal(k, [300000]), [key], [U]),
    }


@pytest.mark.parametrize("name", ["embedding_lookup", "take_along_axis", "concat_split_roundtrip", "random_bits", "random_split",
                                  "random_uniform", "random_normal"])
def test_indexing_and_random_programs(name):
    """Gather (embedding lookup, take-along-axis), Concatenate/Split and the threefry generator traced into programs:
    hip backend against the oracle backend.  Integer and bit results (indices, random bits, key splits) and pure data
    movement must be identical; the normal sampler goes through log/sqrt/cos and is compared within the map tolerance."""
    from jaxjs_hip import jit as J
    from jaxjs_hip.jit import ShapedArray
    fn, arrays, dtypes = _indexing_and_random_cases()[name]
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), d) for a, d in zip(arrays, dtypes)])
    if WARM_ONLY:
        warm(prog)
    want = run_program(OracleBackend(), prog, arrays)
    got = run_program(backend(), prog, arrays)
    for g, w in zip(got, want):
        if name == "random_normal":
            np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-6)
            assert abs(g.mean()) < 0.01 and abs(g.std() - 1) < 0.01
        else:
            np.testing.assert_array_equal(g, w)
