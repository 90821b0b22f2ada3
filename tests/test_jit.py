"""The restated tracing/jit layer: kernel boundaries follow the reference's rules
(src/frontend/jit.ts:792-1096) and the library compositions reproduce the reference's own tables
(test/nn.test.ts, test/numpy.test.ts, test/argreduce.test.ts) when replayed on the CPU oracle."""
import math

import numpy as np
import pytest

from jaxjs_hip import jit as J
from jaxjs_hip import library as L
from jaxjs_hip import workloads as W
from jaxjs_hip.alu import AluOp, DType
from jaxjs_hip.jit import ShapedArray
from jit_util import run_program
from oracle import oracle
from oracle.backend import OracleBackend

F32 = DType.Float32


def run(fn, *arrays, dtype=F32):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), dtype) for a in arrays])
    be = OracleBackend()
    outs = run_program(be, prog, arrays)
    assert be.live_slots() == 0  # every intermediate, constant and output was released exactly once
    return prog, outs


def f32(x):
    return np.asarray(x, dtype=np.float32)


# ---- kernel boundaries ------------------------------------------------------------------------------

def test_elementwise_chain_is_one_kernel():
    prog, (y,) = run(lambda a, b: J.exp(a.mul(b).add(1)).mul(0.5), f32([1, 2, 3]), f32([4, 5, 6]))
    assert len(prog.kernels) == 1 and prog.kernels[0].reduction is None
    np.testing.assert_allclose(y, np.exp(f32([5, 11, 19])) * 0.5, rtol=1e-5)


def test_reduction_fuses_unary_and_literal_epilogue():
    """backend.test.ts:248-286 shape: a reduce followed by +1 stays one kernel with an epilogue."""
    prog, (y,) = run(lambda a: J.neg(a.sum(-1).add(1)), f32([[1, 1], [2, 3], [4, 8]]))
    assert len(prog.kernels) == 1
    np.testing.assert_array_equal(y, f32([-3, -6, -13]))


def test_reduction_epilogue_stops_at_broadcasting_operand_and_second_use():
    # The keepdims reshape is a view op, so the epilogue ends at the sum; the division is a second kernel.
    prog, (y,) = run(lambda a: a.div(a.sum(-1, keepdims=True)), f32([[1, 3], [2, 2]]))
    assert [k.reduction is not None for k in prog.kernels] == [True, False]
    np.testing.assert_allclose(y.reshape(2, 2), [[0.25, 0.75], [0.5, 0.5]], rtol=1e-6)


def test_two_reductions_never_share_a_kernel():
    prog, _ = run(lambda a: a.sum(-1).max(), f32([[1, 2], [3, 4]]))
    assert len(prog.kernels) == 2


def test_dot_operand_with_reuse_is_materialised():
    """An activation feeding a matmul would be recomputed per output column; jit materialises it first."""
    a, b = f32(np.arange(6).reshape(2, 3)), f32(np.arange(12).reshape(3, 4))
    prog, (y,) = run(lambda x, w: L.matmul(J.exp(x), w), a, b)
    assert len(prog.kernels) == 2 and prog.kernels[0].reduction is None
    np.testing.assert_allclose(y.reshape(2, 4), np.exp(a) @ b, rtol=1e-5)
    # A plain input needs no such copy.
    prog, _ = run(lambda x, w: L.matmul(x, w), a, b)
    assert len(prog.kernels) == 1


def test_row_softmax_argmax_program_is_four_row_reductions_plus_one_constant():
    prog = W.rowSoftmaxArgmaxProgram(16, 40)
    assert len(prog.kernels) == 4 and all(k.reduction is not None and k.reduction.size == 40 for k in prog.kernels)
    assert len(prog.consts) == 1 and prog.consts[0].shape == (40,)
    x = np.random.default_rng(0).standard_normal((16, 40)).astype(np.float32)
    x[3, 7] = x[3, 21] = 9.0  # a tie: the first index wins
    y, idx = run_program(OracleBackend(), prog, [x])
    x64 = x.astype(np.float64)
    want = (np.exp(x64 - x64.max(-1, keepdims=True)) / (1 + np.exp(-x64))).sum(-1)
    np.testing.assert_allclose(y, want, rtol=1e-5)
    np.testing.assert_array_equal(idx, np.argmax(x, -1).astype(np.int32))
    assert idx[3] == 7


def test_max_args_splits_wide_expressions():
    n = 6
    arrays = [f32([i, i + 1]) for i in range(n)]

    def f(*xs):
        acc = xs[0]
        for x in xs[1:]:
            acc = acc.add(x)
        return acc
    jaxpr, consts = J.trace(f, [ShapedArray((2,), F32)] * n)
    assert len(J.jitCompile(jaxpr, consts, maxArgs=64).kernels) == 1
    prog = J.jitCompile(jaxpr, consts, maxArgs=3)
    assert len(prog.kernels) > 1 and all(k.nargs <= 3 for k in prog.kernels)
    (y,) = run_program(OracleBackend(), prog, arrays)
    np.testing.assert_array_equal(y, sum(arrays))


def test_jaxpr_simplify_folds_literals_and_noop_views():
    def f(a):
        return a.add(0).mul(1).reshape([2, 2]).transpose([0, 1]).add(J.neg(J.scalar(2.0, F32)))
    jaxpr, _ = J.trace(f, [ShapedArray((2, 2), F32)])
    assert [e.primitive for e in jaxpr.eqns] == ["Add"]
    assert isinstance(jaxpr.eqns[0].inputs[1], J.Lit) and jaxpr.eqns[0].inputs[1].value == -2.0


def test_weak_scalars_take_the_array_dtype():
    jaxpr, _ = J.trace(lambda a: a.mul(0.5), [ShapedArray((4,), DType.Float16)])
    assert jaxpr.outs[0].aval.dtype == DType.Float16
    jaxpr, _ = J.trace(lambda a: a.mean(-1), [ShapedArray((4, 8), DType.Float16)])
    assert jaxpr.outs[0].aval.dtype == DType.Float16
    assert [e.primitive for e in jaxpr.eqns] == ["Cast", "Reduce", "Mul", "Cast"]


# ---- library compositions against the reference's tables ---------------------------------------------

def test_softmax_table():  # test/nn.test.ts:106-118
    _, (y,) = run(lambda x: L.softmax(x), f32([[1, 2, 3], [4, 5, 6]]))
    np.testing.assert_allclose(y.reshape(2, 3), [[0.09003057, 0.24472848, 0.66524094]] * 2, rtol=1e-5, atol=1e-7)


GELU_X = [-10, -1, -0.3, 0, 0.1, 0.5, 3, 5, 500]
GELU_Y = [-0, -0.158655, -0.114627, 0, 0.053983, 0.345731, 2.99595, 5, 500]


def test_gelu_tables():  # test/nn.test.ts:86-103
    _, (y,) = run(lambda x: L.gelu(x), f32(GELU_X))
    np.testing.assert_allclose(y, GELU_Y, atol=1e-3)
    _, (y,) = run(lambda x: L.gelu(x, approximate=False), f32(GELU_X))
    np.testing.assert_allclose(y, GELU_Y, rtol=1e-5, atol=1e-5)  # the table itself carries 6 digits


def test_tanh_matches_libm_and_saturates():
    x = f32([-100, -3, -0.5, 0, 1e-3, 0.5, 3, 100])
    _, (y,) = run(lambda v: L.tanh(v), x)
    np.testing.assert_allclose(y, np.tanh(x.astype(np.float64)), rtol=2e-4, atol=1e-6)
    assert y[0] == -1 and y[-1] == 1


def test_standardize_table():  # test/nn.test.ts:217-229
    _, (y,) = run(lambda x: L.standardize(x), f32([[1, 2, 3], [4, 5, 6]]))
    np.testing.assert_allclose(y.reshape(2, 3), [[-1.22474487, 0, 1.22474487]] * 2, rtol=1e-4, atol=1e-5)


def test_attention_tables():  # test/nn.test.ts:274-390
    q = f32([[[[1, 0, 0, 0]], [[0, 1, 0, 0]]]])
    v = f32([[[[1, 2, 3, 4]], [[5, 6, 7, 8]]]])
    prog, (y,) = run(lambda a, b, c: L.dotProductAttention(a, b, c), q, q, v)
    a, b = 0.62245935, 0.37754068
    np.testing.assert_allclose(y.reshape(1, 2, 1, 4)[0, 0, 0], [a * 1 + b * 5, a * 2 + b * 6, a * 3 + b * 7, a * 4 + b * 8], atol=1e-5)
    e = f32([[[[1, 0]], [[0, 1]]]])
    _, (y,) = run(lambda a, b, c: L.dotProductAttention(a, b, c, scale=1.0), e, e, e)
    np.testing.assert_allclose(y.reshape(1, 2, 1, 2)[0, 0, 0], [0.7310586, 0.26894143], atol=1e-5)


def test_causal_attention_closed_form():  # test/nn.test.ts:371-390
    q = f32([[[[1, 0]], [[0.2, 0.2]], [[1, 1]]]])
    k = f32([[[[1, 0]], [[0, 1]], [[1, 1]]]])
    v = f32([[[[1, 0]], [[0, 1]], [[0, 0]]]])
    prog, (y,) = run(lambda a, b, c: L.dotProductAttention(a, b, c, isCausal=True), q, k, v)
    y = y.reshape(1, 3, 1, 2)
    np.testing.assert_allclose(y[0, 0, 0], [1, 0], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(y[0, 1, 0], [0.5, 0.5], rtol=1e-5, atol=1e-7)
    c = 1 / (2 + math.exp(math.sqrt(0.5)))
    np.testing.assert_allclose(y[0, 2, 0], [c, c], rtol=1e-5, atol=1e-7)
    assert len(prog.consts) == 1 and prog.consts[0].dtype == DType.Bool  # the triangular mask


def test_matmul_integer_cases_are_exact():  # test/numpy.test.ts:1510-1560, 1696-1747
    _, (y,) = run(lambda a, b: L.matmul(a, b), f32([[1, 2], [3, 4]]), f32([[5, 6], [7, 8]]))
    np.testing.assert_array_equal(y.reshape(2, 2), [[19, 22], [43, 50]])
    a = f32(np.arange(1 * 784).reshape(1, 784) % 7)
    b = f32(np.ones((784, 10)))
    _, (y,) = run(lambda p, q: L.matmul(p, q), a, b)
    np.testing.assert_array_equal(y, np.full(10, a.sum()))
    # stacked batch
    a = f32(np.arange(2 * 3 * 3).reshape(2, 3, 3))
    _, (y,) = run(lambda p, q: L.matmul(p, q), a, a)
    np.testing.assert_array_equal(y.reshape(2, 3, 3), a @ a)


def test_einsum_layouts_of_attention():
    rng = np.random.default_rng(1)
    B, Lq, N, H, S = 2, 3, 2, 4, 5
    q = f32(rng.integers(-3, 4, (B, Lq, N, H)))
    k = f32(rng.integers(-3, 4, (B, S, N, H)))
    _, (y,) = run(lambda a, b: L.einsum("BLNH,BSNH->BNLS", a, b), q, k)
    np.testing.assert_array_equal(y.reshape(B, N, Lq, S), np.einsum("BLNH,BSNH->BNLS", q, k))
    p = f32(rng.integers(-3, 4, (B, N, Lq, S)))
    _, (y,) = run(lambda a, b: L.einsum("BNLS,BSNH->BLNH", a, b), p, k)
    np.testing.assert_array_equal(y.reshape(B, Lq, N, H), np.einsum("BNLS,BSNH->BLNH", p, k))


# ---- transformer block ---------------------------------------------------------------------------------

def block_reference(x, P, heads):
    """float64 numpy restatement of the block, for a tolerance check of the whole program."""
    def ln(v, g, b):
        mu = v.mean(-1, keepdims=True)
        var = (v * v).mean(-1, keepdims=True) - mu * mu
        return (v - mu) / np.sqrt(var + 1e-5) * g + b
    B, T, d = x.shape
    H = d // heads
    h = ln(x, P["ln1_g"], P["ln1_b"])
    qkv = h @ P["w_qkv"] + P["b_qkv"]
    q, k, v = (qkv[..., i * d:(i + 1) * d].reshape(B, T, heads, H) for i in range(3))
    s = np.einsum("BLNH,BSNH->BNLS", q, k) / math.sqrt(H)
    s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p = p / p.sum(-1, keepdims=True)
    a = np.einsum("BNLS,BSNH->BLNH", p, v).reshape(B, T, d)
    x = x + a @ P["w_o"] + P["b_o"]
    h = ln(x, P["ln2_g"], P["ln2_b"])
    m = h @ P["w_fc1"] + P["b_fc1"]
    m = 0.5 * m * (1 + np.tanh(math.sqrt(2 / math.pi) * (m + 0.044715 * m ** 3)))
    return x + m @ P["w_fc2"] + P["b_fc2"]


def block_inputs(batch, seq, d, d_ff, dtype, seed=5):
    rng = np.random.default_rng(seed)
    shapes = W.gpt2BlockShapes(batch, seq, d, d_ff)
    arrs = {n: (rng.standard_normal(s) * (1.0 if n == "x" else 0.05)).astype(dtype) for n, s in shapes.items()}
    arrs["ln1_g"] = (1 + arrs["ln1_g"]).astype(dtype)
    arrs["ln2_g"] = (1 + arrs["ln2_g"]).astype(dtype)
    return arrs


def test_gpt2_block_program_structure_and_values_f32():
    batch, seq, d, heads, d_ff = 2, 16, 32, 4, 64
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff, dtype=F32)
    # 6 contractions (QKV, QK^T, AV, out, fc1, fc2), 4 LayerNorm moment reductions, 2 softmax reductions,
    # and the maps between them; one closed-over constant (the causal mask).
    assert len(prog.kernels) == 18 and len(prog.consts) == 1
    assert sum(1 for k in prog.kernels if k.reduction is not None) == 12
    arrs = block_inputs(batch, seq, d, d_ff, np.float32)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    (y,) = run_program(OracleBackend(), prog, [arrs[n] for n in order])
    want = block_reference(arrs["x"].astype(np.float64), {n: arrs[n].astype(np.float64) for n in order[1:]}, heads)
    np.testing.assert_allclose(y.reshape(batch, seq, d), want, rtol=2e-4, atol=2e-5)


# ---- routine primitives inside traced programs (src/frontend/jit.ts:290-327, 990-1008) -----------------------------

def steps_of(prog):
    return [(s.routine.name.value if s.routine is not None else "kernel") for s in prog.steps if s.kind == "execute"]


def test_routine_outputs_and_operands_are_dispatch_boundaries():
    x = np.random.default_rng(0).standard_normal((6, 4)).astype(np.float32)
    # exp feeds the routine: it must be its own kernel; the routine's output feeds a fused map
    prog, (y,) = run(lambda a: J.sort(J.exp(a)).mul(2.0), x)
    assert steps_of(prog) == ["kernel", "Sort", "kernel"]
    np.testing.assert_allclose(y.reshape(6, 4), np.sort(np.exp(x), -1) * 2, rtol=1e-6)
    # sort along axis 0: the transposed operand is realised by a copy kernel, the result is transposed back lazily
    prog, (s0, a0) = run(lambda a: (L.sort(a, 0), L.argsort(a, 0)), x)
    assert steps_of(prog).count("Sort") == 1 and steps_of(prog).count("Argsort") == 1
    np.testing.assert_array_equal(s0.reshape(6, 4), np.sort(x, 0))
    np.testing.assert_array_equal(a0.reshape(6, 4), np.argsort(x, 0, kind="stable"))
    assert prog.routines[0].type.inputShapes == [[4, 6]]


def test_attention_routine_takes_plain_strided_views_and_copies_the_rest():
    """The fused-attention routine reads its operands through strides: slices of one buffer reach it as (buffer,
    strides, offset) with no copy; a view its 128-bit loads cannot take (offset 4) and a computed operand are realised
    by a kernel first.  Values are checked through the CPU checker, which reads the same views."""
    from oracle.routines import attention as attention64
    B, T, N, H = 1, 128, 2, 64
    rng = np.random.default_rng(5)
    qkv = rng.standard_normal((B, T, 3 * N * H)).astype(np.float16)

    def slices(a):
        parts = [J.reshape(J.shrink(a, [(0, B), (0, T), (i * N * H, (i + 1) * N * H)]), (B, T, N, H)) for i in range(3)]
        return J.attention(parts[0], parts[1], parts[2], 0.125, True)
    prog, (y,) = run_typed(slices, [qkv], [DType.Float16])
    assert steps_of(prog) == ["Attention"]
    views = prog.routines[0].params["views"]
    assert [v["offset"] for v in views] == [0, N * H, 2 * N * H] and views[0]["strides"] == [0, 3 * N * H, H, 1]  # batch of one: stride 0
    q, k, v = [qkv[..., i * N * H:(i + 1) * N * H].reshape(B, T, N, H) for i in range(3)]
    want = attention64(q, k, v, 0.125, True)
    np.testing.assert_allclose(y.reshape(B, T, N, H).astype(np.float64), want, rtol=2e-3, atol=2e-3)

    wide = rng.standard_normal((B, T, N, H + 4)).astype(np.float16)
    prog, (y2,) = run_typed(lambda a, b: J.attention(J.shrink(a, [(0, B), (0, T), (0, N), (4, H + 4)]), b.mul(2.0), b, 0.125, False),
                            [wide, np.ascontiguousarray(q)], [DType.Float16] * 2)
    assert steps_of(prog) == ["kernel", "kernel", "Attention"]  # the misaligned slice and the computed operand
    assert prog.routines[0].params.get("views") in (None, [None, None, None])
    want2 = attention64(wide[..., 4:], (q * np.float16(2)).astype(np.float16), q, 0.125, False)
    np.testing.assert_allclose(y2.reshape(B, T, N, H).astype(np.float64), want2, rtol=2e-3, atol=2e-3)


def test_solve_is_lu_plus_two_triangular_solves():
    rng = np.random.default_rng(1)
    a = (rng.standard_normal((3, 8, 8)) + 4 * np.eye(8)).astype(np.float32)
    b = rng.standard_normal((3, 8, 2)).astype(np.float32)
    prog, (x,) = run(lambda a, b: L.solve(a, b), a, b)
    assert [n for n in steps_of(prog) if n != "kernel"] == ["LU", "TriangularSolve", "TriangularSolve"]
    assert [r.params for r in prog.routines] == [None, {"unitDiagonal": True}, {"unitDiagonal": False}]
    np.testing.assert_allclose(x.reshape(3, 8, 2), np.linalg.solve(a.astype(np.float64), b), rtol=1e-4, atol=1e-5)
    v = rng.standard_normal((8,)).astype(np.float32)
    _, (x1,) = run(lambda a, b: L.solve(a, b), a[0], v)
    np.testing.assert_allclose(x1, np.linalg.solve(a[0].astype(np.float64), v), rtol=1e-4, atol=1e-5)


def test_triangular_solve_variants_match_the_reference_tables():  # test/lax-linalg.test.ts:332-436
    Lm, b = f32([[2, 0], [1, 3]]), f32([[4], [7]])
    _, (x,) = run(lambda a, b: L.triangularSolve(a, b, leftSide=True, lower=True), Lm, b)
    np.testing.assert_allclose(x, [2, 5 / 3], rtol=1e-6)
    _, (x,) = run(lambda a, b: L.triangularSolve(a, b, leftSide=True, lower=True, transposeA=True), f32([[1, 1e6], [1, 1]]), f32([[1], [1]]))
    np.testing.assert_allclose(x, [0, 1], atol=1e-6)
    _, (x,) = run(lambda a, b: L.triangularSolve(a, b), f32([[2, 1], [0, 3]]), f32([[4, 7]]))
    np.testing.assert_allclose(x, [2, 5 / 3], rtol=1e-6)


def test_cholesky_upper_eigh_and_fft_along_an_axis():
    rng = np.random.default_rng(2)
    x = f32([[2, 1], [1, 2]])
    _, (lo, up) = run(lambda a: (L.cholesky(a), L.cholesky(a, upper=True)), x)
    np.testing.assert_allclose(lo.reshape(2, 2), [[1.4142135, 0], [0.70710677, 1.2247449]], rtol=1e-6)  # lax-linalg.ts:27-32
    np.testing.assert_allclose(up.reshape(2, 2), lo.reshape(2, 2).T)
    a = rng.standard_normal((2, 6, 6)).astype(np.float32)
    prog, (v, d) = run(lambda a: L.eigh_unsorted(a), a)
    assert prog.routines[0].params == {"maxSweeps": 12, "tolerance": 1e-6}
    sym = (a + a.transpose(0, 2, 1)) * 0.5
    v, d = v.reshape(2, 6, 6), d.reshape(2, 6, 6)
    for k in range(2):
        np.testing.assert_allclose((v[k] * np.diagonal(d[k])) @ v[k].T, sym[k], atol=1e-5)
    re, im = rng.standard_normal((12, 5)).astype(np.float32), rng.standard_normal((12, 5)).astype(np.float32)
    prog, (r, i) = run(lambda r, i: L.fft(r, i, 0), re, im)
    assert prog.routines[0].params == {"factors": [4, 3], "inverse": False} and prog.routines[0].type.inputShapes == [[5, 12]] * 2
    np.testing.assert_allclose((r + 1j * i).reshape(12, 5), np.fft.fft(re + 1j * im, axis=0), atol=1e-5)
    _, (r2, i2) = run(lambda r, i: L.fft(*L.fft(r, i, 0), 0, inverse=True), re, im)
    np.testing.assert_allclose(r2.reshape(12, 5), re, atol=1e-6)
    np.testing.assert_allclose(i2.reshape(12, 5), im, atol=1e-6)


def test_eigh_svd_and_diagonal_reference_tables():
    """test/lax-linalg.test.ts:138-275 and test/numpy-linalg.test.ts:128-225: sorted eigenpairs, the selected triangle,
    thin SVD of tall, wide and batched matrices, singular values alone; `diagonal` for every offset and axis order."""
    d3 = f32([[3, 0, 0], [0, 1, 0], [0, 0, 2]])
    _, (vec, val) = run(lambda a: L.eigh(a), d3)
    np.testing.assert_allclose(val, [1, 2, 3], atol=1e-6)
    np.testing.assert_allclose(vec.reshape(3, 3), [[0, 0, 1], [1, 0, 0], [0, 1, 0]], atol=1e-6)
    _, (vec, val) = run(lambda a: L.eigh(a, sortEigenvalues=False), d3)
    np.testing.assert_allclose(val, [3, 1, 2], atol=1e-6)
    np.testing.assert_allclose(vec.reshape(3, 3), np.eye(3), atol=1e-6)
    x = f32([[4, 1, 2], [1, 3, 0.5], [2, 0.5, 5]])
    _, (vec, val) = run(lambda a: L.eigh(a), x)
    vec = vec.reshape(3, 3)
    np.testing.assert_allclose((vec * val) @ vec.T, x, atol=1e-3)
    np.testing.assert_allclose(vec.T @ vec, np.eye(3), atol=1e-3)
    xb = f32([[[2, 1], [1, 2]], [[3, 1], [1, 3]]])
    _, (vec, val) = run(lambda a: L.eigh(a), xb)
    np.testing.assert_allclose(val.reshape(2, 2), [[1, 3], [2, 4]], atol=1e-4)
    tri = f32([[2, 100], [1, 2]])
    _, (_, lo) = run(lambda a: L.eigh(a, symmetrizeInput=False, lower=True), tri)
    _, (_, up) = run(lambda a: L.eigh(a, symmetrizeInput=False, lower=False), tri)
    np.testing.assert_allclose(lo, [1, 3], atol=1e-4)
    np.testing.assert_allclose(up, [-98, 102], rtol=1e-4, atol=1e-4)

    tall = f32([[1, 2], [3, 4], [5, 6]])
    prog, (u, sv, vh) = run(lambda a: L.svd(a), tall)
    assert steps_of(prog).count("JacobiEigh") == 1 and steps_of(prog).count("Argsort") == 1
    u, vh = u.reshape(3, 2), vh.reshape(2, 2)
    np.testing.assert_allclose((u * sv) @ vh, tall, atol=1e-3)
    np.testing.assert_allclose(u.T @ u, np.eye(2), atol=1e-3)
    np.testing.assert_allclose(vh @ vh.T, np.eye(2), atol=1e-3)
    np.testing.assert_allclose(sv, [9.525518, 0.514301], rtol=1e-4, atol=1e-4)
    wide = f32([[1, 2, 3], [4, 5, 6]])
    _, (u, sv, vh) = run(lambda a: L.svd(a), wide)
    u, vh = u.reshape(2, 2), vh.reshape(2, 3)
    np.testing.assert_allclose((u * sv) @ vh, wide, atol=1e-3)
    np.testing.assert_allclose(vh @ vh.T, np.eye(2), atol=1e-3)
    batched = f32([[[1, 2], [3, 4], [5, 6]], [[2, 0], [0, 3], [4, 0]]])
    _, (u, sv, vh) = run(lambda a: L.svd(a), batched)
    u, sv, vh = u.reshape(2, 3, 2), sv.reshape(2, 2), vh.reshape(2, 2, 2)
    np.testing.assert_allclose((u * sv[:, None, :]) @ vh, batched, atol=1e-3)
    _, (sv,) = run(lambda a: L.svdvals(a), f32([[3, 0], [0, 4]]))
    np.testing.assert_allclose(sv, [4, 3], atol=1e-4)
    with pytest.raises(ValueError):
        run(lambda a: L.svd(a, fullMatrices=True), tall)

    m = np.arange(2 * 4 * 6, dtype=np.float32).reshape(2, 4, 6)
    for offset, a1, a2 in ((0, 1, 2), (1, 1, 2), (-2, 1, 2), (3, 2, 1), (0, 0, 2), (1, 2, 0), (5, -2, -1)):
        prog, (d,) = run(lambda t: L.diagonal(t, offset, a1, a2), m)
        want = np.diagonal(m, offset, a1, a2)
        np.testing.assert_array_equal(d.reshape(want.shape), want)
        assert steps_of(prog) == ["kernel"]  # a view: one copy kernel


# ---- Concatenate / Split / Gather / RandomBits (src/frontend/jit.ts:666-763) -------------------------------------------

U32, I32 = DType.Uint32, DType.Int32


def run_typed(fn, arrays, dtypes):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), d) for a, d in zip(arrays, dtypes)])
    be = OracleBackend()
    outs = run_program(be, prog, arrays)
    assert be.live_slots() == 0
    return prog, outs


def prng_key(seed):
    return np.array([0, seed], np.uint32)  # random.key(seed) = [0, seed] (src/library/random.ts:62-76)


def test_random_bits_and_split_match_jax():  # test/random.test.ts:21-48
    _, (b,) = run_typed(lambda k: L.random_bits(k), [prng_key(0)], [U32])
    assert b.tolist() == [4070199207]
    _, (b,) = run_typed(lambda k: L.random_bits(k, [4]), [prng_key(10)], [U32])
    assert b.tolist() == [169096361, 1572511259, 2689743692, 2228103506]
    prog, (s,) = run_typed(lambda k: L.random_split(k, 3), [prng_key(1)], [U32])
    assert s.reshape(3, 2).tolist() == [[507451445, 1853169794], [1948878966, 4237131848], [2441914641, 3819641963]]
    # RandomBits results are always dispatched (their views are heterogeneous), and Concatenate reads clean inputs
    assert sum(1 for k in prog.kernels if k.exp.collect(lambda n: n.op.name == "Threefry2x32")) == 2


def test_uniform_and_normal_distributions():  # test/random.test.ts:50-120 (ranges and moments)
    _, (z,) = run_typed(lambda k: L.random_uniform(k, [2, 3], 10, 15), [prng_key(42)], [U32])
    assert z.dtype == np.float32 and np.all((z >= 10) & (z < 15))
    _, (u,) = run_typed(lambda k: L.random_uniform(k, [50000]), [prng_key(5)], [U32])
    assert 0 <= u.min() and u.max() < 1 and abs(u.mean() - 0.5) < 0.01 and abs(u.var() * 12 - 1) < 0.03
    _, (n,) = run_typed(lambda k: L.random_normal(k, [50000]), [prng_key(3)], [U32])
    assert abs(n.mean()) < 0.02 and abs(n.std() - 1) < 0.02 and abs(np.mean(np.abs(n) < 1) - 0.6827) < 0.01
    _, (e,) = run_typed(lambda k: L.random_exponential(k, [50000]), [prng_key(4)], [U32])
    assert e.min() >= 0 and abs(e.mean() - 1) < 0.03


def test_gather_take_and_take_along_axis():
    x = np.arange(24, dtype=np.float32).reshape(4, 6)
    idx = np.array([[3, 0], [1, 1]], np.int32)
    prog, (t,) = run_typed(lambda a, i: L.take(a, i, 1), [x, idx], [F32, I32])
    np.testing.assert_array_equal(t.reshape(4, 2, 2), np.take(x, idx, 1))
    assert len(prog.kernels) == 1
    _, (t,) = run_typed(lambda a, i: L.take(a, i), [x, idx], [F32, I32])
    np.testing.assert_array_equal(t.reshape(2, 2), np.take(x, idx))
    order = np.argsort(-x, axis=1).astype(np.int32)
    _, (t,) = run_typed(lambda a, i: L.takeAlongAxis(a, i, 1), [x, order], [F32, I32])
    np.testing.assert_array_equal(t.reshape(4, 6), np.take_along_axis(x, order, 1))
    # two index arrays on non-adjacent axes, index dims placed at outDim=0; a computed operand is gathered in-kernel
    y = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    i0, i2 = np.array([1, 0, 1], np.int32), np.array([3, 2, 0], np.int32)
    prog, (g,) = run_typed(lambda a, p, q: J.gather(a.mul(2.0), [p, q], [0, 2], 0), [y, i0, i2], [F32, I32, I32])
    np.testing.assert_array_equal(g.reshape(3, 3), (y * 2)[i0, :, i2])
    assert len(prog.kernels) == 1
    # eigh's final step: sort eigenvalues, reorder the vectors' columns by the same permutation
    vals = np.array([[3.0, 1.0, 2.0]], np.float32)
    vecs = np.arange(9, dtype=np.float32).reshape(1, 3, 3)
    _, (w, v) = run_typed(lambda d, m: (L.takeAlongAxis(d, L.argsort(d), -1), L.takeAlongAxis(m, L.argsort(d).reshape([1, 1, 3]), -1)),
                          [vals, vecs], [F32, F32])
    assert w.tolist() == [1, 2, 3] and v.reshape(3, 3).tolist() == [[1, 2, 0], [4, 5, 3], [7, 8, 6]]


def test_concatenate_stack_and_split():
    x = np.arange(24, dtype=np.float32).reshape(4, 6)
    prog, (c,) = run_typed(lambda a, b: J.concatenate([a.mul(2.0), b], 0), [x, x[:2]], [F32, F32])
    np.testing.assert_array_equal(c.reshape(6, 6), np.concatenate([x * 2, x[:2]], 0))
    assert len(prog.kernels) == 2  # the scaled operand is dispatched first: padding an expression would pad its views
    _, (c,) = run_typed(lambda a, b: J.concatenate([a, b.astype(F32)], 1), [x, np.ones((4, 1), np.int32)], [F32, I32])
    np.testing.assert_array_equal(c.reshape(4, 7), np.concatenate([x, np.ones((4, 1), np.float32)], 1))
    _, (s,) = run_typed(lambda a, b: L.stack([a, b], 1), [x, -x], [F32, F32])
    np.testing.assert_array_equal(s.reshape(4, 2, 6), np.stack([x, -x], 1))
    prog, (a, b, c) = run_typed(lambda a: J.split(a, 1, [2, 3, 1]), [x], [F32])
    np.testing.assert_array_equal(a.reshape(4, 2), x[:, :2])
    np.testing.assert_array_equal(b.reshape(4, 3), x[:, 2:5])
    np.testing.assert_array_equal(c.reshape(4, 1), x[:, 5:])
    with pytest.raises(ValueError):
        run_typed(lambda a: J.split(a, 1, [2, 3]), [x], [F32])
    with pytest.raises(TypeError):
        run_typed(lambda a, b: J.concatenate([a, b], 0), [x, x[:, :2]], [F32, F32])


# ---- output references (src/frontend/jit.ts:449-458) --------------------------------------------------

def _run_keeping_outputs(fn, *arrays):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), F32) for a in arrays])
    be = OracleBackend()
    ins = [be.malloc(a.nbytes, a.tobytes()) for a in arrays]
    outs = prog.execute(be, ins)
    return prog, be, ins, outs


def test_output_returned_twice_carries_two_references():
    """`return [y, y]`: both entries name one slot, and each can be released on its own."""
    x = f32([1, 2, 3])
    prog, be, ins, outs = _run_keeping_outputs(lambda a: (lambda y: [y, y])(a.mul(a)), x)
    assert outs[0] == outs[1] and sum(1 for s in prog.steps if s.kind == "incref") == 1
    be.decRef(outs[0])
    np.testing.assert_array_equal(np.frombuffer(be.readSync(outs[1]), np.float32), [1, 4, 9])  # still alive
    be.decRef(outs[1])
    be.decRef(ins[0])
    assert be.live_slots() == 0


def test_input_returned_twice_beside_a_result():
    """`return [x, y, x]`: the input gains one reference per appearance and stays the caller's as well."""
    x = f32([1, 2, 3])
    prog, be, ins, outs = _run_keeping_outputs(lambda a: [a, a.add(1), a], x)
    assert outs[0] == ins[0] and outs[2] == ins[0] and sum(1 for s in prog.steps if s.kind == "incref") == 2
    for o in outs:
        be.decRef(o)
    np.testing.assert_array_equal(np.frombuffer(be.readSync(ins[0]), np.float32), x)  # the caller's own reference
    be.decRef(ins[0])
    assert be.live_slots() == 0


# ---- reductions and scans of the numpy surface: the reference's tables (test/numpy.test.ts) ----------------------

def _run_typed(fn, arrays, dtypes):
    prog = J.jit(fn, [ShapedArray(tuple(a.shape), d) for a, d in zip(arrays, dtypes)])
    be = OracleBackend()
    outs = run_program(be, prog, arrays)
    assert be.live_slots() == 0
    return prog, outs


def test_count_nonzero_any_all_tables():
    """test/numpy.test.ts:44-92 (countNonzero: all axes, one axis, keepdims, NaN counts as nonzero, int32 result) and
    :4380-4455 (all / any over booleans and truthy numbers, along an axis, keepdims)."""
    x = f32([[1, 0, -2], [0, 3, 0]])
    prog, (c, c0, c1, ck) = run(lambda a: [L.countNonzero(a), L.countNonzero(a, 0), L.countNonzero(a, 1), L.countNonzero(a, 1, keepdims=True)], x)
    assert c.dtype == np.int32 and c.tolist() == [3] and c0.tolist() == [1, 1, 1] and c1.tolist() == [2, 1] and ck.tolist() == [2, 1]
    _, (cn,) = run(lambda a: L.countNonzero(a), f32([0, np.nan, 2]))
    assert cn.tolist() == [2]
    _, (cr,) = run(lambda a: L.countNonzero(a, 1, keepdims=True), f32([[0, 1, 2], [0, 0, 3]]))
    assert cr.tolist() == [2, 1]
    B = DType.Bool
    b = np.array([[1, 0], [1, 1]], np.int32)  # booleans are stored as int32 0/1
    _, (a0, a1, aa, ak) = _run_typed(lambda v: [L.all_(v, 0), L.all_(v, 1), L.all_(v), L.all_(v, 1, keepdims=True)], [b], [B])
    assert a0.tolist() == [1, 0] and a1.tolist() == [0, 1] and aa.tolist() == [0] and ak.tolist() == [0, 1]
    b = np.array([[0, 0], [1, 0]], np.int32)
    _, (y0, y1, ya) = _run_typed(lambda v: [L.any_(v, 0), L.any_(v, 1), L.any_(v)], [b], [B])
    assert y0.tolist() == [1, 0] and y1.tolist() == [0, 1] and ya.tolist() == [1]
    _, (t1, t2, t3, t4) = run(lambda p, q: [L.all_(p), L.all_(q), L.any_(p.mul(0)), L.any_(q)], f32([1, 2, 3]), f32([1, 0, 3]))
    assert (t1.tolist(), t2.tolist(), t3.tolist(), t4.tolist()) == ([1], [0], [0], [1])


def test_prod_ptp_var_std_average_tables():
    """prod is one Mul reduction (test/basic.test.ts:46); var_ / std (test/numpy.test.ts:4242-4254: 1.25 and its root);
    average with weights (:170-218: 2, [2, 5], [5/3, 25/7], keepdims [[2],[5]]); ptp = max - min."""
    x = f32([1, 2, 3, 4])
    prog, (p, v, s, r) = run(lambda a: [L.prod(a), L.var_(a), L.std(a), L.ptp(a)], x)
    assert p.tolist() == [24] and r.tolist() == [3]
    np.testing.assert_allclose(v, [1.25], rtol=1e-6)
    np.testing.assert_allclose(s, [math.sqrt(1.25)], rtol=1e-6)
    m = f32([[1, 2, 3], [4, 5, 6]])
    _, (pa, v0) = run(lambda a: [L.prod(a, 1), L.var_(a, 0, correction=1)], m)
    assert pa.tolist() == [6, 120]
    np.testing.assert_allclose(v0, [4.5, 4.5, 4.5], rtol=1e-6)
    _, (w1,) = run(lambda a, w: L.average(a, 1, weights=w), m, f32([0.25, 0.5, 0.25]))
    assert w1.tolist() == [2, 5]
    _, (w2,) = run(lambda a, w: L.average(a, 1, weights=w), f32([[1, 2], [3, 4]]), f32([[1, 2], [3, 4]]))
    np.testing.assert_allclose(w2, [5 / 3, 25 / 7], rtol=1e-6)
    _, (w3, w4) = run(lambda a: [L.average(a, 1, keepdims=True), L.average(a)], m)
    assert w3.tolist() == [2, 5] and w4.tolist() == [3.5]
    _, (w5,) = run(lambda a, w: L.average(a, weights=w), f32([1, 2, 3]), f32([1, 1, 2]))
    np.testing.assert_allclose(w5, [2.25], rtol=1e-6)


def test_cumsum_cumprod_tables_and_the_two_stage_scan():
    """test/numpy.test.ts:259-293 ([[1,2,3],[5,7,9]] along 0, [[1,3,6],[4,9,15]] along 1, cumprod [1,2,6,24]); the
    scan is one masked n x n reduction up to 512 elements and chunks of 256 plus an exclusive scan of the chunk
    totals beyond (src/library/numpy.ts:577-614) -- small integers keep every order of summation exact."""
    x = f32([[1, 2, 3], [4, 5, 6]])
    prog, (c0, c1, cp) = run(lambda a: [L.cumsum(a, 0), L.cumsum(a, 1), L.cumprod(a.reshape([-1]))], x)
    assert c0.tolist() == [1, 2, 3, 5, 7, 9] and c1.tolist() == [1, 3, 6, 4, 9, 15] and cp.tolist() == [1, 2, 6, 24, 120, 720]
    _, (cs,) = run(lambda a: L.cumsum(a), f32([5]).reshape(()))
    assert cs.tolist() == [5]
    rng = np.random.default_rng(5)
    for n in (512, 513, 1000):
        v = rng.integers(-3, 4, (3, n)).astype(np.float32)
        prog, (got,) = run(lambda a: L.cumsum(a, 1), v)
        np.testing.assert_array_equal(got.reshape(3, n), np.cumsum(v, axis=1))
        assert len(prog.kernels) == (1 if n <= 512 else 3)
    v = rng.choice([1.0, -1.0, 2.0, 0.5], (2, 600)).astype(np.float32)
    _, (gp,) = run(lambda a: L.cumprod(a, 1), v)
    np.testing.assert_array_equal(gp.reshape(2, 600), np.cumprod(v.astype(np.float64), axis=1).astype(np.float32))


def test_diff_tables():
    """test/numpy.test.ts:296-347: first and higher differences, along an axis, prepend / append (scalar and array),
    != on booleans, n = 0 and n beyond the axis."""
    x = f32([1, 2, 4, 7, 0])
    _, (d1, d2, d3) = run(lambda a: [L.diff(a), L.diff(a, 2), L.diff(a, 3)], x)
    assert d1.tolist() == [1, 2, 3, -7] and d2.tolist() == [1, 1, -10] and d3.tolist() == [0, -11]
    _, (same,) = run(lambda a: L.diff(a, 0, -1, prepend=0, append=10), f32([1, 5, 2]))
    assert same.tolist() == [1, 5, 2]
    m = f32([[1, 3, 6, 10], [0, 5, 6, 8]])
    _, (r, c) = run(lambda a: [L.diff(a), L.diff(a, 1, 0)], m)
    assert r.tolist() == [2, 3, 4, 5, 1, 2] and c.tolist() == [-1, 2, 0, -2]
    _, (pa,) = run(lambda a: L.diff(a, 1, -1, prepend=0, append=10), x)
    assert pa.tolist() == [1, 1, 2, 3, -7, 10]
    _, (pb,) = run(lambda a, p: L.diff(a, 1, -1, prepend=p), x, f32([0, 1]))
    assert pb.tolist() == [1, 0, 1, 2, 3, -7]
    _, (db,) = _run_typed(lambda a: L.diff(a), [np.array([1, 1, 0, 1], np.int32)], [DType.Bool])
    assert db.tolist() == [0, 1, 1]
    prog = J.jit(lambda a: L.diff(a, 5), [ShapedArray((3,), F32)])
    assert prog.out_avals[0].shape == (0,) if hasattr(prog, "out_avals") else True
    with pytest.raises(ValueError, match="non-negative"):
        J.jit(lambda a: L.diff(a, -1), [ShapedArray((3,), F32)])
    with pytest.raises(ValueError, match="at least one-dimensional"):
        J.jit(lambda a: L.diff(a), [ShapedArray((), F32)])


def test_flip_rot90_roll_tables():
    """test/numpy.test.ts:1427-1500 (flip, rot90 incl. negative turns and other axes) and :3627-3678 (roll: flat,
    per axis, several axes, shifts beyond the length, rolls of rolls): views and concatenations only."""
    m = f32([[1, 2, 3], [4, 5, 6]])
    _, (fa, f0, f1) = run(lambda a: [J.flip(a, None).mul(1), J.flip(a, 0).mul(1), J.flip(a, 1).mul(1)], m)
    assert fa.tolist() == [6, 5, 4, 3, 2, 1] and f0.tolist() == [4, 5, 6, 1, 2, 3] and f1.tolist() == [3, 2, 1, 6, 5, 4]
    _, (r1, rm, r2) = run(lambda a: [L.rot90(a).mul(1), L.rot90(a, -1).mul(1), L.rot90(a, 2).mul(1)], m)
    assert r1.tolist() == [3, 6, 2, 5, 1, 4] and rm.tolist() == [4, 1, 5, 2, 6, 3] and r2.tolist() == [6, 5, 4, 3, 2, 1]
    c = f32(np.arange(1, 9).reshape(2, 2, 2))
    _, (r3,) = run(lambda a: L.rot90(a, 1, [1, 2]).mul(1), c)
    assert r3.tolist() == [2, 4, 1, 3, 6, 8, 5, 7]
    v = f32([1, 2, 3, 4, 5])
    _, (o1, o2) = run(lambda a: [L.roll(a, 2), L.roll(a, 20).mul(1)], v)
    assert o1.tolist() == [4, 5, 1, 2, 3] and o2.tolist() == [1, 2, 3, 4, 5]
    _, (y1, y2, y3, y4) = run(lambda a: [L.roll(a, 1), L.roll(a, 1, 0), L.roll(a, -1, 1), L.roll(a, [2, 1], [1, 0])], m)
    assert y1.tolist() == [6, 1, 2, 3, 4, 5] and y2.tolist() == [4, 5, 6, 1, 2, 3] and y3.tolist() == [2, 3, 1, 5, 6, 4] and y4.tolist() == [5, 6, 4, 2, 3, 1]
    _, (rr,) = run(lambda a: L.roll(L.roll(a, 1, 0), 1, 1), f32(np.arange(1, 10).reshape(3, 3)))
    assert rr.tolist() == [9, 7, 8, 3, 1, 2, 6, 4, 5]
    with pytest.raises(ValueError):
        J.jit(lambda a: L.rot90(a, 1, [0, 0]), [ShapedArray((2, 2), F32)])


def test_sign_and_float_class_predicates():
    """test/numpy.test.ts:2425-2431 (sign), :4295-4303 (isnan / isinf / isfinite / isneginf / isposinf on
    [NaN, Inf, -Inf, 1])."""
    _, (s,) = run(lambda a: L.sign(a), f32([-10, 0, 5]))
    assert s.tolist() == [-1, 0, 1]
    x = f32([np.nan, np.inf, -np.inf, 1])
    _, (n, i, f, ni, pi) = run(lambda a: [L.isnan(a), L.isinf(a), L.isfinite(a), L.isneginf(a), L.isposinf(a)], x)
    assert n.tolist() == [1, 0, 0, 0] and i.tolist() == [0, 1, 1, 0] and f.tolist() == [0, 0, 0, 1]
    assert ni.tolist() == [0, 0, 1, 0] and pi.tolist() == [0, 1, 0, 0]


def test_trapezoid_tables():
    """test/numpy.test.ts:415-517: unit spacing, dx (number and array along another axis), sample points x (1-D,
    uneven, shaped like y, lower rank), an axis of a 2-D array, a size-1 axis."""
    y = f32([1, 2, 3])
    _, (t1, t2) = run(lambda a: [L.trapezoid(a), L.trapezoid(a, dx=2)], y)
    assert t1.tolist() == [4] and t2.tolist() == [8]
    _, (t3,) = run(lambda a, d: L.trapezoid(a, dx=d, axis=0), f32([[1, 2], [3, 4], [5, 6]]), f32([[1], [2]]))
    assert t3.tolist() == [10, 13]
    _, (t4,) = run(lambda a, x: L.trapezoid(a, x), y, f32([4, 6, 8]))
    assert t4.tolist() == [8]
    _, (t5,) = run(lambda a, x: L.trapezoid(a, x), y, f32([0, 1, 3]))
    np.testing.assert_allclose(t5, [6.5], rtol=1e-6)
    m = f32([[1, 2, 3], [4, 5, 6]])
    _, (a1, a0) = run(lambda a: [L.trapezoid(a, axis=1), L.trapezoid(a, axis=0)], m)
    assert a1.tolist() == [4, 10] and a0.tolist() == [2.5, 3.5, 4.5]
    _, (b1,) = run(lambda a, x: L.trapezoid(a, x), m, f32([0, 1, 3]))
    np.testing.assert_allclose(b1, [6.5, 15.5], rtol=1e-6)
    _, (b2,) = run(lambda a, x: L.trapezoid(a, x), f32([[1, 1, 1], [2, 2, 2]]), f32([[0, 1, 2], [0, 2, 4]]))
    assert b2.tolist() == [2, 8]
    _, (b3,) = run(lambda a, x: L.trapezoid(a, x), np.ones((2, 2, 3), np.float32), f32([[0, 1, 3], [0, 2, 4]]))
    assert b3.tolist() == [3, 4, 3, 4]
    _, (z,) = run(lambda a: L.trapezoid(a), f32([5]))
    assert z.tolist() == [0]
    _, (big,) = run(lambda a, x: L.trapezoid(a, x), f32([1, 1]), f32([-2e9, 2e9]))
    np.testing.assert_allclose(big, [4e9], rtol=1e-6)


def test_matvec_vecmat_tensordot_outer_inner_tables():
    """test/numpy.test.ts:1611-1690 (matvec: plain, batched matrix, batched vectors -- the rotation example; vecmat),
    :1798-1817 (tensordot 2-3-4 with 3-4-5, by count and by explicit axes); outer / inner / vdot / vecdot against numpy."""
    _, (mv,) = run(lambda a, v: L.matvec(a, v), f32([[1, 2], [3, 4]]), f32([5, 6]))
    assert mv.tolist() == [17, 39]
    _, (mb,) = run(lambda a, v: L.matvec(a, v), f32([[[1, 0], [0, 1]], [[0, 1], [1, 0]]]), f32([3, 7]))
    assert mb.tolist() == [3, 7, 7, 3]
    _, (rot,) = run(lambda a, v: L.matvec(a, v), f32([[0, 1, 0], [-1, 0, 0], [0, 0, 1]]), f32([[1, 0, 0], [0, 1, 0], [0, 0, 1], [0, 6, 8]]))
    assert rot.tolist() == [0, -1, 0, 1, 0, 0, 0, 0, 1, 6, 0, 8]
    _, (vm1,) = run(lambda v, a: L.vecmat(v, a), f32([1, 2]), f32([[3, 4], [5, 6]]))
    _, (vm2,) = run(lambda v, a: L.vecmat(v, a), f32([0, 4, 2]), f32([[1, 0, 0], [0, 1, 0], [0, 0, 0]]))
    assert vm1.tolist() == [13, 16] and vm2.tolist() == [0, 4, 0]
    x1, x2 = f32(np.arange(24).reshape(2, 3, 4)), np.ones((3, 4, 5), np.float32)
    _, (td, te) = run(lambda a, b: [L.tensordot(a, b), L.tensordot(a, b, ([1, 2], [0, 1]))], x1, x2)
    assert td.tolist() == [66] * 5 + [210] * 5 and te.tolist() == td.tolist()
    rng = np.random.default_rng(9)
    a, b = rng.integers(-3, 4, (3, 4)).astype(np.float32), rng.integers(-3, 4, (5, 4)).astype(np.float32)
    _, (o, i, vd, vc) = run(lambda p, q: [L.outer(p, q), L.inner(p, q), L.vdot(p, q.reshape([5, 4])[:3] if False else p), L.vecdot(p, p, axis=0)], a, b)
    np.testing.assert_array_equal(o.reshape(12, 20), np.outer(a, b))
    np.testing.assert_array_equal(i.reshape(3, 5), np.inner(a, b))
    assert vd.tolist() == [float(np.vdot(a, a))]
    np.testing.assert_array_equal(vc, np.sum(a * a, axis=0))


I32, U32, BOOL = DType.Int32, DType.Uint32, DType.Bool


def test_min_max_fmin_fmax_abs_signbit_tables():
    """test/numpy.test.ts:2279-2306 (minimum, also of bools), :2307-2345 (fmin ignores one NaN, broadcasts), :2347-2412
    (maximum, fmax incl. infinities), :2414-2423 (absolute), :2438-2484 (signbit: signed zero, the sign of a NaN, int32,
    uint32 and bool inputs)."""
    x, y = f32([1, 2, 3]), f32([4, 2, 0])
    _, (mn, mx, fn, fx) = run(lambda a, b: [J.minimum(a, b), J.maximum(a, b), L.fmin(a, b), L.fmax(a, b)], x, y)
    assert mn.tolist() == [1, 2, 0] and mx.tolist() == [4, 2, 3] and fn.tolist() == [1, 2, 0] and fx.tolist() == [4, 2, 3]
    _, (mb,) = _run_typed(lambda a, b: J.minimum(a, b), [np.array([1, 0, 1], np.int32), np.array([0, 0, 1], np.int32)], [BOOL, BOOL])
    assert mb.tolist() == [0, 0, 1]
    nan, inf = np.nan, np.inf
    _, (a,) = run(lambda p, q: L.fmin(p, q), f32([nan, 2, nan, -inf]), f32([5, nan, nan, 3]))
    np.testing.assert_array_equal(a, f32([5, 2, nan, -inf]))
    _, (b,) = run(lambda p, q: L.fmin(p, q), f32([[1, 5], [4, 2]]), f32([3]))
    assert b.tolist() == [1, 3, 3, 2]
    _, (c,) = run(lambda p, q: L.fmax(p, q), f32([[1, 5], [4, 2]]), f32([3, 3]))
    assert c.tolist() == [3, 5, 4, 3]
    _, (d,) = run(lambda p, q: L.fmax(p, q), f32([1, nan, nan, 5]), f32([nan, 3, nan, 2]))
    np.testing.assert_array_equal(d, f32([1, 3, nan, 5]))
    _, (e,) = run(lambda p, q: L.fmax(p, q), f32([-inf, inf, nan]), f32([2, nan, -inf]))
    np.testing.assert_array_equal(e, f32([2, inf, -inf]))
    _, (ab,) = run(lambda p: L.absolute(p), f32([-1, 2, -3]))
    assert ab.tolist() == [1, 2, 3]
    _, (sb,) = run(lambda p: L.signbit(p), f32([-inf, -3, -0.0, 0, 2, inf]))
    assert sb.tolist() == [1, 1, 1, 0, 0, 0]
    bits = np.array([0xFFC00000, 0x7FC00000], np.uint32).view(np.float32)
    _, (sn,) = run(lambda p: L.signbit(p), bits)
    assert sn.tolist() == [1, 0]
    _, (si,) = _run_typed(lambda p: L.signbit(p), [np.array([-2, 0, 3], np.int32)], [I32])
    _, (su,) = _run_typed(lambda p: L.signbit(p), [np.array([0, 1, 0xFFFFFFFF], np.uint32)], [U32])
    _, (sl,) = _run_typed(lambda p: L.signbit(p), [np.array([0, 1], np.int32)], [BOOL])
    assert si.tolist() == [1, 0, 0] and su.tolist() == [0, 0, 0] and sl.tolist() == [0, 0]


def test_division_family_tables():
    """test/numpy.test.ts:2486-2527 (reciprocal, divide, 1/0 = Inf), :2529-2560 (floorDivide rounds towards -Inf, f32
    and int32), :2562-2609 (fmod keeps the numerator's sign, remainder the divisor's), :2611-2646 (divmod and
    x == q*y + r), :2648-2682 (modf: both parts carry the input's sign; int32 is promoted)."""
    _, (r, dv, z) = run(lambda a, b: [J.reciprocal(a), L.trueDivide(a, b), J._raise(a).mul(0).add(9).div(a.mul(0))], f32([1, 2, 3]), f32([4, 5, 6]))
    np.testing.assert_allclose(r, [1, 0.5, 1 / 3], rtol=1e-6)
    np.testing.assert_allclose(dv, [0.25, 0.4, 0.5], rtol=1e-6)
    assert z.tolist() == [np.inf] * 3
    x, y = [7, 7, -7, -7], [3, -3, 3, -3]
    _, (q, rm) = run(lambda a, b: L.divmod_(a, b), f32(x), f32(y))
    assert q.tolist() == [2, -3, -3, 2] and rm.tolist() == [1, -2, 2, -1]
    _, (q2,) = run(lambda a, b: L.floorDivide(a, b), f32([5, -5, 10, -10]), f32([2, 2, 3, 3]))
    assert q2.tolist() == [2, -3, 3, -4]
    prog, (qi, ri) = _run_typed(lambda a, b: L.divmod_(a, b), [np.array(x, np.int32), np.array(y, np.int32)], [I32, I32])
    assert qi.dtype == np.int32 and qi.tolist() == [2, -3, -3, 2] and ri.dtype == np.int32 and ri.tolist() == [1, -2, 2, -1]
    _, (fm, rr) = run(lambda a, b: [L.fmod(a, b), L.remainder(a, b)], f32([5, 7, -9, -11]), f32([3, -4, 2, -3]))
    assert fm.tolist() == [2, 3, -1, -2]
    _, (r2,) = run(lambda a, b: L.remainder(a, b), f32([5, 5, -5, -5]), f32([3, -3, 3, -3]))
    assert r2.tolist() == [2, -1, 1, -2]
    _, (rec,) = run(lambda a, b: (lambda qr: J.add(J.mul(qr[0], b), qr[1]))(L.divmod_(a, b)), f32([5, -5, 10, -10]), f32([3, 3, 4, 4]))
    assert rec.tolist() == [5, -5, 10, -10]
    _, (fr, wh) = run(lambda a: L.modf(a), f32([3.5, -3.5, 0, 1.25, -2.75, 2.75]))
    np.testing.assert_allclose(fr, [0.5, -0.5, 0, 0.25, -0.75, 0.75], atol=1e-6)
    assert wh.tolist() == [3, -3, 0, 1, -2, 2]
    v = f32([1.7, -4.2, 100.001, -0.5])
    _, (back,) = run(lambda a: (lambda fw: J.add(fw[0], fw[1]))(L.modf(a)), v)
    np.testing.assert_allclose(back, v, atol=1e-6)
    _, (fi, wi) = _run_typed(lambda a: L.modf(a), [np.array([5, -3], np.int32)], [I32])
    assert fi.dtype == np.float32 and wi.dtype == np.float32 and fi.tolist() == [0, 0] and wi.tolist() == [5, -3]


def test_exponential_and_power_tables():
    """test/numpy.test.ts:2803-2853 (exp over [-1000, 1000], exp2), :2855-2871 (expm1 near 0, rtol 2e-5), :2873-2910
    (log, log(0), log2/log10), :2912-2928 (log1p), :2930-2946 (logaddexp, logaddexp2 without overflow), :2948-2960
    (sqrt), :2962-2979 (cbrt of negatives), :2981-3006 (power: negative bases, power of zero), :3008-3039 (floatPower)."""
    _, (e,) = run(lambda a: J.exp(a), f32([-1000, -100, -50, -10, 0, 10, 50, 100, 1000]))
    with np.errstate(over="ignore"):  # e^100 is beyond float32: Inf on both sides
        np.testing.assert_allclose(e, f32([0, 3.720075976020836e-44, 1.9287498479639178e-22, 4.5399929762484854e-5, 1, 22026.465794806718,
                                          5.184705528587072e21, 2.6881171418161356e43, np.inf]), rtol=1e-5, atol=1e-8)
    _, (e2,) = run(lambda a: L.exp2(a), f32([10, 0]))
    np.testing.assert_allclose(e2, [1024, 1], rtol=1e-5)
    vals = [-1, -0.1, -0.01, -1e-4, -1e-8, 0, 1e-8, 1e-4, 0.01, 0.1, 1]
    _, (em,) = run(lambda a: L.expm1(a), f32(vals))
    np.testing.assert_allclose(em, np.expm1(np.array(vals)), rtol=2e-5, atol=0)
    _, (lg, l2, l10) = run(lambda a: [J.log(a), L.log2(a), L.log10(a)], f32([1, 2, 4, 8, 0, math.e]))
    np.testing.assert_allclose(lg[[0, 5]], [0, 1], atol=1e-6)
    assert lg[4] == -np.inf
    np.testing.assert_allclose(l2[:4], [0, 1, 2, 3], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(l10[:4], np.log10([1, 2, 4, 8]), rtol=1e-5, atol=1e-6)
    v1 = [-0.9, -0.2, -0.1, -0.01, -1e-4, -1e-8, 0, 1e-8, 1e-4, 0.01, 0.1, 0.2, 1]
    _, (lp,) = run(lambda a: L.log1p(a), f32(v1))
    np.testing.assert_allclose(lp, np.log1p(np.array(v1)), rtol=2e-5, atol=0)
    _, (la, la2) = run(lambda a, b: [L.logaddexp(a, b), L.logaddexp2(a.mul(0).add(1000), b.mul(0).add(1000))], f32([1, 2, 3]), f32([4, 5, 6]))
    np.testing.assert_allclose(la, np.logaddexp([1, 2, 3], [4, 5, 6]), rtol=1e-5)
    np.testing.assert_allclose(la2, [1001] * 3, rtol=1e-5)
    _, (sq,) = run(lambda a: J.sqrt(a), f32([-1, -4, 9, 1, 4]))
    np.testing.assert_array_equal(sq, f32([np.nan, np.nan, 3, 1, 2]))
    _, (cb,) = run(lambda a: L.cbrt(a), f32([-8, -1, 0, 1, 8]))
    np.testing.assert_allclose(cb, [-2, -1, 0, 1, 2], rtol=1e-5, atol=1e-6)
    _, (p3,) = run(lambda a: L.power(a, 3), f32([-1, 2, 3, 4]))
    np.testing.assert_allclose(p3, [-1, 8, 27, 64], rtol=1e-5)
    _, (pe, pn, p0) = run(lambda a, h, z: [L.power(3, a), L.power(-3, h), L.power(0, z)], f32([-2, 0, 0.5, 1, 2]), f32([0.5, 1.5, 2.5]), f32([-2, -1, 0, 0.5, 1, 2]))
    np.testing.assert_allclose(pe, [1 / 9, 1, math.sqrt(3), 3, 9], rtol=1e-5)
    assert np.isnan(pn).all()
    np.testing.assert_array_equal(p0, f32([np.inf, np.inf, np.nan, 0, 0, 0]))
    prog, (fp,) = _run_typed(lambda a, b: L.floatPower(a, b), [np.array([1, 2, 3, 4], np.int32), f32(3).reshape(())], [I32, F32])
    assert fp.dtype == np.float32
    np.testing.assert_allclose(fp, [1, 8, 27, 64], rtol=1e-5)
    _, (fq, fr) = run(lambda a, b: [L.floatPower(a, 2), L.floatPower(b, 0.5)], f32([1.5, 2.5]), f32([4, 9, 16]))
    np.testing.assert_allclose(fq, [2.25, 6.25], rtol=1e-5)
    np.testing.assert_allclose(fr, [2, 3, 4], rtol=1e-5)


def test_trigonometric_and_hyperbolic_tables():
    """test/numpy.test.ts:4035-4056 (sinh / cosh / tanh over [-1, 1000]), :4058-4088 (sinc: 1 at 0, 0 at integers,
    symmetric), :4118-4152 (atan, asin, acos to 5 digits), :4154-4166 (atan2 in all quadrants and on the axes)."""
    vals = [-1, -0.7, 0, 0.5, 1.7, 10, 50, 100, 1000]
    with np.errstate(over="ignore"):
        _, (sh, ch, th) = run(lambda a: [L.sinh(a), L.cosh(a), L.tanh(a)], f32(vals))
        np.testing.assert_allclose(sh, np.sinh(f32(vals)), rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(ch, np.cosh(f32(vals)), rtol=1e-5)
    np.testing.assert_allclose(th, np.tanh(vals), rtol=1e-5, atol=1e-7)
    _, (ti,) = run(lambda a: L.tanh(a), f32([np.inf]))
    assert ti.tolist() == [1]
    _, (sc,) = run(lambda a: L.sinc(a), f32([0, 0.5, 1, 2, 3, -1, -2, -3, 0.1, -0.1, 1.5, -1.5, 2.5, -2.5]))
    np.testing.assert_allclose(sc[:3], [1, 2 / math.pi, 0], atol=2e-7)
    np.testing.assert_allclose(sc[3:8], 0, atol=1e-5)
    np.testing.assert_array_equal(sc[8::2], sc[9::2])
    av = [-1000, -100, -10, -1, 0, 1, 10, 100, 1000, np.inf]
    _, (at,) = run(lambda a: J.atan(a), f32(av))
    np.testing.assert_allclose(at, np.arctan(av), atol=5e-6)
    sv = [-1, -0.7, 0, 0.5, 1]
    _, (as_, ac) = run(lambda a: [J.asin(a), L.acos(a)], f32(sv))
    np.testing.assert_allclose(as_, np.arcsin(sv), atol=5e-6)
    np.testing.assert_allclose(ac, np.arccos(sv), atol=5e-6)
    yy, xx = [3, 5, -7, -2, 4, -6, 0, 0, 1.5, -2.5], [4, -2, -3, 8, 0, 0, 5, -9, 1.5, -2.5]
    _, (a2,) = run(lambda p, q: L.atan2(p, q), f32(yy), f32(xx))
    np.testing.assert_allclose(a2, np.arctan2(yy, xx), atol=5e-6)
    _, (hy, tn) = run(lambda p, q: [L.hypot(p, q), L.tan(p)], f32([3, 5]), f32([4, 12]))
    np.testing.assert_allclose(hy, [5, 13], rtol=1e-6)
    np.testing.assert_allclose(tn, np.tan([3.0, 5.0]), rtol=1e-4)


def test_nan_to_num_rounding_and_copysign_tables():
    """test/numpy.test.ts:4305-4341 (nanToNum: defaults and overrides), :5152-5165 (copysign; a zero sign source gives
    0), :5167-5190 (round: half to even, decimals, negative decimals; rint)."""
    nan, inf = np.nan, np.inf
    _, (a, b) = run(lambda p: [L.nanToNum(p), L.nanToNum(p, nan=99)], f32([1, nan, 3]))
    assert a.tolist() == [1, 0, 3] and b.tolist() == [1, 99, 3]
    _, (c, d, e) = run(lambda p: [L.nanToNum(p, posinf=999), L.nanToNum(p, neginf=-999), L.nanToNum(p)], f32([1, inf, -inf]))
    assert c.tolist() == [1, 999, np.finfo(np.float32).min] and d.tolist() == [1, np.finfo(np.float32).max, -999]
    np.testing.assert_allclose(e[1:], [3.40282347e38, -3.40282347e38], rtol=1e-7)
    _, (f,) = run(lambda p: L.nanToNum(p, nan=0, posinf=100, neginf=-100), f32([nan, inf, -inf, 42]))
    assert f.tolist() == [0, 100, -100, 42]
    _, (cs, cz) = run(lambda p, q: [L.copysign(p, q), L.copysign(p, q.mul(0))], f32([1, -2, 3, -4]), f32([-1, 1, -1, 1]))
    assert cs.tolist() == [-1, 2, -3, 4] and cz.tolist() == [0, 0, 0, 0]
    _, (r0, ri) = run(lambda p: [L.round_(p, 0), L.rint(p)], f32([1.4, 1.5, 2.5, 3.5, -0.5, 3.6]))
    np.testing.assert_allclose(r0, [1, 2, 2, 4, 0, 4], atol=1e-6)
    np.testing.assert_allclose(ri, [1, 2, 2, 4, 0, 4], atol=1e-6)
    _, (r2,) = run(lambda p: L.round_(p, 2), f32([1.234, 2.567, 3.891]))
    np.testing.assert_allclose(r2, [1.23, 2.57, 3.89], rtol=1e-6)
    _, (rn,) = run(lambda p: L.round_(p, -2), f32([123, 456, 789]))
    np.testing.assert_allclose(rn, [100, 500, 800], rtol=1e-6)


def test_logical_and_bitwise_tables():
    """test/numpy.test.ts:5038-5081 (logical and / or / xor / not over numbers and booleans), :5083-5130 (bitwise and /
    or / xor on uint32 and bool, invert on uint32 / bool / int32), :5132-5150 (shifts; the right shift is logical)."""
    a, b = f32([1, 0, 3, 0]), np.array([0, 0, 1, 0], np.int32)
    _, (an,) = _run_typed(lambda p, q: L.logicalAnd(p, q), [a, b], [F32, BOOL])
    assert an.tolist() == [0, 0, 1, 0]
    _, (af,) = run(lambda p, q: L.logicalAnd(p, q), f32([1.5, 0.0, -2.0]), f32([0.5, 0.0, 1.0]))
    assert af.tolist() == [1, 0, 1]
    _, (o, x, n) = run(lambda p, q: [L.logicalOr(p, q), L.logicalXor(p, q), L.logicalNot(p)], a, f32([0, 0, 1, 0]))
    assert o.tolist() == [1, 0, 1, 0] and x.tolist() == [1, 0, 0, 0] and n.tolist() == [0, 1, 0, 1]
    u = lambda *v: np.array(v, np.uint32)
    _, (ba,) = _run_typed(lambda p, q: L.bitwiseAnd(p, q), [u(0xFF00FF00, 0x0F0F0F0F), u(0x00FF00FF, 0xF0F0F0F0)], [U32, U32])
    _, (bo,) = _run_typed(lambda p, q: L.bitwiseOr(p, q), [u(0xFF00FF00, 7), u(0x00FF00FF, 3)], [U32, U32])
    _, (bx,) = _run_typed(lambda p, q: L.bitwiseXor(p, q), [u(0xAAAAAAAA, 7), u(0x55555555, 3)], [U32, U32])
    assert ba.tolist() == [0, 0] and bo.tolist() == [0xFFFFFFFF, 7] and bx.tolist() == [0xFFFFFFFF, 4]
    _, (bb,) = _run_typed(lambda p, q: L.bitwiseAnd(p, q), [np.array([1, 1, 0, 0], np.int32), np.array([1, 0, 1, 0], np.int32)], [BOOL, BOOL])
    assert bb.tolist() == [1, 0, 0, 0]
    _, (iu,) = _run_typed(lambda p: L.invert(p), [u(0, 0xFFFFFFFF)], [U32])
    _, (ib,) = _run_typed(lambda p: L.invert(p), [np.array([1, 0], np.int32)], [BOOL])
    _, (ii,) = _run_typed(lambda p: L.invert(p), [np.array([0, -3], np.int32)], [I32])
    assert iu.tolist() == [0xFFFFFFFF, 0] and ib.tolist() == [0, 1] and ii.tolist() == [-1, 2]
    with pytest.raises(TypeError):
        J.jit(lambda p: L.invert(p), [ShapedArray((2,), F32)])
    _, (sl,) = _run_typed(lambda p, q: L.leftShift(p, q), [u(1, 1, 1), u(0, 8, 16)], [U32, U32])
    _, (sr,) = _run_typed(lambda p, q: L.rightShift(p, q), [u(256, 65536, 0xFFFF0000), u(0, 1, 8)], [U32, U32])
    assert sl.tolist() == [1, 256, 65536] and sr.tolist() == [256, 32768, 0x00FFFF00]


def run0(fn):
    """A program without inputs: everything comes from lazy constants."""
    return run(fn)[1]


def test_creation_tables():
    """test/numpy.test.ts:563-590 (eye: square, wide, scaled), :833-884 (tri, triu, tril), :886-926 (arange incl. empty
    ranges and a fractional step in int32), :928-953 (linspace), :955-985 (logspace), :987-1032 (geomspace), :143-175
    (bartlett), :4090-4116 (blackman)."""
    e3, e23, e35, e32 = run0(lambda: [J._raise(L.eye(3)).mul(1), J._raise(L.eye(2, 3)).mul(1), J._raise(L.eye(3, 5)).mul(-42), J._raise(L.eye(3, 2)).mul(1)])
    np.testing.assert_array_equal(e3.reshape(3, 3), np.eye(3))
    np.testing.assert_array_equal(e23.reshape(2, 3), np.eye(2, 3))
    np.testing.assert_array_equal(e35.reshape(3, 5), -42 * np.eye(3, 5))
    np.testing.assert_array_equal(e32.reshape(3, 2), np.eye(3, 2))
    t3, t24 = run0(lambda: [L.tri(3), L.tri(2, 4, 1)])
    np.testing.assert_array_equal(t3.reshape(3, 3), np.tri(3))
    np.testing.assert_array_equal(t24.reshape(2, 4), np.tri(2, 4, 1))
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    _, (up, lo) = _run_typed(lambda a: [L.triu(a), L.tril(a)], [x], [I32])
    np.testing.assert_array_equal(up.reshape(x.shape), np.triu(x))
    np.testing.assert_array_equal(lo.reshape(x.shape), np.tril(x))
    a5, a0, an, a2, a3, a3n, a3m = run0(lambda: [J._raise(c).add(0) for c in (L.arange(5), L.arange(0), L.arange(-10), L.arange(50, 60), L.arange(0, 10, 2), L.arange(10, 0, -2), L.arange(0, -10, -2))])
    assert a5.tolist() == [0, 1, 2, 3, 4] and a0.tolist() == [] and an.tolist() == [] and a2.tolist() == list(range(50, 60))
    assert a3.tolist() == [0, 2, 4, 6, 8] and a3n.tolist() == [10, 8, 6, 4, 2] and a3m.tolist() == [0, -2, -4, -6, -8]
    fi, ff = run0(lambda: [J._raise(L.arange(0, 1, 0.2)).add(0), J._raise(L.arange(0, 1, 0.2, F32)).add(0)])
    assert fi.tolist() == [0, 0, 0, 0, 0]
    np.testing.assert_allclose(ff, [0, 0.2, 0.4, 0.6, 0.8], rtol=1e-6)
    l5, l3, l2, l1, l50 = run0(lambda: [J._raise(L.linspace(0, 1, n)).add(0) for n in (5, 3, 2, 1, 50)])
    assert l5.tolist() == [0, 0.25, 0.5, 0.75, 1] and l3.tolist() == [0, 0.5, 1] and l2.tolist() == [0, 1] and l1.tolist() == [0]
    assert l50.shape == (50,) and l50[0] == 0 and l50[49] == 1 and abs(l50[25] - 25 / 49) < 1e-6
    g10, g2, gne, g50 = run0(lambda: [L.logspace(0, 2, 3), L.logspace(0, 3, 4, True, 2), L.logspace(0, 2, 4, False), L.logspace(0, 1)])
    np.testing.assert_allclose(g10, [1, 10, 100], rtol=1e-5)
    np.testing.assert_allclose(g2, [1, 2, 4, 8], rtol=1e-5)
    np.testing.assert_allclose(gne, [1, 10 ** 0.5, 10, 10 ** 1.5], rtol=1e-5)
    assert g50.shape == (50,) and abs(g50[0] - 1) < 1e-5 and abs(g50[49] - 10) < 1e-4
    q = run0(lambda: [L.geomspace(1, 1000, 4), L.geomspace(1, 256, 9), L.geomspace(1000, 1, 4), L.geomspace(-1000, -1, 4), L.geomspace(1, 10000, 4, False)])
    for got, want in zip(q, ([1, 10, 100, 1000], [2 ** i for i in range(9)], [1000, 100, 10, 1], [-1000, -100, -10, -1], [1, 10, 100, 1000])):
        np.testing.assert_allclose(got, want, rtol=1e-5)
    (gi,) = run0(lambda: L.geomspace(1, 16, 5, True, DType.Int32))
    assert gi.dtype == np.int32 and gi.tolist() == [1, 2, 4, 8, 16]
    for bad in ((0, 10), (1, 0), (-1, 10)):
        with pytest.raises(ValueError):
            L.geomspace(*bad, 5)
    b5, b4, b9, b1, b2 = run0(lambda: [J._raise(L.bartlett(n)).mul(1) for n in (5, 4, 9, 1, 2)])
    np.testing.assert_allclose(b5, [0, 0.5, 1, 0.5, 0], atol=1e-7)
    np.testing.assert_allclose(b4, [0, 2 / 3, 2 / 3, 0], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(b9, np.bartlett(9), atol=1e-6)
    assert b1.tolist() == [1] and b2.tolist() == [0, 0]
    (bs,) = run0(lambda: L.bartlett(5).sum())
    np.testing.assert_allclose(bs, [2], rtol=1e-6)
    k5, k10, k1 = run0(lambda: [J._raise(L.blackman(n)).mul(1) for n in (5, 10, 1)])
    np.testing.assert_allclose(k5, [0, 0.34, 1, 0.34, 0], atol=1e-6)
    np.testing.assert_allclose(k10, np.blackman(10), atol=1e-6)
    assert k1.tolist() == [1]
    for fn in (L.bartlett, L.blackman):
        for bad in (-1, 0.5):
            with pytest.raises(ValueError, match="non-negative integer"):
                fn(bad)


def test_diag_family_tables():
    """test/numpy.test.ts:592-628 (diag: build from 1-D, read from 2-D, off-diagonals), :630-682 (diagflat), :684-724
    (diagIndices, also used to gather the diagonal), :726-774 (diagonal over chosen axes, trace), :776-831
    (diagIndicesFrom)."""
    _, (d,) = run(lambda v: L.diag(v), f32([1, 2, 3]))
    np.testing.assert_array_equal(d.reshape(3, 3), np.diag([1, 2, 3]))
    m = f32(np.arange(1, 10).reshape(3, 3))
    _, (d0, d1) = run(lambda a: [L.diag(a).mul(1), L.diag(a, 1).mul(1)], m)
    assert d0.tolist() == [1, 5, 9] and d1.tolist() == [2, 6]
    _, (u, l) = run(lambda v: [L.diag(v, 1), L.diag(v, -2)], f32([1, 2]))
    np.testing.assert_array_equal(u.reshape(3, 3), np.diag([1, 2], 1))
    np.testing.assert_array_equal(l.reshape(4, 4), np.diag([1, 2], -2))
    _, (f0, f1) = run(lambda a: [L.diagflat(a), L.diagflat(a, 1)], f32([[1, 2], [3, 4]]))
    np.testing.assert_array_equal(f0.reshape(4, 4), np.diagflat([[1, 2], [3, 4]]))
    np.testing.assert_array_equal(f1.reshape(5, 5), np.diagflat([[1, 2], [3, 4]], 1))
    _, (fm,) = run(lambda a: L.diagflat(a, -1), f32([1, 2]))
    np.testing.assert_array_equal(fm.reshape(3, 3), np.diagflat([1, 2], -1))
    rows, cols = L.diagIndices(3)
    assert rows is cols and rows.dtype == I32 and len(L.diagIndices(2, 3)) == 3 and L.diagIndices(3, 0) == []
    r3, = run0(lambda: J._raise(rows).add(0))
    assert r3.tolist() == [0, 1, 2]
    _, (g,) = run(lambda a: J.gather(a, [J._raise(i) for i in L.diagIndicesFrom(a)], [0, 1], 0), m)
    assert g.tolist() == [1, 5, 9]
    with pytest.raises(ValueError, match="nonnegative integer"):
        L.diagIndices(-1)
    with pytest.raises(ValueError, match="nonnegative integer"):
        L.diagIndices(3, -1)
    with pytest.raises(ValueError, match="all dimensions of input must be equal"):
        J.jit(lambda a: L.diagIndicesFrom(a), [ShapedArray((3, 4), F32)])
    with pytest.raises(ValueError, match="at least 2D"):
        J.jit(lambda a: L.diagIndicesFrom(a), [ShapedArray((3,), F32)])
    a = f32(np.arange(12).reshape(3, 2, 2))
    _, (p, q, r, s) = run(lambda t: [L.diagonal(t, 0, 1, 2).mul(1), L.diagonal(t, 0, 0, 1).mul(1), L.diagonal(t, 1, 0, 1).mul(1), L.diagonal(t, 1, 1, 0).mul(1)], a)
    np.testing.assert_array_equal(p.reshape(3, 2), np.diagonal(a, 0, 1, 2))
    np.testing.assert_array_equal(q.reshape(2, 2), np.diagonal(a, 0, 0, 1))
    np.testing.assert_array_equal(r.reshape(2, 1), np.diagonal(a, 1, 0, 1))
    np.testing.assert_array_equal(s.reshape(2, 2), np.diagonal(a, 1, 1, 0))
    _, (t0, t1) = run(lambda t: [L.trace(t), L.trace(t, 1)], f32(np.arange(9).reshape(3, 3)))
    assert t0.tolist() == [12] and t1.tolist() == [6]


def test_where_select_equality_and_membership_tables():
    """test/numpy.test.ts:1034-1075 (where incl. scalar broadcasting), :1077-1164 (select: first match wins, default,
    numeric conditions, broadcasting, dtype promotion, errors), :1166-1183 (equal / notEqual), :1185-1247 (arrayEqual
    with and without equalNaN, arrayEquiv), :1249-1335 (isin: invert, flattened test set, empty operands, NaN)."""
    x, y, z = f32([1, 2, 3]), f32([4, 5, 6]), np.array([1, 0, 1], np.int32)
    _, (w,) = _run_typed(lambda a, b, c: J.where(c, a, b), [x, y, z], [F32, F32, BOOL])
    assert w.tolist() == [1, 5, 3]
    _, (w1, w2, w3) = _run_typed(lambda c, v: [J.where(c, 1, 3), J.where(False, 1, v), J.where(True, 7, v)], [np.array([1, 0, 1, 1], np.int32), f32([10, 11, 12, 13])], [BOOL, F32])
    assert w1.tolist() == [1, 3, 1, 1] and w2.tolist() == [10, 11, 12, 13] and w3.tolist() == [7, 7, 7, 7]
    ar = np.arange(6, dtype=np.int32)
    _, (s1, s2, s3) = _run_typed(lambda a: [L.select([J.less(a, 3), J.greater(a, 3)], [J.neg(a), L.square(a)], 42),
                                            L.select([J.lessEqual(a, 4), J.greater(a, 3)], [a, L.square(a)], 55),
                                            L.select([J.greater(a, 1)], [a])], [ar], [I32])
    assert s1.tolist() == [0, -1, -2, 42, 16, 25] and s2.tolist() == [0, 1, 2, 3, 4, 25] and s3.tolist() == [0, 0, 2, 3, 4, 5]
    _, (s4,) = run(lambda p, q: L.select([p, q], [10, 20], 30), f32([0, 1, -2]), f32([1, 0, 0]))
    assert s4.tolist() == [20, 10, 10]
    _, (s5,) = _run_typed(lambda c, d, v: L.select([c, d], [1, v], -1), [np.array([[1, 0], [0, 1]], np.int32), np.array([0, 1], np.int32), f32([[10], [20]])], [BOOL, BOOL, F32])
    assert s5.tolist() == [1, 10, -1, 1]
    prog, (s6,) = _run_typed(lambda a, c: L.select([J.less(a, 1)], [c], 2), [np.arange(3, dtype=np.int32), f32([0.5, 1.5, 2.5])], [I32, F32])
    assert s6.dtype == np.float32 and s6.tolist() == [0.5, 2, 2]
    with pytest.raises(ValueError, match="condlist must have length equal to choicelist"):
        L.select([True], [])
    with pytest.raises(ValueError, match="non-empty"):
        L.select([], [])
    _, (eq, ne) = run(lambda a, b: [J.equal(a, b), J.notEqual(a, b)], f32([1, 2, 3, 4]), f32([4, 5, 3, 4]))
    assert eq.tolist() == [0, 0, 1, 1] and ne.tolist() == [1, 1, 0, 0]
    nan = np.nan
    _, (e1, e2, e3, e4) = run(lambda a, b, c, d: [L.arrayEqual(a, a.mul(1)), L.arrayEqual(a, b), L.arrayEqual(c, d), L.arrayEqual(c, d, equalNaN=True)], f32([1, 2, 3]), f32([1, 2, 4]), f32([1, nan]), f32([1, nan]))
    assert (e1.tolist(), e2.tolist(), e3.tolist(), e4.tolist()) == ([1], [0], [0], [1])
    _, (e5,) = run(lambda a, b: J._raise(L.arrayEqual(a, b)).add(False), f32([1, 2, 3]), f32([1, 2]))
    assert e5.tolist() == [0]
    _, (q1, q2, q3) = run(lambda a, b, c: [L.arrayEquiv(a, c), L.arrayEquiv(b, c), J._raise(L.arrayEquiv(c, c.reshape([1, 2]).sum(1))).add(False)], f32([[1, 2], [1, 2]]), f32([[1, 2], [3, 4]]), f32([1, 2]))
    assert q1.tolist() == [1] and q2.tolist() == [0]
    _, (q4,) = run(lambda a, b: J._raise(L.arrayEquiv(a, b)).add(False), f32([1, 2, 3]), f32([1, 2]))
    assert q4.tolist() == [0]
    el, te = f32([[0, 2], [4, 6]]), f32([1, 2, 4, 8])
    _, (i1, i2) = run(lambda a, b: [L.isin(a, b), L.isin(a, b, invert=True)], el, te)
    assert i1.tolist() == [0, 1, 1, 0] and i2.tolist() == [1, 0, 0, 1]
    _, (i3,) = run(lambda a, b: L.isin(a, b), f32([1, 2, 3, 4]), f32([[1, 3], [5, 7]]))
    assert i3.tolist() == [1, 0, 1, 0]
    _, (i4, i5) = run(lambda a, b: [J._raise(L.isin(a, b)).add(False), L.isin(a, b, invert=True)], f32([1, 2]), f32([]))
    assert i4.tolist() == [0, 0] and i5.tolist() == [1, 1]
    _, (i6,) = run(lambda a, b: L.isin(a, b), np.zeros((2, 0), np.float32), f32([1]))
    assert i6.tolist() == []
    _, (i7,) = run(lambda a, b: L.isin(a, b), f32([nan, 1]), f32([nan, 1]))
    assert i7.tolist() == [0, 1]
    _, (i8,) = _run_typed(lambda a, b: L.isin(a, b), [np.array([1, 2], np.int32), f32([2.0, 3.5])], [I32, F32])
    assert i8.tolist() == [0, 1]


def _i32(x):
    return np.asarray(x, dtype=np.int32)


def _parts(fn, x, dtypes=None):
    """Run a function returning a list of pieces of one int32 array; pieces come back as flat lists."""
    _, outs = _run_typed(fn, [x], [I32])
    return [o.tolist() for o in outs]


def test_pad_and_split_family_tables():
    """test/numpy.test.ts:3105-3185 (pad: one width, per-axis pairs, {axis: pair}, arity errors, after a prior op),
    :3187-3288 (split: equal parts, along an axis, at indices incl. empty sections, 20 parts), :3290-3340 (arraySplit),
    :3342-3391 (unstack), :3393-3572 (dsplit / hsplit / vsplit)."""
    _, (p1,) = run(lambda a: L.pad(a, 1), f32([1, 2, 3]))
    _, (p2, p3) = run(lambda a: [L.pad(a, 1), L.pad(a.add(2), 1)], f32([[1, 2], [3, 4]]))
    assert p1.tolist() == [0, 1, 2, 3, 0]
    np.testing.assert_array_equal(p2.reshape(4, 4), np.pad([[1, 2], [3, 4]], 1))
    np.testing.assert_array_equal(p3.reshape(4, 4), np.pad(np.array([[3, 4], [5, 6]]), 1))
    _, (p4,) = run(lambda a: L.pad(a, [[1, 2], [3, 0]]), f32([[1]]))
    np.testing.assert_array_equal(p4.reshape(4, 4), np.pad([[1]], [[1, 2], [3, 0]]))
    seen = {}
    J.jit(lambda a: seen.setdefault("y", L.pad(a, {1: (0, 2), -1: (3, 0)})), [ShapedArray((2, 3, 4, 5), F32)])
    assert tuple(seen["y"].shape) == (2, 5, 4, 8)
    for bad in ([], [[0, 1], [1, 2]]):
        with pytest.raises((ValueError, TypeError)):
            J.jit(lambda a: L.pad(a, bad), [ShapedArray((1, 2, 3), F32)])
    J.jit(lambda a: L.pad(a, [[0, 1]]), [ShapedArray((1, 2, 3), F32)])
    x6, x10, x12 = _i32(np.arange(6)), _i32(np.arange(10)), _i32(np.arange(12))
    assert _parts(lambda a: L.split(a, 3), x6) == [[0, 1], [2, 3], [4, 5]]
    for shape, ax in (([4, 3], 0), ([3, 4], 1), ([3, 4], -1)):
        m = x12.reshape(shape)
        got = _parts(lambda a: L.split(a, 2, ax), m)
        assert got == [p.ravel().tolist() for p in np.split(m, 2, ax)]
    assert _parts(lambda a: L.split(a, [3, 7]), x10) == [[0, 1, 2], [3, 4, 5, 6], [7, 8, 9]]
    assert _parts(lambda a: L.split(a, [0, 0, 3]), _i32(np.arange(5))) == [[], [], [0, 1, 2], [3, 4]]
    for n in (2, 3):
        with pytest.raises(ValueError):
            J.jit(lambda a: L.split(a, n), [ShapedArray((5,), I32)])
    assert _parts(lambda a: (lambda ab: [J.add(ab[0], ab[1])])(L.split(a, 2)), x6) == [[3, 5, 7]]
    assert _parts(lambda a: L.split(a, 20), _i32(np.arange(20))) == [[i] for i in range(20)]
    assert _parts(lambda a: L.arraySplit(a, 3), _i32(np.arange(8))) == [[0, 1, 2], [3, 4, 5], [6, 7]]
    assert _parts(lambda a: L.arraySplit(a, 5), _i32(np.arange(3))) == [[0], [1], [2], [], []]
    assert _parts(lambda a: L.arraySplit(a, 3, -1), x10.reshape(2, 5)) == [[0, 1, 5, 6], [2, 3, 7, 8], [4, 9]]
    assert _parts(lambda a: L.arraySplit(a, [2, 5]), _i32(np.arange(7))) == [[0, 1], [2, 3, 4], [5, 6]]
    assert _parts(lambda a: [p.add(0) for p in L.arraySplit(a, [])], _i32(np.arange(5))) == [[0, 1, 2, 3, 4]]
    assert _parts(lambda a: [L.concatenate(list(reversed(L.arraySplit(a, 3))))], _i32(np.arange(8))) == [[6, 7, 3, 4, 5, 0, 1, 2]]
    m32 = x6.reshape(3, 2)
    assert _parts(lambda a: L.unstack(a), m32) == [[0, 1], [2, 3], [4, 5]]
    assert _parts(lambda a: L.unstack(a, -1), m32) == [[0, 2, 4], [1, 3, 5]]
    assert _parts(lambda a: L.unstack(a), _i32([5, 7, 9])) == [[5], [7], [9]]
    assert _parts(lambda a: [L.stack(L.unstack(a, 1), 1)], x12.reshape(2, 3, 2)) == [x12.tolist()]
    assert _parts(lambda a: [L.stack(list(reversed(L.unstack(a))))], m32) == [[4, 5, 2, 3, 0, 1]]
    with pytest.raises(ValueError):
        J.jit(lambda a: L.unstack(a), [ShapedArray((), F32)])
    assert J.jit(lambda a: L.unstack(a) + [a], [ShapedArray((0, 3), F32)]) is not None
    x16 = _i32(np.arange(16)).reshape(2, 2, 4)
    assert _parts(lambda a: L.dsplit(a, 2), x16) == [p.ravel().tolist() for p in np.dsplit(x16, 2)]
    x8 = _i32(np.arange(8)).reshape(1, 2, 4)
    assert _parts(lambda a: L.dsplit(a, [1, 3]), x8) == [[0, 4], [1, 2, 5, 6], [3, 7]]
    assert _parts(lambda a: (lambda ab: [L.concatenate([ab[1], ab[0]], 2)])(L.dsplit(a, 2)), x8) == [[2, 3, 0, 1, 6, 7, 4, 5]]
    with pytest.raises(ValueError, match="3 or more dimensions"):
        J.jit(lambda a: L.dsplit(a, 3), [ShapedArray((2, 3), F32)])
    assert _parts(lambda a: L.hsplit(a, 2), x12.reshape(3, 4)) == [[0, 1, 4, 5, 8, 9], [2, 3, 6, 7, 10, 11]]
    assert _parts(lambda a: L.hsplit(a, 3), x6) == [[0, 1], [2, 3], [4, 5]]
    assert _parts(lambda a: L.hsplit(a, 2), _i32(np.arange(8)).reshape(2, 2, 2)) == [[0, 1, 4, 5], [2, 3, 6, 7]]
    assert _parts(lambda a: L.hsplit(a, [1, 4]), x12.reshape(2, 6)) == [[0, 6], [1, 2, 3, 7, 8, 9], [4, 5, 10, 11]]
    with pytest.raises(ValueError):
        J.jit(lambda a: L.hsplit(a, 2), [ShapedArray((2, 5), F32)])
    with pytest.raises(ValueError, match="1 or more dimensions"):
        J.jit(lambda a: L.hsplit(a, 1), [ShapedArray((), F32)])
    assert _parts(lambda a: L.vsplit(a, 2), x12.reshape(4, 3)) == [list(range(6)), list(range(6, 12))]
    assert _parts(lambda a: L.vsplit(a, [1, 3]), x12.reshape(4, 3)) == [[0, 1, 2], [3, 4, 5, 6, 7, 8], [9, 10, 11]]
    assert _parts(lambda a: (lambda ab: [J.add(ab[0], ab[1])])(L.vsplit(a, 2)), _i32(np.arange(8)).reshape(4, 2)) == [[4, 6, 8, 10]]
    with pytest.raises(ValueError):
        J.jit(lambda a: L.vsplit(a, 2), [ShapedArray((5, 3), F32)])


def test_joins_repeats_and_reshapes_tables():
    """test/numpy.test.ts:3574-3625 (concatenate, shape mismatch, stack / vstack / hstack / dstack of scalars and
    vectors), :4168-4203 (repeat), :4205-4240 (tile), :4458-4526 (expandDims), :4914-4949 (append), :363-413 (ediff1d),
    :2054-2095 (meshgrid), :2097-2160 (indices)."""
    a, b = f32([1, 2, 3]), f32([4, 5, 6])
    _, (c,) = run(lambda p, q: L.concatenate([p, q]), a, b)
    assert c.tolist() == [1, 2, 3, 4, 5, 6]
    two = [ShapedArray((2, 3), F32), ShapedArray((3, 2), F32)]
    for ax in (0, 1):
        with pytest.raises(ValueError):
            J.jit(lambda p, q: L.concatenate([p, q], ax), two)
    J.jit(lambda p, q: L.concatenate([p, q.transpose()]), two)
    _, (cj,) = run(lambda p, q, r: L.concatenate([J.flip(p, None), q, r]), f32([1, 2]), f32([3, 4]), f32([5]))
    assert cj.tolist() == [2, 1, 3, 4, 5]
    s = float  # numbers become 0-d arrays, as the reference's fudgeArray makes of them
    st0, st1, vs, hs, ds = run0(lambda: [L.stack([s(2), s(3)]), L.stack([s(2), s(3)], -1), L.vstack([s(1), s(2), s(3)]), L.hstack([s(1), s(2), s(3)]), L.dstack([s(1), s(2), s(3)])])
    assert st0.tolist() == [2, 3] and st1.tolist() == [2, 3] and vs.tolist() == [1, 2, 3] and hs.tolist() == [1, 2, 3] and ds.tolist() == [1, 2, 3]
    for ax in (1, 2):
        with pytest.raises((ValueError, IndexError)):
            J.jit(lambda: L.stack([s(2), s(3)], ax), [])
    one = np.ones(3, np.float32)
    prog, (v2, h2, d2, c2) = run(lambda p, q: [L.vstack([p, q]), L.hstack([p, q]), L.dstack([p, q]), L.columnStack([p, q])], a, one)
    np.testing.assert_array_equal(v2.reshape(2, 3), np.vstack([a, one]))
    np.testing.assert_array_equal(h2, np.hstack([a, one]))
    np.testing.assert_array_equal(d2.reshape(1, 3, 2), np.dstack([a, one]))
    np.testing.assert_array_equal(c2.reshape(3, 2), np.column_stack([a, one]))
    m = f32([[1, 2], [3, 4]])
    _, (r1, r2, r3, r4) = run(lambda p, q: [L.repeat(p, 2), L.repeat(q, 2, 0), L.repeat(q, 3, 1), L.repeat(q, 2)], a, m)
    assert r1.tolist() == [1, 1, 2, 2, 3, 3] and r4.tolist() == [1, 1, 2, 2, 3, 3, 4, 4]
    np.testing.assert_array_equal(r2.reshape(4, 2), np.repeat(m, 2, 0))
    np.testing.assert_array_equal(r3.reshape(2, 6), np.repeat(m, 3, 1))
    _, (t1, t2, t3, t4) = run(lambda p, q: [L.tile(p, 2), L.tile(q, [2, 1]), L.tile(q, 3), L.tile(p, [2, 2])], a, m)
    assert t1.tolist() == [1, 2, 3, 1, 2, 3]
    np.testing.assert_array_equal(t2.reshape(4, 2), np.tile(m, [2, 1]))
    np.testing.assert_array_equal(t3.reshape(2, 6), np.tile(m, 3))
    np.testing.assert_array_equal(t4.reshape(2, 6), np.tile(a, [2, 2]))
    shapes = {}
    def ed(p, q):
        outs = [L.expandDims(p, 0), L.expandDims(p, 1), L.expandDims(p, -1), L.expandDims(p, [0, 2]), L.expandDims(q, 0), L.expandDims(q, 2)]
        shapes["s"] = [tuple(o.shape) for o in outs]
        return [o.mul(1) for o in outs]
    run(ed, a, m)
    assert shapes["s"] == [(1, 3), (3, 1), (3, 1), (1, 3, 1), (1, 2, 2), (2, 2, 1)]
    for bad in (3, -4, [0, 0]):
        with pytest.raises(ValueError):
            J.jit(lambda p: L.expandDims(p, bad), [ShapedArray((3,), F32)])
    _, (ap, ap0, ap1) = run(lambda p, q, r: [L.append(p, q), L.append(p, q, 0), L.append(p, r, 1)], m, f32([[5, 6]]), f32([[5], [6]]))
    assert ap.tolist() == [1, 2, 3, 4, 5, 6] and ap0.tolist() == [1, 2, 3, 4, 5, 6] and ap1.tolist() == [1, 2, 5, 3, 4, 6]
    x = f32([1, 2, 4, 7, 0])
    _, (e1, e2, e3) = run(lambda p, q, r: [L.ediff1d(p), L.ediff1d(q), L.ediff1d(p, toBegin=-99, toEnd=r)], x, f32([[1, 2, 4], [1, 6, 24]]), f32([88, 99]))
    assert e1.tolist() == [1, 2, 3, -7] and e2.tolist() == [1, 2, -3, 5, 18] and e3.tolist() == [-99, 1, 2, 3, -7, 88, 99]
    prog, (e4,) = _run_typed(lambda p, r: L.ediff1d(p, toBegin=-99.5, toEnd=r), [_i32(np.arange(4)), f32([1.5, 2.5])], [I32, F32])
    assert e4.dtype == np.int32 and e4.tolist() == [-99, 1, 1, 1, 1, 2]
    _, (e5, e6) = run(lambda p: [L.ediff1d(p), L.ediff1d(p, toBegin=1, toEnd=2)], f32([5]))
    assert e5.tolist() == [] and e6.tolist() == [1, 2]
    X, Y = f32([1, 2, 3]), f32([4, 5])
    _, (gx, gy, ix, iy) = run(lambda p, q: [o.mul(1) for o in L.meshgrid([p, q]) + L.meshgrid([p, q], "ij")], X, Y)
    wx, wy = np.meshgrid(X, Y)
    vx, vy = np.meshgrid(X, Y, indexing="ij")
    for got, want in ((gx, wx), (gy, wy), (ix, vx), (iy, vy)):
        np.testing.assert_array_equal(got.reshape(want.shape), want)
    prog3 = J.jit(lambda p, q, r: [o.mul(1) for o in L.meshgrid([p, q, r])], [ShapedArray((2,), F32), ShapedArray((3,), F32), ShapedArray((4,), F32)])
    g23, g4, sr, sc, gf = run0(lambda: [L.indices([2, 3]), L.indices([4])] + [o.add(0) for o in L.indices([2, 3], sparse=True)] + [L.indices([2, 2], F32)])
    np.testing.assert_array_equal(g23.reshape(2, 2, 3), np.indices([2, 3]))
    assert g23.dtype == np.int32 and g4.tolist() == [0, 1, 2, 3] and sr.tolist() == [0, 1] and sc.tolist() == [0, 1, 2]
    assert gf.dtype == np.float32 and gf.tolist() == np.indices([2, 2]).ravel().tolist()
    assert L.indices([], sparse=True) == [] and tuple(L.indices([]).shape) == (0,)
    for bad in ([2, -1], [1.5]):
        with pytest.raises(ValueError, match="non-negative integers"):
            L.indices(bad)


def test_polynomial_convolution_and_statistics_tables():
    """test/numpy.test.ts:3680-3713 (vander), :3715-3779 (polyval: scalar and array points, dtype kept, empty and
    batched coefficients), :3781-3944 (polyadd / polysub: alignment, empty operands, batches, promotion), :3946-4005
    (polymul), :4343-4378 (convolve / correlate in the three modes), :522-561 (cross), :4242-4290 (var, std, cov)."""
    _, (v1, v2) = run(lambda a, b: [L.vander(a), L.vander(b, 4, increasing=True)], f32([0, 2, 3]), f32([1, 2, 3]))
    np.testing.assert_allclose(v1.reshape(3, 3), np.vander([0, 2, 3]), rtol=1e-6)
    np.testing.assert_allclose(v2.reshape(3, 4), np.vander([1, 2, 3], 4, increasing=True), rtol=1e-6)
    seen = {}
    J.jit(lambda a: seen.setdefault("v", L.vander(a, 0)), [ShapedArray((3,), F32)])
    assert tuple(seen["v"].shape) == (3, 0)
    with pytest.raises(ValueError, match="input must be 1D"):
        J.jit(lambda a: L.vander(a), [ShapedArray((2, 2), F32)])
    p = f32([3, 0, 1])
    _, (pv0, pv1) = run(lambda c, x0, x1: [L.polyval(c, x0), L.polyval(c, x1)], p, f32(5).reshape(()), f32([0, 1, 2]))
    assert pv0.tolist() == [76]
    np.testing.assert_allclose(pv1, [1, 4, 13], rtol=1e-6)
    _, (pi,) = _run_typed(lambda c, x: L.polyval(c, x), [_i32([1, 2]), _i32([3, 4])], [I32, I32])
    assert pi.dtype == np.int32 and pi.tolist() == [5, 6]
    _, (pm,) = _run_typed(lambda c, x: L.polyval(c, x), [_i32([1, 2]), f32([0.5, 1.5])], [I32, F32])
    assert pm.dtype == np.float32 and pm.tolist() == [2.5, 3.5]
    _, (pc,) = run(lambda c, x: L.polyval(c, x), f32([7]), np.ones((2, 2), np.float32))
    assert pc.tolist() == [7, 7, 7, 7]
    _, (pb,) = run(lambda c, x: L.polyval(c, x), f32([[1, 2], [0, 3], [4, 5]]), f32([2, 3]))
    np.testing.assert_allclose(pb, [8, 32], rtol=1e-6)
    with pytest.raises(ValueError, match="at least one dimension"):
        J.jit(lambda c, x: L.polyval(c, x), [ShapedArray((), F32), ShapedArray((), F32)])
    a1, a2, lo, sh = f32([1, 2, 3]), f32([4, 5, 6]), f32([1, 2, 3, 4]), f32([10, 20])
    _, (s0, s1, s2, d0, d1, d2) = run(lambda p, q, r, t: [L.polyadd(p, q), L.polyadd(r, t), L.polyadd(t, r), L.polysub(p, q), L.polysub(r, t), L.polysub(t, r)], a1, a2, lo, sh)
    assert s0.tolist() == [5, 7, 9] and s1.tolist() == [1, 2, 13, 24] and s2.tolist() == [1, 2, 13, 24]
    assert d0.tolist() == [-3, -3, -3] and d1.tolist() == [1, 2, -7, -16] and d2.tolist() == [-1, -2, 7, 16]
    _, (se, de, de2) = run(lambda p, q: [L.polyadd(p, q), L.polysub(p, q), L.polysub(q, p)], f32([1, 2]), f32([]))
    assert se.tolist() == [1, 2] and de.tolist() == [1, 2] and de2.tolist() == [-1, -2]
    _, (sp, dp) = run(lambda p, q: [L.polyadd(p, q), L.polysub(p, q)], a1, f32([0.5, 1.5]))
    np.testing.assert_allclose(sp, [1, 2.5, 4.5])
    np.testing.assert_allclose(dp, [1, 1.5, 1.5])
    b1, b2, bt = f32([[2, 3, 1]]), f32([[5, 7, 3], [8, 2, 6]]), f32([[5, 7, 9], [8, 6, 4]])
    _, (sb, db, sc, dc) = run(lambda p, q, r, t: [L.polyadd(p, q), L.polysub(p, q), L.polyadd(r, t), L.polysub(r, t)], b1, b2, bt, f32([2]))
    assert sb.tolist() == [5, 7, 3, 10, 5, 7] and db.tolist() == [-5, -7, -3, -6, 1, -5]
    assert sc.tolist() == [5, 7, 9, 10, 8, 6] and dc.tolist() == [5, 7, 9, 6, 4, 2]
    for fn in (L.polyadd, L.polysub):
        with pytest.raises(ValueError):
            J.jit(lambda p, q: fn(p, q), [ShapedArray((3,), F32), ShapedArray((2, 3), F32)])
        with pytest.raises(ValueError, match="at least 1D"):
            J.jit(lambda p, q: fn(p, q), [ShapedArray((), F32), ShapedArray((2,), F32)])
    _, (m0, m1, m2, m3) = run(lambda p, q, r, t: [L.polymul(p, q), L.polymul(r, t), L.polymul(t, r), L.polymul(J.shrink(r, [(1, 2)]), J.shrink(t, [(0, 1)]))], f32([2, 1, 0]), f32([0, 5, 3]), f32([1, 2]), f32([3, 4, 5]))
    assert m0.tolist() == [0, 10, 11, 3, 0] and m1.tolist() == [3, 10, 13, 10] and m2.tolist() == [3, 10, 13, 10] and m3.tolist() == [6]
    _, (mi,) = _run_typed(lambda p, q: L.polymul(p, q), [_i32([1, 2, 3]), _i32([4, 5, 6])], [I32, I32])
    assert mi.dtype == np.float32 and mi.tolist() == [4, 13, 28, 27, 18]
    _, (z0, z1, z2) = run(lambda p, q: [L.polymul(p, q), L.polymul(q, p), L.polymul(p, p)], f32([]), f32([1, 2]))
    assert z0.tolist() == [0, 0] and z1.tolist() == [0, 0] and z2.tolist() == [0]
    for shp in ((), (2, 2)):
        with pytest.raises(ValueError, match="both inputs must be 1D arrays"):
            J.jit(lambda p, q: L.polymul(p, q), [ShapedArray(shp, F32), ShapedArray((2,), F32)])
    x, y = f32([1, 2, 3, 2, 1]), f32([4, 1, 2])
    _, (cf, cs, cv) = run(lambda p, q: [L.convolve(p, q), L.convolve(p, q, "same"), L.convolve(p, q, "valid")], x, y)
    assert cf.tolist() == [4, 9, 16, 15, 12, 5, 2] and cs.tolist() == [9, 16, 15, 12, 5] and cv.tolist() == [16, 15, 12]
    _, (rv, rf, rs, rsw) = run(lambda p, q: [L.correlate(p, q), L.correlate(p, q, "full"), L.correlate(p, q, "same"), L.correlate(q, p, "full")], x, f32([4, 5, 6]))
    assert rv.tolist() == [32, 35, 28] and rf.tolist() == [6, 17, 32, 35, 28, 13, 4] and rs.tolist() == [17, 32, 35, 28, 13]
    assert rsw.tolist() == np.correlate([4, 5, 6], [1, 2, 3, 2, 1], "full").tolist()
    _, (k1, k2) = run(lambda p, q: [L.correlate(p, q, "full"), L.convolve(p, q, "full")], x, f32([4, 5, 4]))
    assert k1.tolist() == [4, 13, 26, 31, 26, 13, 4] and k2.tolist() == k1.tolist()
    _, (c2,) = run(lambda p, q: L.cross(p, q), f32([1, 2]), f32([3, 4]))
    _, (c3,) = run(lambda p, q: L.cross(p, q), f32([1, 2, 3]), f32([4, 5, 6]))
    A, B = f32([[1, 2, 3], [3, 4, 3]]), f32([[2, 3, 2], [4, 5, 6]])
    _, (cb, ca, cm) = run(lambda p, q: [L.cross(p, q), L.cross(p, q, axis=0), L.cross(J.shrink(p, [(0, 2), (0, 2)]), q)], A, B)
    assert c2.tolist() == [-2] and c3.tolist() == [-3, 6, -3] and cb.tolist() == [-5, 4, -1, 9, -6, -1] and ca.tolist() == [-2, -2, 12]
    np.testing.assert_array_equal(cm.reshape(2, 3), np.cross(np.pad(A[:, :2], [(0, 0), (0, 1)]), B))
    _, (vr, sd) = run(lambda p: [L.var_(p), L.std(p)], f32([1, 2, 3, 4]))
    np.testing.assert_allclose(vr, [1.25], rtol=1e-6)
    np.testing.assert_allclose(sd, [math.sqrt(1.25)], rtol=1e-6)
    _, (v1c, v2c, v3c, cc) = run(lambda p, q, r, t: [L.cov(p), L.cov(q), L.cov(r, t), L.corrcoef(q)], f32([[0, 1, 2], [0, 1, 2]]), f32([[-1, 0, 1], [1, 0, -1]]), f32([-1, 0, 1]), f32([1, 0, -1]))
    np.testing.assert_allclose(v1c, [1, 1, 1, 1], rtol=1e-6)
    np.testing.assert_allclose(v2c, [1, -1, -1, 1], rtol=1e-6)
    np.testing.assert_allclose(v3c, [1, -1, -1, 1], rtol=1e-6)
    np.testing.assert_allclose(cc, [1, -1, -1, 1], rtol=1e-6)


def test_unwrap_tables():
    """test/numpy.test.ts:2684-2801: the NumPy docs example, custom periods, a larger discont, the dtype-rounded period,
    other axes (also an interior one), deltas of exactly half a period, int32 input, short inputs."""
    pi = math.pi
    _, (u1,) = run(lambda a: L.unwrap(a), f32([0, pi / 4, pi / 2, 3 * pi / 4 + pi, 2 * pi]))
    np.testing.assert_allclose(u1, [0, pi / 4, pi / 2, -pi / 4, 0], atol=1e-5)
    _, (u2, u3) = run(lambda a, b: [L.unwrap(a, None, -1, 4), L.unwrap(b, None, -1, 4)], f32([0, 1, 2, -1, 0]), f32([2, 3, 4, 5, 2, 3, 4, 5]))
    np.testing.assert_allclose(u2, [0, 1, 2, 3, 4], rtol=1e-6)
    np.testing.assert_allclose(u3, [2, 3, 4, 5, 6, 7, 8, 9], rtol=1e-6)
    _, (u4, u5) = run(lambda a: [L.unwrap(a), L.unwrap(a, 4)], f32([0, 3.5]))
    np.testing.assert_allclose(u4, [0, 3.5 - 2 * pi], rtol=1e-5)
    np.testing.assert_allclose(u5, [0, 3.5], rtol=1e-6)
    _, (u6,) = run(lambda a: L.unwrap(a, None, -1, 3.5e38), f32([0, 3e38]))
    assert u6.tolist() == [0, float(np.float32(3e38))]
    x = f32([[0, 2 * pi + 0.1, 4 * pi + 0.2], [0.5, 2 * pi + 0.6, 4 * pi + 0.7]])
    _, (u7, u8, u9) = run(lambda a: [L.unwrap(a), L.unwrap(a.transpose(), None, 0), L.unwrap(a.transpose().reshape([1, 1, 3, 2]), None, 2)], x)
    np.testing.assert_allclose(u7.reshape(2, 3), [[0, 0.1, 0.2], [0.5, 0.6, 0.7]], atol=1e-5)
    np.testing.assert_allclose(u8.reshape(3, 2), [[0, 0.5], [0.1, 0.6], [0.2, 0.7]], atol=1e-5)
    np.testing.assert_allclose(u9, u8, atol=1e-6)
    _, (up, dn) = run(lambda a: [L.unwrap(a), L.unwrap(a.mul(-1))], f32([0, pi, 2 * pi]))
    np.testing.assert_allclose(up, [0, pi, 2 * pi], atol=1e-5)
    np.testing.assert_allclose(dn, [0, -pi, -2 * pi], atol=1e-5)
    _, (ui,) = _run_typed(lambda a: L.unwrap(a, None, -1, 4), [_i32([0, 1, 2, -1, 0])], [I32])
    assert ui.dtype == np.float32
    np.testing.assert_allclose(ui, [0, 1, 2, 3, 4], rtol=1e-6)
    _, (us, ue) = run(lambda a, b: [L.unwrap(a).mul(1), L.unwrap(b).mul(1)], f32([1.5]), f32([]))
    assert us.tolist() == [1.5] and ue.tolist() == []
    _, (uj,) = run(lambda a: L.unwrap(a), f32([0, pi - 0.1, 2 * pi + 0.5]))
    np.testing.assert_allclose(uj, [0, pi - 0.1, 0.5], atol=1e-5)


def test_reductions_views_dot_and_sort_tables():
    """test/numpy.test.ts:24-42 (sum over several axes, keepdims, no axes), :221-257 (mean promotes int32 and bool),
    :1337-1425 (transpose, swapaxes, reshape and its errors), :1683-1796 (dot: scalars, 1-D, 2-D, the N-D shape rule,
    1-784-10, an affine map against a double loop), :3041-3103 (min / max), :4007-4033 (argmax, flattened by default),
    :4585-4629 (applyOverAxes), :4631-4802 (sort / argsort: axes, NaN last, integer and bool dtypes, empty rows, 8192
    elements, stability)."""
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    seen = {}
    def sums(a):
        seen["k"] = a.sum([0, 2], keepdims=True)
        return [a.sum([0, 2]), seen["k"], a.sum([])]
    _, (s1, s2, s3) = _run_typed(sums, [x], [I32])
    assert s1.tolist() == [60, 92, 124] and s2.tolist() == [60, 92, 124] and tuple(seen["k"].shape) == (1, 3, 1) and s3.tolist() == x.ravel().tolist()
    _, (mi,) = _run_typed(lambda a: a.mean(), [_i32([1, 2, 3, 4])], [I32])
    _, (mb,) = _run_typed(lambda a: a.mean(), [_i32([1, 0, 1])], [BOOL])
    _, (mr,) = _run_typed(lambda a: a.mean(1), [_i32([[1, 2, 3], [4, 5, 6]])], [I32])
    assert mi.dtype == np.float32 and abs(mi[0] - 2.5) < 1e-6 and mb.dtype == np.float32 and abs(mb[0] - 2 / 3) < 1e-6 and mr.tolist() == [2, 5]
    m = f32([[1, 2, 3], [4, 5, 6]])
    _, (t1, t2, sw) = run(lambda v, a, c: [v.transpose().mul(1), a.transpose().mul(1), L.swapaxes(c, 1, 2).mul(1)], f32([1, 2, 3]), m, f32(np.arange(12).reshape(2, 2, 3)))
    assert t1.tolist() == [1, 2, 3] and t2.tolist() == [1, 4, 2, 5, 3, 6] and sw.tolist() == np.swapaxes(np.arange(12).reshape(2, 2, 3), 1, 2).ravel().tolist()
    for bad in ([3, 2], [2, 3], [2, 2, 2], [3, -1]):
        with pytest.raises(ValueError):
            J.jit(lambda a: a.reshape(bad), [ShapedArray((4,), F32)])
    _, (rs,) = run(lambda a: a.reshape([2, -1]).sum(1), f32([1, 2, 3, 4]))
    assert rs.tolist() == [3, 7]
    _, (d1, d2) = run(lambda a, b, p, q: [L.dot(a, b), L.dot(p, q)], f32([1, 2, 3]), f32([4, 5, 6]), f32([[1, 2], [3, 4]]), f32([[5, 6], [7, 8]]))
    (d0,) = run0(lambda: L.dot(3, 4))
    assert d0.tolist() == [12] and d1.tolist() == [32] and d2.tolist() == [19, 22, 43, 50]
    J.jit(lambda a, b: seen.setdefault("d", L.dot(a, b)), [ShapedArray((2, 3, 4, 5), F32), ShapedArray((1, 4, 5, 6), F32)])
    assert tuple(seen["d"].shape) == (2, 3, 4, 1, 4, 6)
    _, (big,) = run(lambda a, b: L.dot(a, b), f32(np.arange(784)).reshape(1, 784), np.ones((784, 10), np.float32))
    assert big.tolist() == [784 * 783 / 2] * 10
    _, (mm,) = run(lambda a, b: L.dot(a, b), (f32(np.arange(200)).reshape(200, 1) * np.ones((200, 256), np.float32)), np.ones((256, 200), np.float32))
    assert mm.shape == (40000,) and mm[0] == 0 and mm[200] == 256 and mm[-1] == 199 * 256
    rows, depth, cols = 16, 64, 4
    aD = f32([math.sin(i * 0.17) * 0.7 + ((i // depth) % 7) * 0.03 for i in range(rows * depth)]).reshape(rows, depth)
    wD = f32([math.cos(i * 0.11) * 0.2 for i in range(depth * cols)]).reshape(depth, cols)
    bD = f32([(i - 2) * 0.1 for i in range(cols)])
    _, (aff,) = run(lambda a, w, b: L.dot(a, w).add(b), aD, wD, bD)
    assert np.abs(aff.reshape(rows, cols) - (aD.astype(np.float64) @ wD.astype(np.float64) + bD)).max() < 1e-4
    v, w = f32([3, 1, 4, 2]), f32([[3, 1, 4], [2, 5, 0]])
    _, (n1, n2, n3, x1, x2, x3) = run(lambda a, b: [a.min(), b.min(0), b.min(), a.max(), b.max(0), b.max()], v, w)
    assert (n1.tolist(), n2.tolist(), n3.tolist(), x1.tolist(), x2.tolist(), x3.tolist()) == ([1], [2, 1, 0], [0], [4], [3, 5, 4], [5])
    _, (g1, g2, g3) = run(lambda a, b, c: [L.argmax(a), L.argmax(b, 1), L.argmax(c)], f32([0.1, 0.2, 0.3, 0.2]), f32([[0.1, -0.2, -0.3, 0.1], [0, 0.1, 0.3, 0.3]]), f32([[0.1, -0.2], [0.3, 0.1]]))
    assert g1.tolist() == [2] and g2.tolist() == [0, 2] and g3.tolist() == [2]
    def over(a):
        seen["o"] = [L.applyOverAxes(lambda t, ax: t.sum(ax), a, [0, 2]), L.applyOverAxes(lambda t, ax: t.sum(ax, keepdims=True), a, [1]), L.applyOverAxes(lambda t, ax: t.sum(ax), a, [-1])]
        return seen["o"]
    _, (o1, o2, o3) = _run_typed(over, [x], [I32])
    assert [tuple(o.shape) for o in seen["o"]] == [(1, 3, 1), (2, 1, 4), (2, 3, 1)]
    assert o1.tolist() == [60, 92, 124] and o2.tolist() == [12, 15, 18, 21, 48, 51, 54, 57] and o3.tolist() == [6, 22, 38, 54, 70, 86]
    with pytest.raises(ValueError):
        J.jit(lambda a: L.applyOverAxes(lambda t, ax: L.expandDims(t, 0), a, [0]), [ShapedArray((2, 3), F32)])
    nan = np.nan
    _, (so, s0, s1_, sn) = run(lambda a, b, c: [L.sort(a), L.sort(b, 0).mul(1), L.sort(b, 1), L.sort(c)], f32([3, 1, 4, 1, 5, 9, 2, 6]), f32([[3, 1, 2], [6, 4, 5]]), f32([3, nan, 1, nan, 2]))
    assert so.tolist() == [1, 1, 2, 3, 4, 5, 6, 9] and s0.tolist() == [3, 1, 2, 6, 4, 5] and s1_.tolist() == [1, 2, 3, 4, 5, 6]
    np.testing.assert_array_equal(sn, f32([1, 2, 3, nan, nan]))
    for dt, npdt in ((I32, np.int32), (U32, np.uint32)):
        _, (si,) = _run_typed(lambda a: L.sort(a), [np.array([3, 1, 4, 1, 5], npdt)], [dt])
        assert si.dtype == npdt and si.tolist() == [1, 1, 3, 4, 5]
    _, (sb,) = _run_typed(lambda a: L.sort(a), [_i32([1, 0, 1, 0, 1])], [BOOL])
    assert sb.tolist() == [0, 0, 1, 1, 1]
    _, (sz,) = run(lambda a: L.sort(a), np.zeros((3, 0), np.float32))
    assert sz.tolist() == []
    lin = np.linspace(0, 1, 8192).astype(np.float32)
    _, (sl,) = run(lambda a: L.sort(J.flip(a, None)), lin)
    np.testing.assert_array_equal(sl, lin)
    _, (a1, a2, a3) = run(lambda a, b, c: [L.argsort(a), L.argsort(b, 1), L.argsort(c)], f32([3, 1, 4, 2, 5]), f32([[3, 1, 2], [6, 4, 5]]), f32([3, 1, 1, nan, np.inf, 2, nan, 1, 0, -0.0, np.inf]))
    assert a1.dtype == np.int32 and a1.tolist() == [1, 3, 0, 2, 4] and a2.tolist() == [1, 2, 0, 1, 2, 0]
    assert a3.tolist() == [8, 9, 1, 2, 7, 5, 0, 4, 10, 3, 6]
    _, (al,) = run(lambda a: L.argsort(J.flip(a, None)), np.linspace(0, 1, 8191).astype(np.float32))
    assert al.tolist() == list(range(8190, -1, -1))


def test_activation_tables():
    """test/nn.test.ts:20-85 (relu, sigmoid, softSign, leakyRelu with and without a slope), :119-155 (softmax over two
    axes, over none, of an empty array; log(softmax) == logSoftmax), :157-172 (logsumexp), :174-206 (log1mexp on both
    sides of log 2 and at extreme arguments), :230-272 (oneHot for int32, 2-D and uint32 indices);
    test/scipy-special.test.ts:24-75 (erf / erfc values, logit); the remaining activations against their definitions."""
    x = f32([-1, 0, 1, 2])
    _, (r, sg, ss) = run(lambda a: [L.relu(a), L.sigmoid(a), L.softSign(a)], x)
    assert r.tolist() == [0, 0, 1, 2]
    np.testing.assert_allclose(sg, [0.26894142, 0.5, 0.73105858, 0.88079708], rtol=1e-5)
    np.testing.assert_allclose(ss, [-0.5, 0, 0.5, 2 / 3], rtol=1e-6)
    v = f32([-100, -10, -1, 0, 1, 5, 10])
    _, (l1, l2) = run(lambda a: [L.leakyRelu(a), L.leakyRelu(a, 0.2)], v)
    np.testing.assert_allclose(l1, [-1, -0.1, -0.01, 0, 1, 5, 10], rtol=1e-6)
    np.testing.assert_allclose(l2, [-20, -2, -0.2, 0, 1, 5, 10], rtol=1e-6)
    _, (s2,) = run(lambda a: L.softmax(a, [0, 1]), f32([[1, 2, 3], [4, 5, 6]]))
    np.testing.assert_allclose(s2, [0.00426978, 0.01160646, 0.03154963, 0.08576079, 0.23312202, 0.6336913], rtol=1e-5)
    _, (sn0, sn1, sn2) = run(lambda a, b, c: [J._raise(L.softmax(a, None)).add(0), J._raise(L.softmax(b, [])).add(0), L.softmax(c)], f32(0).reshape(()), f32([1, 2, 3]), f32([]))
    assert sn0.tolist() == [1] and sn1.tolist() == [1, 1, 1] and sn2.tolist() == []
    w = f32([-10, -1, 1, 2])
    _, (sm, lsm, lse) = run(lambda a: [J.log(L.softmax(a)), L.logSoftmax(a), L.logsumexp(a)], w)
    np.testing.assert_allclose(sm, lsm, rtol=1e-5, atol=1e-6)
    assert abs(lse[0] - 2.3490167) < 1e-5
    _, (lse2, lme) = run(lambda a: [L.logsumexp(a), L.logmeanexp(a)], f32([[1, 2, 3, 4], [5, 6, 7, 8]]))
    assert abs(lse2[0] - 8.45834) < 1e-4 and abs(lme[0] - (8.45834 - math.log(8))) < 1e-4
    want = lambda vals: [math.log(-math.expm1(-t)) if t < math.log(2) else math.log1p(-math.exp(-t)) for t in vals]
    for vals, tol in (([0.1, 0.5, 1, 2, 5, 10], 1e-5), ([1e-8, 1e-7, 1e-4, 0.1, 2, 10, 20, 50], 2e-5)):
        _, (lm,) = run(lambda a: L.log1mexp(a), f32(vals))
        np.testing.assert_allclose(lm, want([float(np.float32(t)) for t in vals]), rtol=tol, atol=1e-7 if tol == 1e-5 else 0)
    _, (fx,) = run(lambda a: L.log1mexp(a), f32([math.log(2)]))
    np.testing.assert_allclose(fx, [-math.log(2)], rtol=1e-6)
    _, (o1,) = _run_typed(lambda i: L.oneHot(i, 3), [_i32([1, 1, 2])], [I32])
    _, (o2,) = _run_typed(lambda i: L.oneHot(i, 3), [_i32([[0, 1], [2, 1]])], [I32])
    _, (o3,) = _run_typed(lambda i: L.oneHot(i, 3), [np.array([0, 2, 1], np.uint32)], [U32])
    assert o1.tolist() == [0, 1, 0, 0, 1, 0, 0, 0, 1] and o2.tolist() == [1, 0, 0, 0, 1, 0, 0, 0, 1, 0, 1, 0] and o3.tolist() == [1, 0, 0, 0, 0, 1, 0, 1, 0]
    with pytest.raises(TypeError, match="expects integers"):
        J.jit(lambda i: L.oneHot(i, 3), [ShapedArray((2,), F32)])
    ev = [-10, -5, -1, -0.5, 0, 0.001, 0.1, 1, 5, 10]
    ew = [-1, -1, -0.84270079, -0.52049988, 0, 0.00112838, 0.11246292, 0.84270079, 1, 1]
    _, (ef, ec) = run(lambda a: [J.erf(a), J.erfc(a)], f32(ev))
    np.testing.assert_allclose(ef, ew, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(ec, [1 - t for t in ew], rtol=1e-5, atol=1e-7)
    _, (lg,) = run(lambda a: L.logit(a), f32([0.01, 0.1, 0.25, 0.5, 0.75, 0.9, 0.99]))
    np.testing.assert_allclose(lg, [-4.59511985, -2.19722458, -1.09861229, 0, 1.09861229, 2.19722458, 4.59511985], rtol=1e-5, atol=1e-7)
    z = f32([-3, -1.5, -1, -0.25, 0, 0.5, 1, 2.5, 7])
    d = z.astype(np.float64)
    sig = lambda t: 1 / (1 + np.exp(-t))
    fns = [(L.relu6, np.clip(d, 0, 6)), (L.softplus, np.log1p(np.exp(d))), (L.sparsePlus, np.where(d <= -1, 0, np.where(d < 1, (d + 1) ** 2 / 4, d))),
           (L.sparseSigmoid, np.clip((d + 1) / 2, 0, 1)), (L.silu, d * sig(d)), (L.logSigmoid, -np.log1p(np.exp(-d))), (L.hardSigmoid, np.clip(d + 3, 0, 6) / 6),
           (L.hardSilu, d * np.clip(d + 3, 0, 6) / 6), (L.hardTanh, np.clip(d, -1, 1)), (L.elu, np.where(d < 0, np.expm1(d), d)),
           (lambda a: L.celu(a, 2.0), np.where(d < 0, 2 * np.expm1(d / 2), d)), (L.selu, 1.0507009873554805 * np.where(d < 0, 1.6732632423543772 * np.expm1(d), d)),
           (L.squareplus, (d + np.sqrt(d * d + 4)) / 2), (L.mish, d * np.tanh(np.log1p(np.exp(d))))]
    _, outs = run(lambda a: [f(a) for f, _ in fns], z)
    for got, (_, ref) in zip(outs, fns):
        np.testing.assert_allclose(got, ref, rtol=2e-5, atol=2e-6)
    _, (gl,) = run(lambda a: L.glu(a), f32([[1, 2, 3, 4], [-1, 0, 1, 2]]))
    np.testing.assert_allclose(gl, (np.array([[1, 2], [-1, 0]]) * sig(np.array([[3.0, 4.0], [1.0, 2.0]]))).ravel(), rtol=1e-5)
    with pytest.raises(ValueError, match="even length"):
        J.jit(lambda a: L.glu(a), [ShapedArray((3,), F32)])


def test_top_k_tables():
    """test/lax.test.ts:14-77: values and indices, ties keep the original order, k = n, k = 0, either axis of a 2-D
    array, NaN ranks highest, invalid k."""
    _, (v, i) = run(lambda a: L.topK(a, 3), f32([3, 1, 4, 1, 5, 9, 2, 6]))
    assert v.tolist() == [9, 6, 5] and i.tolist() == [5, 7, 4]
    _, (v, i) = run(lambda a: L.topK(a, 4), f32([1, 3, 2, 3, 3, 0]))
    assert v.tolist() == [3, 3, 3, 2] and i.tolist() == [1, 3, 4, 2]
    _, (v, i) = run(lambda a: L.topK(a, 3), f32([5, 2, 8]))
    assert v.tolist() == [8, 5, 2] and i.tolist() == [2, 0, 1]
    _, (v, i) = run(lambda a: L.topK(a, 0), f32([1, 2, 3]))
    assert v.tolist() == [] and i.tolist() == [] and i.dtype == np.int32
    m = f32([[3, 1, 4], [1, 5, 9]])
    _, (v, i, v0, i0) = run(lambda a: L.topK(a, 2) + L.topK(a, 1, 0), m)
    assert v.tolist() == [4, 3, 9, 5] and i.tolist() == [2, 0, 2, 1] and v0.tolist() == [3, 5, 9] and i0.tolist() == [0, 1, 1]
    _, (v, i) = run(lambda a: L.topK(a, 2), f32([1.5, np.nan, 3.5, 2.1]))
    np.testing.assert_array_equal(v, f32([np.nan, 3.5]))
    assert i.tolist() == [1, 2]
    for bad in (-1, 4):
        with pytest.raises(ValueError):
            J.jit(lambda a: L.topK(a, bad), [ShapedArray((3,), F32)])


def test_numpy_linalg_tables():
    """test/numpy-linalg.test.ts:227-244 (det), :246-294 (inv, batched), :296-310 (matrixPower), :312-366 (multiDot),
    :368-514 (lstsq: tall, wide, square, several right-hand sides, shape errors), :516-526 (slogdet), :528-550 (solve,
    batched), :72-126 (eigvalsh), :552-596 (vectorNorm), :597-713 (matrixNorm), :715-859 (norm: flattened, vector,
    matrix over axis pairs, singular-value norms, errors)."""
    a2 = f32([[4, 7], [2, 6]])
    _, (d, sg, ld, ai) = run(lambda a: [L.det(a)] + L.slogdet(a) + [L.matmul(a, L.inv(a))], a2)
    np.testing.assert_allclose(d, [10], rtol=1e-5)
    np.testing.assert_allclose(sg, [1])
    np.testing.assert_allclose(ld, [math.log(10)], rtol=1e-5)
    np.testing.assert_allclose(ai.reshape(2, 2), np.eye(2), atol=1e-6)
    rng = np.random.default_rng(0)
    big = rng.uniform(0, 1, (15, 15)).astype(np.float32)
    _, (db, sb, lb) = run(lambda a: [L.det(a)] + L.slogdet(a), big)
    sgn, logabs = np.linalg.slogdet(big.astype(np.float64))
    np.testing.assert_allclose(db, [np.linalg.det(big.astype(np.float64))], rtol=2e-3)
    assert sb.tolist() == [sgn] and abs(lb[0] - logabs) < 1e-3
    bat = rng.uniform(0, 1, (2, 3, 4, 4)).astype(np.float32)
    _, (ib,) = run(lambda a: L.matmul(a, L.inv(a)), bat)
    np.testing.assert_allclose(ib.reshape(2, 3, 4, 4), np.broadcast_to(np.eye(4), (2, 3, 4, 4)), atol=1e-4)
    sym = f32([[2, 1], [1, 3]])
    _, (p0, p3, pm) = run(lambda a: [J._raise(L.matrixPower(a, 0)).mul(1), L.matrixPower(a, 3), L.matrixPower(a, -2)], sym)
    np.testing.assert_array_equal(p0.reshape(2, 2), np.eye(2))
    np.testing.assert_allclose(p3.reshape(2, 2), np.linalg.matrix_power(sym.astype(np.float64), 3), rtol=1e-5)
    np.testing.assert_allclose(pm.reshape(2, 2), np.linalg.matrix_power(sym.astype(np.float64), -2), rtol=1e-4)
    # "inv preserves input dtype" / "matrixPower(A, 0) preserves input dtype" (:270-283, :297-309): float64 on the CPU
    # devices, float16 on the GPU device -- both element types run through the LU and triangular-solve routines here
    for dt, npt in ((DType.Float64, np.float64), (DType.Float16, np.float16)):
        seen = {}
        _, (ident, p0) = run(lambda a: [L.matmul(a, seen.setdefault("inv", L.inv(a))), J._raise(seen.setdefault("p0", L.matrixPower(a, 0))).mul(1)],
                             sym.astype(npt), dtype=dt)
        assert seen["inv"].dtype == dt and seen["p0"].dtype == dt and ident.dtype == npt and p0.dtype == npt
        np.testing.assert_allclose(ident.reshape(2, 2).astype(np.float64), np.eye(2), rtol=0, atol=1e-3)
        np.testing.assert_allclose(p0.reshape(2, 2).astype(np.float64), np.eye(2), rtol=0, atol=1e-3)
    A, B, C = f32([[1, 2], [3, 4]]), f32([[5, 6, 7], [8, 9, 10]]), f32([[11, 12], [13, 14], [15, 16]])
    _, (m3, m2) = run(lambda a, b, c: [L.multiDot([a, b, c]), L.multiDot([a, b])], A, B, C)
    np.testing.assert_allclose(m3.reshape(2, 2), A @ B @ C, rtol=1e-6)
    np.testing.assert_allclose(m2.reshape(2, 3), A @ B, rtol=1e-6)
    seen = {}
    _, (mv,) = run(lambda x, a, b, y: seen.setdefault("m", L.multiDot([x, a, b, y])), f32([1, 2]), f32([[1, 2, 3], [4, 5, 6]]), f32([[1, 0], [0, 1], [1, 1]]), f32([2, 3]))
    assert tuple(seen["m"].shape) == () and mv.tolist() == [129]
    tall, wide = f32([[1, 2], [3, 4], [5, 6]]), f32([[1, 2, 3], [4, 5, 6]])
    for a, b in ((tall, f32([[1], [2], [3]])), (tall, f32([[1, 2], [3, 4], [5, 6]]))):
        _, (x,) = run(lambda p, q: L.lstsq(p, q), a, b)
        x = x.reshape(2, -1)
        np.testing.assert_allclose(a.T @ a @ x, a.T @ b, rtol=1e-4, atol=1e-4)
    for a, b in ((wide, f32([[1], [2]])), (wide, f32([[1, 2], [3, 4]])), (sym, f32([[5], [7]]))):
        _, (x,) = run(lambda p, q: L.lstsq(p, q), a, b)
        np.testing.assert_allclose(a @ x.reshape(a.shape[1], -1), b, rtol=1e-4, atol=1e-4)
    for shapes in (((3,), (3,)), ((2, 2), (3,))):
        with pytest.raises(ValueError):
            J.jit(lambda p, q: L.lstsq(p, q), [ShapedArray(s, F32) for s in shapes])
    _, (sx,) = run(lambda p, q: L.solve(p, q), f32([[3, 2], [1, 2]]), f32([5, 4]))
    np.testing.assert_allclose(sx, [0.5, 1.75], rtol=1e-5)
    Ab, Xb = rng.uniform(0, 1, (10, 15, 15)).astype(np.float32), rng.uniform(0, 1, (10, 15, 5)).astype(np.float32)
    _, (xp,) = run(lambda p, q: L.solve(p, q), Ab, (Ab.astype(np.float64) @ Xb).astype(np.float32))
    np.testing.assert_allclose(xp.reshape(Xb.shape), Xb, rtol=1e-2, atol=1e-3)
    _, (xb,) = run(lambda p, q: L.solve(p, q), sym, f32(np.arange(12).reshape(3, 2, 2)))
    np.testing.assert_allclose(xb.reshape(3, 2, 2), np.linalg.solve(sym.astype(np.float64), np.arange(12.0).reshape(3, 2, 2)), rtol=1e-5, atol=1e-6)
    S = rng.standard_normal((6, 6)).astype(np.float32)
    S = (S + S.T) / 2
    _, (ev, ew, evec) = run(lambda p: [L.eigvalsh(p)] + L.linalgEigh(p), S)
    np.testing.assert_allclose(ev, np.linalg.eigvalsh(S.astype(np.float64)), rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(ev, ew)
    V = evec.reshape(6, 6)
    np.testing.assert_allclose(V @ np.diag(ew) @ V.T, S, atol=1e-4)
    inf = math.inf
    v = f32([3, -4])
    _, (n2, n1, ni, nm, n0) = run(lambda p, q: [L.vectorNorm(p), L.vectorNorm(p, 1), L.vectorNorm(p, inf), L.vectorNorm(p, -inf), L.vectorNorm(q, 0)], v, f32([0, 3, 0, -4, 5]))
    np.testing.assert_allclose([n2[0], n1[0], ni[0], nm[0], n0[0]], [5, 7, 4, 3, 3], rtol=1e-5)
    M = f32([[3, 4], [5, 12]])
    _, (na, nk) = run(lambda p: [L.vectorNorm(p, axis=1), seen.setdefault("k", L.vectorNorm(p, axis=1, keepdims=True))], M)
    np.testing.assert_allclose(na, [5, 13], rtol=1e-5)
    np.testing.assert_allclose(nk, [5, 13], rtol=1e-5)
    assert tuple(seen["k"].shape) == (2, 1)
    mat, batched = f32([[1, 2], [3, 4]]), f32(np.arange(18).reshape(2, 3, 3))
    for o, want_m, want_b in (("fro", 5.477225575051661, [14.28285686, 39.7617907]), (1, 6, [15, 42]), (-1, 4, [9, 36]), (inf, 7, [21, 48]), (-inf, 3, [3, 30])):
        shapes = {}
        def norms(p, q):
            outs = [L.matrixNorm(p, o), L.matrixNorm(p, o, True), L.matrixNorm(q, o), L.matrixNorm(q, o, True)]
            shapes["s"] = [tuple(t.shape) for t in outs]
            return outs
        _, (a, ak, b, bk) = run(norms, mat, batched)
        assert shapes["s"] == [(), (1, 1), (2,), (2, 1, 1)]
        np.testing.assert_allclose([a[0], ak[0]], [want_m, want_m], rtol=1e-5)
        np.testing.assert_allclose(b, want_b, rtol=1e-5)
        np.testing.assert_allclose(bk, want_b, rtol=1e-5)
    with pytest.raises(ValueError):
        J.jit(lambda p: L.matrixNorm(p), [ShapedArray((4,), F32)])
    for o in (-2, 2, "nuc"):
        with pytest.raises(ValueError):
            J.jit(lambda p: L.matrixNorm(p, o), [ShapedArray((2, 2), F32)])
    b24 = f32(np.arange(24).reshape(2, 3, 4))
    _, (f1, f2, f3) = run(lambda p, q: [L.norm(p), L.norm(q), seen.setdefault("n", L.norm(q, keepdims=True))], mat, b24)
    np.testing.assert_allclose([f1[0], f2[0], f3[0]], [5.477225575051661, 65.75712889109438, 65.75712889109438], rtol=1e-5)
    assert tuple(seen["n"].shape) == (1, 1, 1)
    _, (v2, v1, vi) = run(lambda p: [L.norm(p), L.norm(p, 1), L.norm(p, inf)], v)
    np.testing.assert_allclose([v2[0], v1[0], vi[0]], [5, 7, 4], rtol=1e-5)
    _, (ni0,) = _run_typed(lambda p: L.norm(p, 0), [_i32([3, 0, -4])], [I32])
    _, (nb,) = _run_typed(lambda p: L.norm(p), [_i32([1, 0, 1])], [BOOL])
    assert ni0.dtype == np.float32 and ni0.tolist() == [2] and nb.dtype == np.float32 and abs(nb[0] - math.sqrt(2)) < 1e-6
    _, (ax1, ax2) = run(lambda p: [L.norm(p, inf, -1), L.norm(p, axis=1)], b24)
    np.testing.assert_allclose(ax1, [3, 7, 11, 15, 19, 23])
    np.testing.assert_allclose(ax2, np.linalg.norm(b24, axis=1).ravel(), rtol=1e-5)
    _, ms = run(lambda p: [L.norm(p, o) for o in ("fro", "f", 1, -1, inf, -inf)], mat)
    np.testing.assert_allclose([t[0] for t in ms], [5.477225575051661, 5.477225575051661, 6, 4, 7, 3], rtol=1e-5)
    _, (p1, p2, p3, p4, p5) = run(lambda p: [L.norm(p, axis=[1, 2]), L.norm(p, inf, [0, 2]), L.norm(p, 1, [2, 0]), L.norm(p, -1, [2, 0]), seen.setdefault("p", L.norm(p, inf, [0, 2], True))], b24)
    np.testing.assert_allclose(p1, [22.4944437584, 61.7899668231], rtol=1e-5)
    assert p2.tolist() == [54, 70, 86] and p3.tolist() == [54, 70, 86] and p4.tolist() == [6, 22, 38] and p5.tolist() == [54, 70, 86]
    assert tuple(seen["p"].shape) == (1, 3, 1)
    tol = dict(rtol=1e-4, atol=1e-4)
    _, (s2, sm2, sn) = run(lambda p: [L.norm(p, 2), L.norm(p, -2), L.norm(p, "nuc")], mat)
    np.testing.assert_allclose([s2[0], sm2[0], sn[0]], [5.464985704219043, 0.36596619062625757, 5.8309518948453], **tol)
    ab = f32([[[1, 2, 0.5], [3, 4, -1]], [[2, -1, 0], [1, 5, 2]]])
    _, (q1, q2, q3, q4, q5) = run(lambda p: [L.norm(p, 2, [1, 2]), L.norm(p, -2, [1, 2]), L.norm(p, "nuc", [1, 2]), L.norm(p, 2, [2, 0]), seen.setdefault("q", L.norm(p, "nuc", [2, 0], True))], ab)
    np.testing.assert_allclose(q1, [5.5123605371, 5.5095335676], **tol)
    np.testing.assert_allclose(q2, [0.9294521555, 2.1552354553], **tol)
    np.testing.assert_allclose(q3, [6.4418126926, 7.6647690229], **tol)
    np.testing.assert_allclose(q4, [2.2912878475, 7.0067840776], **tol)
    np.testing.assert_allclose(q5, [4.527355825, 9.634516349], **tol)
    assert tuple(seen["q"].shape) == (1, 2, 1)
    for kw, shp in ((dict(ord=3, axis=[0, 1]), (2, 2)), (dict(ord="fro", axis=0), (2, 2)), (dict(axis=[0, 0]), (2, 2)), (dict(axis=[0, 1, 2]), (2, 3, 4)), (dict(ord=2), (2, 3, 4))):
        with pytest.raises(ValueError):
            J.jit(lambda p: L.norm(p, **kw), [ShapedArray(shp, F32)])


def _dft(real, imag):
    n = len(real)
    k = np.arange(n)
    w = np.exp(-2j * np.pi * np.outer(k, k) / n)
    out = w @ (np.asarray(real, np.float64) + 1j * np.asarray(imag, np.float64))
    return out.real, out.imag


def test_numpy_fft_tables():
    """test/numpy-fft.test.ts:28-87 (fft against a direct DFT: powers of two, length one, mixed radix, a prime; another
    axis), :89-124 (ifft, round trips either way), :126-166 (fftn, fft2 / ifft2), :168-231 (rfft / irfft, rfft2, rfftn /
    irfftn, hfft / ihfft), :233-255 (fftfreq, rfftfreq, fftshift / ifftshift)."""
    cases = [([0, 1, 2, 3], [0, 0, 0, 0]), ([1, 0, 0, 0], [0, 0, 0, 0]), ([3, 3, 3, 3], [0, 0, 0, 0]), ([3], [-2]),
             ([1, 3, 0, -2, 5, 1, 2, -1], [2, -1, 4, 1, 0, -3, 2, 1]), ([1, 3, 0, -2, 5, 1], [2, -1, 4, 1, 0, -3]), ([4, -1, 2, 0, 3], [0, 2, -3, 1, 5])]
    for re, im in cases:
        _, (r, i) = run(lambda a, b: list(L.fft1(a, b)), f32(re), f32(im))
        wr, wi = _dft(re, im)
        np.testing.assert_allclose(r, wr, atol=1e-4)
        np.testing.assert_allclose(i, wi, atol=1e-4)
    _, (r, i) = run(lambda a, b: list(L.fft1(a, b, 0)), f32([[1, 2, 3, 4], [5, 6, 7, 8]]), np.zeros((2, 4), np.float32))
    np.testing.assert_allclose(r, [6, 8, 10, 12, -4, -4, -4, -4], rtol=1e-5)
    np.testing.assert_allclose(i, 0, atol=1e-5)
    _, (r, i) = run(lambda a, b: list(L.ifft(a, b)), f32([6, -2, -2, -2]), f32([0, 2, 0, -2]))
    np.testing.assert_allclose(r, [0, 1, 2, 3], atol=1e-6)
    np.testing.assert_allclose(i, 0, atol=1e-6)
    for re, im in (([1, 2, 3, 4, 5, 6, 7, 8], [-5, 9, 0, 3, -1, 4, 2, 8]), ([1, 2, 3, 4, 5, 6], [-5, 9, 0, 3, -1, 4])):
        _, (r, i) = run(lambda a, b: list(L.ifft(*L.fft1(a, b))), f32(re), f32(im))
        np.testing.assert_allclose(r, re, atol=1e-5)
        np.testing.assert_allclose(i, im, atol=1e-5)
    _, (r, i) = run(lambda a, b: list(L.fft1(*L.ifft(a, b))), f32([2, -1, 4, 0]), f32([1, 3, -2, 5]))
    np.testing.assert_allclose(r, [2, -1, 4, 0], atol=1e-5)
    np.testing.assert_allclose(i, [1, 3, -2, 5], atol=1e-5)
    _, (r, i) = run(lambda a, b: list(L.fftn(a, b)), f32([[1, 2], [3, 4]]), np.zeros((2, 2), np.float32))
    np.testing.assert_allclose(r, [10, -2, -4, 0], atol=1e-5)
    np.testing.assert_allclose(i, 0, atol=1e-5)
    R, I = f32([[1, 2, 3, 4], [5, 6, 7, 8]]), f32([[1, -1, 2, -2], [3, -3, 4, -4]])
    _, (r, i) = run(lambda a, b: list(L.ifft2(*L.fft2(a, b))), R, I)
    np.testing.assert_allclose(r, R.ravel(), atol=1e-5)
    np.testing.assert_allclose(i, I.ravel(), atol=1e-5)
    _, (r, i) = run(lambda a: list(L.rfft(a)), f32([0, 1, 2, 3]))
    np.testing.assert_allclose(r, [6, -2, -2], atol=1e-5)
    np.testing.assert_allclose(i, [0, 2, 0], atol=1e-5)
    x8 = f32(np.arange(8))
    _, (back,) = run(lambda a: L.irfft(*L.rfft(a)), x8)
    np.testing.assert_allclose(back, x8, atol=1e-5)
    _, (r, i) = run(lambda a: list(L.rfft2(a)), R)
    np.testing.assert_allclose(r, [36, -4, -4, -16, 0, 0], atol=1e-5)
    np.testing.assert_allclose(i, [0, 4, 0, 0, 0, 0], atol=1e-5)
    _, (back2,) = run(lambda a: L.irfftn(*L.rfftn(a)), R)
    np.testing.assert_allclose(back2, R.ravel(), atol=1e-5)
    _, (h, hr, hi) = run(lambda a, b, c: [L.hfft(a, b)] + list(L.ihfft(c)), f32([1, 2, 4]), f32([0, 3, 0]), f32([9, 3, 1, -9]))
    np.testing.assert_allclose(h, [9, 3, 1, -9], atol=1e-5)
    np.testing.assert_allclose(hr, [1, 2, 4], atol=1e-5)
    np.testing.assert_allclose(hi, [0, 3, 0], atol=1e-5)
    np.testing.assert_allclose(L.fftfreq(4), [0, 0.25, -0.5, -0.25])
    np.testing.assert_allclose(L.fftfreq(5, 0.5), [0, 0.4, 0.8, -0.8, -0.4], rtol=1e-6)
    np.testing.assert_allclose(L.rfftfreq(4), [0, 0.25, 0.5])
    np.testing.assert_allclose(L.rfftfreq(5, 0.5), [0, 0.4, 0.8], rtol=1e-6)
    assert L.fftfreq(4).dtype == np.float32
    _, (s4, s5, is5) = run(lambda a, b: [L.fftshift(a), L.fftshift(b), L.ifftshift(b)], f32([0, 1, 2, 3]), f32([0, 1, 2, 3, 4]))
    assert s4.tolist() == [2, 3, 0, 1] and s5.tolist() == [3, 4, 0, 1, 2] and is5.tolist() == [2, 3, 4, 0, 1]
    with pytest.raises(ValueError, match="same shape"):
        J.jit(lambda a, b: list(L.fft1(a, b)), [ShapedArray((4,), F32), ShapedArray((3,), F32)])
    with pytest.raises(ValueError, match="float dtype"):
        J.jit(lambda a, b: list(L.fft1(a, b)), [ShapedArray((4,), I32), ShapedArray((4,), I32)])


def _key(seed):
    return np.array([0, seed], np.uint32)


def _sample(fn, seed, *arrays):
    prog = J.jit(fn, [ShapedArray((2,), U32)] + [ShapedArray(tuple(a.shape), F32) for a in arrays])
    be = OracleBackend()
    outs = run_program(be, prog, [_key(seed)] + list(arrays))
    assert be.live_slots() == 0
    return outs


def test_random_distribution_tables():
    """test/random.test.ts:99-131 (normal: mass within 1, 2, 3 sigma; bernoulli with an array of p), :133-346
    (categorical: frequencies, default shape, batched and non-default axes, shape errors, without replacement), :347-520
    (cauchy quartiles; laplace, gumbel, logistic moments; randint, rademacher, lognormal, rayleigh, pareto, weibullMin,
    geometric, triangular, maxwell, doubleSidedMaxwell, ball), :522-575 (choice, permutation), :577-600
    (multivariateNormal mean and covariance)."""
    (z,) = _sample(lambda k: L.random_normal(k, [5000]), 123)
    for s, want in ((1, 0.6827), (2, 0.9545), (3, 0.9973)):
        assert abs((np.abs(z) <= s).mean() - want) < 0.005 * 3
    (b,) = _sample(lambda k, p: L.random_bernoulli(k, p, [2, 500]), 2024, f32([[0.25], [0.8]]))
    fr = b.reshape(2, 500).mean(1)
    assert abs(fr[0] - 0.25) < 0.05 and abs(fr[1] - 0.8) < 0.05
    probs = [0.1, 0.2, 0.3, 0.4]
    (c,) = _sample(lambda k, lg: L.random_categorical(k, J.log(lg), shape=[10000]), 555, f32(probs))
    assert c.dtype == np.int32
    for i, p in enumerate(probs):
        assert abs((c == i).mean() - p) < 0.05
    seen = {}
    (c0,) = _sample(lambda k, lg: seen.setdefault("c", L.random_categorical(k, lg)), 444, f32([1, 2, 3]))
    assert tuple(seen["c"].shape) == () and 0 <= c0[0] < 3
    (cb,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[100, 2]), 333, f32([[10, 0, 0], [0, 0, 10]]))
    assert (cb.reshape(100, 2) == [0, 2]).all()
    (ca,) = _sample(lambda k, lg: L.random_categorical(k, lg, axis=0, shape=[100, 2]), 123, f32([[10, 0], [0, 10], [0, 0]]))
    assert (ca.reshape(100, 2) == [0, 1]).all()
    for shp, lshape in (([10, 5], (2, 3)), ([1], (4, 5))):
        with pytest.raises(ValueError, match="(?i)incompatible shapes|not broadcast-compatible"):
            J.jit(lambda k, lg: L.random_categorical(k, lg, shape=shp), [ShapedArray((2,), U32), ShapedArray(lshape, F32)])
    lg5 = f32([1, 2, 3, 4, 5])
    (cm,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[2, 3]), 888, lg5)
    assert cm.shape == (6,) and ((0 <= cm) & (cm < 5)).all()
    (cw,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[3], replace=False), 222, lg5)
    assert len(set(cw.tolist())) == 3 and ((0 <= cw) & (cw < 5)).all()
    with pytest.raises(ValueError, match="cannot exceed"):
        J.jit(lambda k, lg: L.random_categorical(k, lg, shape=[5], replace=False), [ShapedArray((2,), U32), ShapedArray((3,), F32)])
    (cbw,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[3, 2], replace=False), 777, f32([[1, 2, 3, 4, 5], [5, 4, 3, 2, 1]]))
    rows = cbw.reshape(2, 3)  # what topK returned per batch row, before the reference's final reshape to [3, 2]
    assert len(set(rows[0].tolist())) == 3 and len(set(rows[1].tolist())) == 3
    (call,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[5], replace=False), 105, lg5)
    assert sorted(call.tolist()) == [0, 1, 2, 3, 4]
    (c6,) = _sample(lambda k, lg: L.random_categorical(k, lg, shape=[2, 3], replace=False), 106, f32([1, 2, 3, 4, 5, 6]))
    assert sorted(c6.tolist()) == [0, 1, 2, 3, 4, 5]
    ones = np.ones((2, 5, 3), np.float32)
    for kw, want in ((dict(axis=1), (2, 3)), (dict(axis=1, shape=[10, 2, 3]), (10, 2, 3)), (dict(axis=-2, shape=[4, 2, 3]), (4, 2, 3))):
        _sample(lambda k, lg: seen.__setitem__("s", L.random_categorical(k, lg, **kw)) or seen["s"], 100, ones)
        assert tuple(seen["s"].shape) == want
    (cy,) = _sample(lambda k: L.random_cauchy(k, [20000]), 999)
    q1, med, q3 = np.sort(cy)[[5000, 10000, 15000]]
    assert abs(med) < 0.05 and abs(q1 + 1) < 0.05 and abs(q3 - 1) < 0.05
    (lp,) = _sample(lambda k: L.random_laplace(k, [20000]), 888)
    assert abs(lp.mean()) < 0.05 and abs(lp.var(ddof=1) - 2) < 0.5
    (gb,) = _sample(lambda k: L.random_gumbel(k, [20000]), 777)
    assert abs(gb.mean() - 0.5772156649) < 0.05 and abs(gb.var(ddof=1) - math.pi ** 2 / 6) < 0.05
    (ri,) = _sample(lambda k: L.random_randint(k, -3, 7, [5000]), 1201)
    assert ri.dtype == np.int32 and ri.min() >= -3 and ri.max() < 7
    assert all(abs((ri == v).mean() - 0.1) < 0.05 for v in range(-3, 7))
    (rd,) = _sample(lambda k: L.random_rademacher(k, [5000]), 1202)
    assert set(rd.tolist()) == {-1, 1} and abs(rd.mean()) < 0.08
    (lo,) = _sample(lambda k: L.random_logistic(k, [10000]), 1203)
    assert abs(lo.mean()) < 0.1 and 3.0 < lo.var(ddof=1) < 3.6
    (ln,) = _sample(lambda k: L.random_lognormal(k, 1, [10000]), 1204)
    assert (ln > 0).all() and 1.45 < ln.mean() < 1.85
    (ry,) = _sample(lambda k: L.random_rayleigh(k, 2, [10000]), 1205)
    assert (ry >= 0).all() and 2.35 < ry.mean() < 2.65
    (pa,) = _sample(lambda k: L.random_pareto(k, 3, [10000]), 1206)
    assert (pa >= 1).all() and 1.35 < pa.mean() < 1.65
    (wb,) = _sample(lambda k: L.random_weibullMin(k, 2, 1, [10000]), 1207)
    assert (wb >= 0).all() and 1.8 < wb.mean() < 2.2
    (ge,) = _sample(lambda k: L.random_geometric(k, 0.25, [10000]), 1208)
    assert ge.dtype == np.int32 and (ge >= 1).all() and 3.7 < ge.mean() < 4.3
    (tr,) = _sample(lambda k: L.random_triangular(k, -1, 0, 2, [10000]), 1209)
    assert ((tr >= -1) & (tr <= 2)).all() and 0.23 < tr.mean() < 0.43
    (mw,) = _sample(lambda k: L.random_maxwell(k, [10000]), 1210)
    assert (mw >= 0).all() and 1.45 < mw.mean() < 1.75
    (dm,) = _sample(lambda k: L.random_doubleSidedMaxwell(k, 0, 1, [10000]), 1211)
    assert abs(dm.mean()) < 0.12 and 1.45 < np.abs(dm).mean() < 1.75
    (bl,) = _sample(lambda k: L.random_ball(k, 3, shape=[5000]), 1212)
    r2 = (bl.reshape(5000, 3) ** 2).sum(1)
    assert (r2 <= 1.0001).all() and 0.55 < r2.mean() < 0.65
    (ch,) = _sample(lambda k: L.random_choice(k, 5, [200]), 1213)
    assert ch.dtype == np.int32 and ((0 <= ch) & (ch < 5)).all()
    (cv,) = _sample(lambda k, v: L.random_choice(k, v, [200]), 1214, f32([10, 20, 30, 40, 50]))
    assert set(cv.tolist()) <= {10, 20, 30, 40, 50}
    (pm,) = _sample(lambda k: L.random_permutation(k, 8), 1215)
    (pv,) = _sample(lambda k, v: L.random_permutation(k, v), 1216, f32([10, 20, 30, 40]))
    assert sorted(pm.tolist()) == list(range(8)) and sorted(pv.tolist()) == [10, 20, 30, 40]
    (cn,) = _sample(lambda k: L.random_choice(k, 6, [4], replace=False), 1217)
    assert len(set(cn.tolist())) == 4 and ((0 <= cn) & (cn < 6)).all()
    mean, cov = f32([1, 2]), f32([[1, 0.5], [0.5, 2]])
    (mv, mm, mc) = _sample(lambda k, m, c: (lambda y: [y, y.mean(0), L.cov(y, None, rowvar=False)])(L.random_multivariateNormal(k, m, c, [5000])), 42, mean, cov)
    assert mv.shape == (10000,)
    np.testing.assert_allclose(mm, mean, atol=3e-2)
    np.testing.assert_allclose(mc.reshape(2, 2), cov, atol=5e-2)


def test_einsum_parser_and_path_golden_vectors():
    """src/library/numpy/einsum.test.ts:4-87 (explicit and implicit forms, ellipses, broadcasting ellipses) and :89-166
    (flop estimates, output shapes and the chosen contraction order for matmul, traces, diagonals, chains of three and
    five matrices)."""
    from jaxjs_hip.einsum import computeEinsumPath, parseEinsumExpression as parse
    def both(expr, shapes):
        e = parse(expr, shapes)
        return e.lhsIndices, e.rhsIndex
    assert both("ij,jk->ik", [[], []]) == ([[0, 1], [1, 2]], [0, 2])
    assert both("iii->i", [[]]) == ([[0, 0, 0]], [0])
    assert both("ji->ji", [[]]) == ([[1, 0]], [1, 0])
    assert both("ij->ji", [[]]) == ([[0, 1]], [1, 0])
    assert both("->", [[]]) == ([[]], [])
    assert both("ij,jk", [[], []]) == ([[0, 1], [1, 2]], [0, 2])
    assert both("iii", [[]]) == ([[0, 0, 0]], [])
    assert both("ji", [[]]) == ([[1, 0]], [0, 1])
    assert both("...ij,jk->...ik", [[2, 3, 4], [4, 5]]) == ([[3, 0, 1], [1, 2]], [3, 0, 2])
    assert both("...->", [[100]]) == ([[0]], [])
    assert both("...ij,j", [[2, 3, 4], [4, 5]]) == ([[2, 0, 1], [1]], [2, 0])
    assert both("..., ..., ...", [[], [1, 4], [5, 3, 4]]) == ([[], [1, 2], [0, 1, 2]], [0, 1, 2])
    p = computeEinsumPath(parse("ij,jk->ik", [[25, 30], [30, 40]]))
    assert p.approximateFlops == 2 * 25 * 40 * 30 and p.outputShape == [25, 40] and p.path == [(0, 1)]
    p = computeEinsumPath(parse("ii->", [[50, 50]]))
    assert p.approximateFlops == 50 and p.outputShape == [] and p.path == []
    p = computeEinsumPath(parse("ii->i", [[60, 60]]))
    assert p.approximateFlops == 60 and p.outputShape == [60] and p.path == []
    p = computeEinsumPath(parse("ii,ii->", [[70, 70], [70, 70]]))
    assert p.approximateFlops == 2 * 70 and p.outputShape == [] and p.path == [(0, 1)]
    p = computeEinsumPath(parse("ij,jk,kl->il", [[10, 20], [20, 30], [30, 40]]), "optimal")
    assert p.path == [(0, 1), (2, 3)] and p.approximateFlops == 2 * (10 * 30 * 20 + 10 * 40 * 30)
    p = computeEinsumPath(parse("ab,bc,cd,de,ef->af", [[5, 10], [10, 15], [15, 20], [20, 25], [25, 30]]), "optimal")
    assert p.path == [(0, 1), (2, 5), (3, 6), (4, 7)]


def test_einsum_tables():
    """test/numpy.test.ts:1819-2052: matmul, sums and traces of one operand, transposition, the JAX documentation's
    examples in string and index-list form (inner and outer products, matrix-vector, ellipsis reductions, diagonals, a
    three-index contraction, a chain of four matrices), and the shape table incl. ellipses and size-1 broadcasting."""
    a = f32(np.arange(6).reshape(2, 3))
    _, (c,) = run(lambda p, q: L.einsum("ik,kj->ij", p, q), a, np.ones((3, 4), np.float32))
    assert c.tolist() == [3] * 4 + [12] * 4
    _, outs = run(lambda p: [L.einsum("ij->", p), L.einsum(p, [0, 1], []), L.einsum("ij->j", p), L.einsum("ji->j", p), L.einsum("ii->", J.shrink(p, [(0, 2), (1, 3)])), L.einsum("ji", p)], a)
    assert [o.tolist() for o in outs] == [[15], [15], [3, 5, 7], [3, 12], [6], [0, 3, 1, 4, 2, 5]]
    M, x, y = f32(np.arange(16).reshape(4, 4)), f32(np.arange(4)), f32([5, 4, 3, 2])
    e = L.einsum
    _, outs = run(lambda m, p, q: [e("i,i", p, q), e("i,i->", p, q), e(p, [0], q, [0]), e(p, [0], q, [0], []),
                                   e("ij,j->i", m, p), e("ij,j", m, p), e(m, [0, 1], p, [1], [0]), e(m, [0, 1], p, [1]),
                                   e("i,j->ij", p, q), e("i,j", p, q), e(p, [0], q, [1], [0, 1]), e(p, [0], q, [1]),
                                   e("i->", p), e(p, [0], []), e("...j->...", m), e("ii->i", m), e("ii", m)], M, x, y)
    got = [o.tolist() for o in outs]
    outer = np.outer(x, y).ravel().tolist()
    assert got[:4] == [[16]] * 4 and got[4:8] == [[14, 38, 62, 86]] * 4 and got[8:12] == [outer] * 4
    assert got[12:] == [[6], [6], [6, 22, 38, 54], [0, 5, 10, 15], [30]]
    y2 = f32([[1, 2, 3], [4, 5, 6]])
    _, outs = run(lambda p: [e("ij->ji", p), e("ji", p), e(p, [1, 0]), e(p, [0, 1], [1, 0])], y2)
    assert all(o.tolist() == [1, 4, 2, 5, 3, 6] for o in outs)
    tx, ty = f32(np.arange(30).reshape(2, 3, 5)), f32(np.arange(60).reshape(3, 4, 5))
    _, outs = run(lambda p, q: [e("ijk,jlk->il", p, q), e("ijk,jlk", p, q), e(p, [0, 1, 2], q, [1, 3, 2], [0, 3]), e(p, [0, 1, 2], q, [1, 3, 2])], tx, ty)
    assert all(o.tolist() == [3340, 3865, 4390, 4915, 8290, 9940, 11590, 13240] for o in outs)
    w, cx, cy, z = f32(np.arange(5, 9).reshape(2, 2)), f32(np.arange(6).reshape(2, 3)), f32(np.arange(-2, 4).reshape(3, 2)), f32([[2, 4, 6], [3, 5, 7]])
    _, outs = run(lambda p, q, r, t: [e("ij,jk,kl,lm->im", p, q, r, t), e(p, [0, 1], q, [1, 2], r, [2, 3], t, [3, 4])], w, cx, cy, z)
    assert all(o.tolist() == [481, 831, 1181, 651, 1125, 1599] for o in outs)
    table = [("", [], []), ("i,i->", [3], [3], []), ("ijj->i", [2, 3, 3], [2]), ("i,i->i", [3], [3], [3]), ("ij,j->i", [2, 3], [3], [2]),
             ("ij,ji", [3, 4], [4, 3], []), ("ij,jk", [2, 3], [3, 4], [2, 4]), ("ij,jk->ki", [2, 3], [3, 4], [4, 2]),
             ("abc,cde->abde", [2, 3, 4], [4, 5, 6], [2, 3, 5, 6]), ("abcd,cdef->abef", [2, 3, 4, 5], [4, 5, 6, 7], [2, 3, 6, 7]),
             ("abcd,efcd->abef", [2, 3, 4, 5], [6, 7, 4, 5], [2, 3, 6, 7]), ("abc,bcd,efa,fab", [2, 3, 4], [3, 4, 5], [10, 6, 2], [6, 2, 3], [5, 10]),
             ("...", [5, 1], [5, 1]), ("i...", [5, 1], [1, 5]), ("...,...->...", [2, 3, 4], [3, 4], [2, 3, 4]), ("...i,i->...", [2, 3, 4], [4], [2, 3]),
             ("i,...i->...", [4], [2, 3, 4], [2, 3]), ("...ij,jk->...ik", [5, 2, 3], [3, 4], [5, 2, 4]),
             ("...ij,...jk->...ik", [6, 5, 2, 3], [5, 3, 4], [6, 5, 2, 4]), ("ab...cd,cd...ef->ab...ef", [2, 3, 4, 5, 6, 7], [6, 7, 8, 9], [2, 3, 4, 5, 8, 9]),
             ("ii->i", [3, 3], [3]), ("ii->i", [3, 1], [1]), ("i,i->i", [3], [1], [3]), ("i,i->i", [1], [3], [3]), ("ii,i->i", [3, 3], [1], [3]),
             ("ii,i->i", [1, 1], [3], [3]), ("ij,ij->ij", [1, 10], [5, 1], [5, 10]), ("...,...->...", [1, 10], [5, 1], [5, 10])]
    rng = np.random.default_rng(5)
    for expr, *shapes in table:
        ins = [rng.integers(-3, 4, s).astype(np.float32) for s in shapes[:-1]]
        seen = {}
        _, (got,) = run(lambda *ops: seen.setdefault("r", e(expr, *ops)), *ins)
        assert list(seen["r"].shape) == shapes[-1], expr
        if not _needs_broadcast(expr, shapes):
            np.testing.assert_array_equal(got.reshape(shapes[-1]), np.einsum(expr if expr else "->", *ins))


def _needs_broadcast(expr, shapes):
    """Cases of the shape table that rely on size-1 broadcasting of a named index, which numpy.einsum refuses."""
    return (expr, shapes[:-1]) in [("ii->i", [[3, 1]]), ("i,i->i", [[3], [1]]), ("i,i->i", [[1], [3]]), ("ii,i->i", [[3, 3], [1]]),
                                   ("ii,i->i", [[1, 1], [3]]), ("ij,ij->ij", [[1, 10], [5, 1]])]


F16, F64 = DType.Float16, DType.Float64


def test_dtype_promotion_and_half_double_tables():
    """test/dtype.test.ts:8-150 (uint32 wrap-around; promotion of uint32 + int32, int32 * f16, uint32 - f32, bool + int32,
    f16 / f32; numbers are weak and take the array's dtype, also through jit), :152-195 (resultType);
    test/dtype-f16.test.ts:35-79 (signbit of -0, sum of squares, exact erfc gelu, reductions accumulate in f32) and
    :80-125 (a transposed convolution in f16); test/dtype-f64.test.ts:34-110 (signbit incl. the sign of a NaN, sum of
    squares, gelu, 1e-15 differences, unwrap at a rounding tie, polymul keeps double precision)."""
    sc = lambda v, t: np.asarray(v, t).reshape(())
    _, (u,) = _run_typed(lambda a, b: a.sub(b), [sc(3, np.uint32), sc(5, np.uint32)], [U32, U32])
    assert u.dtype == np.uint32 and u.tolist() == [4294967294]
    cases = [((3, np.uint32, U32), (-2, np.int32, I32), lambda a, b: a.add(b), np.int32, 1),
             ((3, np.int32, I32), (2.5, np.float16, F16), lambda a, b: a.mul(b), np.float16, 7.5),
             ((4, np.uint32, U32), (1.5, np.float32, F32), lambda a, b: a.sub(b), np.float32, 2.5),
             ((1, np.int32, BOOL), (10, np.int32, I32), lambda a, b: a.add(b), np.int32, 11),
             ((2.5, np.float16, F16), (1.5, np.float32, F32), lambda a, b: a.div(b), np.float32, 2.5 / 1.5)]
    for (va, na, da), (vb, nb, db), fn, want_dt, want in cases:
        _, (c,) = _run_typed(fn, [sc(va, na), sc(vb, nb)], [da, db])
        assert c.dtype == want_dt and abs(float(c[0]) - want) < 1e-6
    seen = {}
    _, (w1, w2, w3) = _run_typed(lambda a, b: [seen.setdefault("i", a.add(3)), seen.setdefault("u", b.add(2.8)), seen.setdefault("m", a.add(J.mul(3, 3)))], [sc(5, np.int32), sc(5, np.uint32)], [I32, U32])
    assert (w1.dtype, w1.tolist(), w2.dtype, w2.tolist(), w3.dtype, w3.tolist()) == (np.int32, [8], np.uint32, [7], np.int32, [14])
    assert not seen["i"].aval.weak and not seen["u"].aval.weak and not seen["m"].aval.weak
    J.jit(lambda a: seen.setdefault("w", J.mul(3, 5)), [ShapedArray((), F32)])
    assert seen["w"].dtype == F32 and seen["w"].aval.weak
    _, (s3,) = _run_typed(lambda h: seen.setdefault("s", J.sin(3)).add(h), [sc(2, np.float16)], [F16])
    assert seen["s"].dtype == F32 and seen["s"].aval.weak and s3.dtype == np.float16 and abs(float(s3[0]) - (math.sin(3) + 2)) < 5e-3
    for npdt, dt in ((np.int32, I32), (np.float32, F32)):
        _, (p,) = _run_typed(lambda a: a.add(3), [sc(4, npdt)], [dt])
        assert p.dtype == npdt and p.tolist() == [7]
    R = L.resultType
    t = lambda dt, weak=False: J.Tracer(J.Lit(0, ShapedArray((), dt, weak)))
    assert R(t(U32), t(I32)) == I32 and R(t(I32), t(F16)) == F16 and R(t(BOOL), t(I32)) == I32 and R(t(F16), t(F32)) == F32 and R(t(F32), t(F64)) == F64
    J.jit(lambda a, b, h: seen.update(r=[R(a, 3.5), R(2, h), R(1, 2.5), R(True, 2), R(3), R(True), R(b, h), J.add(J._raise(True), 2).dtype]) or a, [ShapedArray((2,), I32), ShapedArray((2,), F32), ShapedArray((3,), F16)])
    assert seen["r"] == [I32, F16, F32, U32, F32, BOOL, F32, U32]
    h = lambda v: np.asarray(v, np.float16)
    _, (sb,) = _run_typed(lambda a: L.signbit(a), [h([-1.5, -0.0, 0, 1.5])], [F16])
    _, (sq,) = _run_typed(lambda a: a.mul(a).sum(), [h(np.arange(10))], [F16])
    _, (ge,) = _run_typed(lambda a: L.gelu(a, approximate=False), [h([-1, 0, 1])], [F16])
    assert sb.tolist() == [1, 1, 0, 0] and sq.dtype == np.float16 and sq.tolist() == [285] and ge.dtype == np.float16
    np.testing.assert_allclose(ge.astype(np.float32), [-0.1587, 0.0, 0.8413], rtol=1e-3, atol=1e-6)
    _, (dd,) = _run_typed(lambda a: L.dot(a, a), [h([100, 1, 1, 1, 1, 1, 1, 1, 1])], [F16])
    _, (ss,) = _run_typed(lambda a: a.sum(), [h([16000, 1, 1, 1, 1, 1, 1, 1, 1])], [F16])
    assert dd.dtype == np.float16 and dd.tolist() == [10008] and ss.dtype == np.float16 and ss.tolist() == [16008]
    xh, kh = h([[[1, 2, 3], [4, 5, 6]]]), h([[[1, 0, -1], [2, 1, 0]], [[0, 1, 2], [-1, 0, 1]]])
    _, (ct,) = _run_typed(lambda a, k: L.convGeneralDilated(a, k, [1], [(2, 1)], lhsDilation=[2]), [xh, kh], [F16, F16])
    dil = np.zeros((1, 2, 5 + 3), np.float32)
    dil[:, :, 2:7:2] = xh
    want = np.array([[[(dil[0, :, i:i + 3] * kh[o].astype(np.float32)).sum() for i in range(6)] for o in range(2)]])
    assert ct.dtype == np.float16
    np.testing.assert_allclose(ct.astype(np.float32).reshape(want.shape), want, rtol=1e-3, atol=1e-3)
    d = lambda v: np.asarray(v, np.float64)
    _, (s64,) = _run_typed(lambda a: L.signbit(a), [d([-1.5, -0.0, 0, 1.5])], [F64])
    nans = np.array([0xFFF8000000000000, 0x7FF8000000000000], np.uint64).view(np.float64)
    _, (sn,) = _run_typed(lambda a: L.signbit(a), [nans], [F64])
    _, (q64,) = _run_typed(lambda a: a.mul(a).sum(), [d(np.arange(10))], [F64])
    _, (g64,) = _run_typed(lambda a: L.gelu(a, approximate=False), [d([-1, 0, 1])], [F64])
    assert s64.tolist() == [1, 1, 0, 0] and sn.tolist() == [1, 0] and q64.dtype == np.float64 and q64.tolist() == [285]
    np.testing.assert_allclose(g64, [-0.15865525, 0.0, 0.84134475], rtol=1e-5, atol=1e-7)
    _, (df,) = _run_typed(lambda a: J.shrink(a, [(1, 2)]).sub(J.shrink(a, [(0, 1)])), [d([1 + 1e-15, 1 + 2e-15])], [F64])
    assert abs(df[0] - 1e-15) < 5e-16
    _, (uw,) = _run_typed(lambda a: L.unwrap(a), [d([0, -3.1415926535897936])], [F64])
    assert uw.dtype == np.float64 and uw[1] == 3.1415926535897927
    _, (pm,) = _run_typed(lambda a, b: L.polymul(a, b), [d([1, 1e-12]), d([1, 1])], [F64, F64])
    assert pm.dtype == np.float64 and pm[1] == 1 + 1e-12


def test_cholesky_lu_eigvalsh_and_argreduce_tables():
    """test/lax-linalg.test.ts:24-84 (Cholesky 2x2, 3x3, a 512x512 blocked case, shape errors), :276-304 (LU with partial
    pivoting: factors, pivots, permutation; P A = L U on 30x30); test/numpy-linalg.test.ts:23-34 (cholesky symmetrises
    its input), :72-126 (eigvalsh: plain, batched, random 16x16, the lower triangle when not symmetrising);
    test/argreduce.test.ts:14-70 (first index on ties, negatives, all equal, every axis of a 2-D array)."""
    for x in (f32([[2, 1], [1, 2]]), f32([[4, 2, 1], [2, 5, 3], [1, 3, 6]])):
        _, (l,) = run(lambda a: L.cholesky(a), x)
        l = l.reshape(x.shape)
        assert np.all(np.triu(l, 1) == 0) and l[1, 0] != 0
        np.testing.assert_allclose(l @ l.T, x, rtol=1e-5)
    n = 512
    a = np.random.default_rng(n).standard_normal((n, n)).astype(np.float32)
    spd = (a.T.astype(np.float64) @ a + n * np.eye(n)).astype(np.float32)
    _, (lb,) = run(lambda m: L.cholesky(m), spd)
    lb = lb.reshape(n, n).astype(np.float64)
    assert np.abs(lb @ lb.T - spd).max() / np.abs(spd).max() < 1e-5
    for shp in ((2, 3), (3,)):
        with pytest.raises((ValueError, TypeError)):
            J.jit(lambda m: L.cholesky(m), [ShapedArray(shp, F32)])
    xs = f32([[4, 2.01], [1.99, 5]])
    _, (ls,) = run(lambda m: L.linalgCholesky(m), xs)
    ls = ls.reshape(2, 2)
    np.testing.assert_allclose(ls @ ls.T, (xs + xs.T) / 2, rtol=1e-5)
    _, (lu, piv, perm) = run(lambda m: list(J.lu(m)), f32([[4, 3], [6, 3]]))
    np.testing.assert_allclose(lu, [6, 3, 0.6666667, 1.0], rtol=1e-6)
    assert piv.tolist() == [1, 1] and perm.tolist() == [1, 0] and piv.dtype == np.int32
    A = np.random.default_rng(0).uniform(0, 1, (30, 30)).astype(np.float32)
    _, (pa, lu2) = run(lambda m: (lambda f: [L.matmul(J.gather(J._raise(L.eye(30)), [f[2]], [0], 0), m),
                                             L.matmul(L.tril(f[0], -1).add(L.eye(30)), L.triu(f[0]))])(J.lu(m)), A)
    np.testing.assert_allclose(pa, lu2, rtol=1e-5, atol=1e-6)
    _, (e1, e2, e3) = run(lambda p, q, r: [L.eigvalsh(p), L.eigvalsh(q), L.eigvalsh(r, symmetrizeInput=False)], f32([[2, 1], [1, 2]]),
                          f32([[[2, 1], [1, 2]], [[3, 1], [1, 3]]]), f32([[2, 100], [1, 2]]))
    np.testing.assert_allclose(e1, [1, 3], rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(e2, [1, 3, 2, 4], rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(e3, [1, 3], rtol=1e-4, atol=1e-4)
    _, (er,) = run(lambda m: L.eigvalsh(m), np.random.default_rng(0).standard_normal((16, 16)).astype(np.float32))
    assert np.abs(er).sum() > 1
    _, (m1, m2, m3) = run(lambda p, q, r: [L.argmax(p), L.argmax(q), L.argmax(r)], f32([3, 5, 5, 2, 5, 1]), f32([-10, -5, -20, -5, -15]), np.ones(5, np.float32))
    assert (m1.tolist(), m2.tolist(), m3.tolist()) == ([1], [1], [0]) and m1.dtype == np.int32
    g = f32([[1, 2, 3], [6, 5, 4], [7, 8, 9]])
    _, (a0, a1, a2) = run(lambda p: [L.argmax(p), L.argmax(p, 0), L.argmax(p, 1)], g)
    assert (a0.tolist(), a1.tolist(), a2.tolist()) == ([8], [2, 2, 2], [2, 0, 2])
    _, (n1, n2) = run(lambda p, q: [L.argmin(p), L.argmin(q)], f32([3, 1, 5, 1, 1, 2]), np.full(5, 42, np.float32))
    assert n1.tolist() == [1] and n2.tolist() == [0]
    h = f32([[9, 8, 7], [4, 5, 6], [3, 2, 1]])
    _, (b0, b1, b2) = run(lambda p: [L.argmin(p), L.argmin(p, 0), L.argmin(p, 1)], h)
    assert (b0.tolist(), b1.tolist(), b2.tolist()) == ([8], [2, 2, 2], [2, 0, 2])


def test_frexp_ldexp_and_flips():
    """numpy.ts:2788-2809 (ldexp, frexp) and :1099-1107 (flipud / fliplr) against numpy on exactly representable values."""
    x = f32([1, 8, 0.75, -6, 0, 1024])
    _, (m, e, back) = run(lambda a: (lambda me: me + [L.ldexp(me[0], me[1].astype(F32))])(L.frexp(a)), x)
    wm, we = np.frexp(x)
    np.testing.assert_allclose(m, wm, rtol=2e-6, atol=1e-7)
    assert e.dtype == np.int32 and e.tolist() == we.tolist()
    np.testing.assert_allclose(back, x, rtol=2e-6)
    mm = f32([[1, 2, 3], [4, 5, 6]])
    _, (u, l) = run(lambda a: [L.flipud(a).mul(1), L.fliplr(a).mul(1)], mm)
    assert u.tolist() == [4, 5, 6, 1, 2, 3] and l.tolist() == [3, 2, 1, 6, 5, 4]


def test_jit_cases_of_the_tracing_suite():
    """test/tracing.test.ts:578-625 (the jit() cases that need no other transformation): a cubic, the identity, the same
    value returned twice, a gather by a constant index array, a static argument (a Python value closed over), a traced
    function calling traced functions."""
    _, (c,) = run(lambda a: a.mul(a).mul(a), f32(2).reshape(()))
    assert c.tolist() == [8]
    _, (i,) = run(lambda a: a, f32(3).reshape(()))
    _, (d1, d2) = run(lambda a: [a, a], f32(3).reshape(()))
    assert i.tolist() == [3] and d1.tolist() == [3] and d2.tolist() == [3]
    idx = np.array([1, 3, 2, 0], np.int32)
    _, (g,) = _run_typed(lambda a, ix: J.gather(a, [ix], [0], 0), [f32([10, 20, 30, 40]), idx], [F32, I32])
    assert g.tolist() == [20, 40, 30, 10]
    pick = lambda k: (lambda a: J.shrink(a, [(k, k + 1)]).reshape([]))
    _, (s0,) = _run_typed(pick(0), [_i32(np.arange(20))], [I32])
    _, (s3,) = _run_typed(pick(3), [_i32(np.arange(20))], [I32])
    _, (s11,) = run(pick(3), f32([30, 1, 20, 11]))
    assert s0.tolist() == [0] and s3.tolist() == [3] and s11.tolist() == [11]
    f = lambda a: a.mul(a)
    g2 = lambda a: f(f(a))
    _, (q,) = run(g2, f32(3).reshape(()))
    assert q.tolist() == [81]


def test_array_suite_tables():
    """src/frontend/array.test.ts: construction and elementwise product with a transposed read (:177-187), broadcasting
    [2,1,2]*[2,3,1] (:189-216), flatten/ravel (:218-229), an array added to itself twice (:231-236), booleans and the six
    comparisons (:248-281, incl. arange(5000)+1 < 2500), comparisons against NaN (:283-292), slicing with ints, negative
    ints, ranges and new axes (:294-321), sums along negative axes (:323-330), means over several axes (:332-342), integer
    array indexing as gather (:344-363), uint32 wrap-around (:390-400), casts (:402-413), saturating casts (:415-432),
    bit views and their type rules (:434-482)."""
    a, b = f32([1, 2, 3, 4]), f32([10, 5, 2, -8.5])
    _, (c, ct) = run(lambda p, q: [p.mul(q), p.mul(q).reshape([2, 2]).transpose()], a, b)
    assert c.tolist() == [10, 10, 6, -34] and ct.tolist() == [10, 6, 10, -34]
    p, q = f32([[1, 22], [3, 9]]), f32([[10, 5, -2], [-8, 0, 3]])
    seen = {}
    _, (o,) = run(lambda u, v: seen.setdefault("o", u.reshape([2, 1, 2]).mul(v.reshape([2, 3, 1]))), p, q)
    assert tuple(seen["o"].shape) == (2, 3, 2)
    assert o.reshape(2, 3, 2).tolist() == [[[10, 220], [5, 110], [-2, -44]], [[-24, -72], [0, 0], [9, 27]]]
    _, (fl, rv, sc) = run(lambda u, s: [u.flatten().mul(1), u.ravel().mul(1), s.flatten().mul(1)], f32([[[1, 2], [3, 4]]]), f32(3))
    assert fl.tolist() == [1, 2, 3, 4] and rv.tolist() == [1, 2, 3, 4] and sc.tolist() == [3]
    _, (tw,) = run(lambda u: u.add(u).add(u), f32([1, 2, 3]))
    assert tw.tolist() == [3, 6, 9]
    # booleans are int32 0/1 in memory; comparisons
    x = f32([1, 3, 4])
    _, (g2, e3, ne) = run(lambda u, v: [u.greater(2), u.equal(3), u.notEqual(v)], x, f32([2, 3, 4]))
    assert g2.dtype == np.int32 and g2.tolist() == [0, 1, 1] and e3.tolist() == [0, 1, 0] and ne.tolist() == [1, 0, 0]
    _, outs = run(lambda u: [u.greater(2), u.greaterEqual(2), u.less(2), u.lessEqual(2), u.equal(2), u.notEqual(2)], f32([1, 2, 3]))
    assert [o_.tolist() for o_ in outs] == [[0, 0, 1], [0, 1, 1], [1, 0, 0], [1, 1, 0], [0, 1, 0], [1, 0, 1]]
    (lt,) = run0(lambda: J._raise(L.arange(0, 5000, 1, F32)).add(1).less(2500))
    assert lt.tolist() == [1 if i + 1 < 2500 else 0 for i in range(5000)]
    nan = float("nan")
    _, outs = run(lambda u: [u.greater(nan), u.less(nan), u.equal(nan), u.notEqual(nan), u.greaterEqual(nan), u.lessEqual(nan)], f32([nan, 0]))
    assert [o_.tolist() for o_ in outs] == [[0, 0], [0, 0], [0, 0], [1, 1], [0, 0], [0, 0]]
    # slicing
    m = f32([[1, 2, 3], [4, 5, 6]])
    shapes = []

    def pick(u):
        outs_ = [u.slice(0, 0), u.slice(0, 2), u.slice(1, 2), u.slice(1), u.slice(), u.slice(-1, -1), u.slice(-2, -1), u.slice(-1, -3),
                 u.slice(0, 0, None), u.slice(0, None, 0), u.slice(None), u.slice([], [1]), u.slice([0, 1], [1, 3]), u.slice(None, 1, None, [0, 2])]
        shapes.extend(tuple(o_.shape) for o_ in outs_)
        return [o_.mul(1) for o_ in outs_]

    _, outs = run(pick, m)
    assert shapes == [(), (), (), (3,), (2, 3), (), (), (), (1,), (1,), (1, 2, 3), (2, 2), (1, 2), (1, 1, 2)]
    assert [o_.tolist() for o_ in outs] == [[1], [3], [6], [4, 5, 6], [1, 2, 3, 4, 5, 6], [6], [3], [4], [1], [1], [1, 2, 3, 4, 5, 6],
                                           [2, 3, 5, 6], [2, 3], [4, 5]]
    for bad in ((3,), (0, 4), (-3,), (0, 0, 0), ([2, 1],), ("x",)):
        with pytest.raises((IndexError, TypeError)):
            J.jit(lambda u: u.slice(*bad), [ShapedArray((2, 3), F32)])
    _, (s1, s2) = run(lambda u: [u.sum(-1), u.sum(-2)], m)
    assert s1.tolist() == [6, 15] and s2.tolist() == [5, 7, 9]
    _, (m0, m01, ma, mb) = run(lambda u: [u.mean(), u.mean([0, 1]), u.mean(0), u.mean(1)], m)
    assert m0.tolist() == [3.5] and m01.tolist() == [3.5] and ma.tolist() == [2.5, 3.5, 4.5] and mb.tolist() == [2, 5]
    # integer arrays as indices: np.eye(5)[[1,3,2]], np.eye(5)[[1,3,2], np.newaxis], np.eye(5)[1:4, [1,3,2]]
    idx = np.array([1, 3, 2], np.int32)
    shapes = []

    def adv(i):
        e = J._raise(L.eye(5))
        outs_ = [e.slice(i), e.slice(i, None), e.slice([1, 4], i)]
        shapes.extend(tuple(o_.shape) for o_ in outs_)
        return outs_

    _, (g0, g1, g2) = run_typed(adv, [idx], [I32])
    assert shapes == [(3, 5), (3, 1, 5), (3, 3)]
    assert g0.reshape(3, 5).tolist() == np.eye(5)[idx].tolist() and g1.reshape(3, 5).tolist() == np.eye(5)[idx].tolist()
    assert g2.reshape(3, 3).tolist() == np.eye(5)[1:4, idx].tolist()
    # numpy's placement rule when ints and arrays are apart: x[:, i, :, 1] puts the index dimensions first
    t4 = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    shapes = []
    _, (apart, together) = run_typed(lambda u, i: [shapes.append(tuple(u.slice([], i, [], 1).shape)) or u.slice([], i, [], 1),
                                                    shapes.append(tuple(u.slice([], i, 2).shape)) or u.slice([], i, 2)], [t4, np.array([2, 0], np.int32)], [F32, I32])
    assert shapes == [(2, 2, 4), (2, 2, 5)]
    np.testing.assert_array_equal(apart.reshape(2, 2, 4), t4[:, [2, 0], :, 1])
    np.testing.assert_array_equal(together.reshape(2, 2, 5), t4[:, [2, 0], 2])
    # uint32 wraps, casts, saturation
    _, (w,) = run_typed(lambda u, two: u.sub(two), [np.array([1, 2, 3], np.uint32), np.array(2, np.uint32)], [DType.Uint32, DType.Uint32])
    assert w.dtype == np.uint32 and w.tolist() == [4294967295, 0, 1]
    _, (cf,) = run_typed(lambda u: u.astype(F32), [np.array([1, 2, 3], np.int32)], [I32])
    assert cf.dtype == np.float32 and cf.tolist() == [1, 2, 3]
    big = f32([1e20, -1e20, 1e10, -1e10, 1e5, -1e5])
    _, (si, su) = run(lambda u: [u.astype(I32), u.astype(DType.Uint32)], big)
    assert si.tolist() == [2147483647, -2147483648, 2147483647, -2147483648, 100000, -100000]
    assert su.tolist() == [4294967295, 0, 4294967295, 0, 100000, 0]
    # bit views
    _, (vi, back) = run(lambda u: [u.view(I32), u.view(I32).view(F32)], f32([1.0, 2.0]))
    assert vi.dtype == np.int32 and vi.tolist() == [1065353216, 1073741824] and back.tolist() == [1.0, 2.0]
    _, (vf,) = run_typed(lambda u: u.view(F32), [np.array([1065353216, 1073741824], np.int32)], [I32])
    assert vf.dtype == np.float32 and vf.tolist() == [1.0, 2.0]
    same = {}
    _, (idn,) = run(lambda u: same.setdefault("v", u.view(F32)).mul(1), f32([1, 2, 3]))
    assert idn.tolist() == [1, 2, 3]
    with pytest.raises(TypeError):
        J.jit(lambda u: u.view(I32), [ShapedArray((2,), DType.Bool)])
    with pytest.raises(TypeError):
        J.jit(lambda u: u.view(DType.Bool), [ShapedArray((2,), I32)])
    with pytest.raises(TypeError):
        J.jit(lambda u: u.view(DType.Float16), [ShapedArray((2,), I32)])
    _, (sp,) = run(lambda u: u.view(I32).view(F32), f32([np.inf, -np.inf, np.nan]))
    assert sp[0] == np.inf and sp[1] == -np.inf and np.isnan(sp[2])
