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
