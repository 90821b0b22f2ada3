"""The fused attention kernel (an extension routine, `Routines.Attention`) on the GPU against the float64 checker, and
the GPT-2 block traced with it against the block traced the reference's way.  Float16 in, float16 out, f32 softmax
statistics: bound = 1e-2 relative + a few f16 ulps of values of order 1 (the stated f16 tolerance)."""
import math

import numpy as np
import pytest

import routine_util as R
from gpu_util import WARM_ONLY, backend
from jaxjs_hip import DType
from jaxjs_hip import workloads as W
from jaxjs_hip.errors import UnsupportedRoutineError
from jaxjs_hip.routine import Routine, Routines, RoutineType
from jit_util import run_program
from test_jit import block_inputs, block_reference

pytestmark = pytest.mark.gpu
F16 = DType.Float16


def attention_routine(B, L, S, N, causal, scale=None, H=64):
    t = RoutineType([[B, L, N, H], [B, S, N, H], [B, S, N, H]], [F16] * 3, [[B, L, N, H]], [F16])
    return Routine(Routines.Attention, t, dict(scale=1 / math.sqrt(H) if scale is None else scale, isCausal=causal))


CASES = [(1, 128, 64, 1, 64), (1, 128, 128, 1, 64), (2, 256, 256, 3, 64), (1, 384, 192, 2, 64), (1, 128, 320, 2, 64), (2, 1024, 1024, 4, 64),
         # other head sizes, and lengths that are not whole tiles (a last query block and a last key tile that are partly
         # empty, fewer queries than a wave holds, one key)
         (2, 256, 256, 2, 32), (1, 256, 192, 3, 128), (1, 100, 128, 1, 64), (1, 128, 100, 1, 64), (2, 77, 333, 3, 32), (1, 130, 65, 2, 128),
         (1, 1, 1, 1, 64), (3, 5, 700, 2, 64), (1, 1000, 1000, 2, 128), (2, 513, 511, 1, 32)]


@pytest.mark.parametrize("causal", [False, True], ids=["full", "causal"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_L%d_S%d_N%d_H%d" % c)
def test_attention_matches_float64(case, causal):
    B, L, S, N, H = case
    rng = np.random.default_rng(B * 1000 + L + S + N + H)
    q, k, v = [rng.standard_normal((B, T, N, H)).astype(np.float16) for T in (L, S, S)]
    routine = attention_routine(B, L, S, N, causal, H=H)
    got, ks = R.run_gpu(routine, [q, k, v])
    want = R.run_oracle(routine, [q, k, v])
    np.testing.assert_allclose(got[0].astype(np.float64), want[0].astype(np.float64), rtol=1e-2, atol=3e-3, err_msg=str(ks.info))


def test_attention_is_stable_for_large_scores_and_peaked_rows():
    rng = np.random.default_rng(4)
    q, k, v = [rng.standard_normal((1, 256, 2, 64)).astype(np.float16) for _ in range(3)]
    q *= np.float16(6.0)   # scores of order +-50: exp would overflow f16/f32 without the running maximum
    k[:, 17] *= np.float16(4.0)  # one dominant key
    for causal in (False, True):
        routine = attention_routine(1, 256, 256, 2, causal, scale=1.0)
        got, _ = R.run_gpu(routine, [q, k, v])
        want = R.run_oracle(routine, [q, k, v])
        assert np.isfinite(got[0]).all()
        np.testing.assert_allclose(got[0].astype(np.float64), want[0].astype(np.float64), rtol=1e-2, atol=4e-3)


@pytest.mark.parametrize("scale", [-0.125, 0.0, 1e-3, 3.0], ids=lambda s: "scale%g" % s)
def test_attention_takes_any_scale(scale):
    """A scale that is zero or negative does not commute with the row maximum (the kernel then scales the scores before
    taking it); ragged lengths so the masked key tile and the diagonal are covered under both forms."""
    rng = np.random.default_rng(11)
    q, k, v = [rng.standard_normal((2, T, 2, 64)).astype(np.float16) for T in (200, 200, 200)]
    for causal in (False, True):
        routine = attention_routine(2, 200, 200, 2, causal, scale=scale)
        got, _ = R.run_gpu(routine, [q, k, v])
        want = R.run_oracle(routine, [q, k, v])
        assert np.isfinite(got[0]).all()
        np.testing.assert_allclose(got[0].astype(np.float64), want[0].astype(np.float64), rtol=1e-2, atol=4e-3)


def _view(strides, offset, shape):
    return dict(strides=list(strides), offset=offset, elements=offset + sum((d - 1) * s for d, s in zip(shape, strides)) + 1)


@pytest.mark.parametrize("causal", [False, True], ids=["full", "causal"])
def test_attention_reads_operands_through_strides(causal):
    """q, k and v as three windows of one [B, L, 3*N*64] buffer (the output of a fused QKV projection), and k/v stored
    head-major ([B, N, S, 64]): the routine takes the base buffers with strides and offsets, no copies."""
    B, L, N, H = 2, 256, 3, 64
    rng = np.random.default_rng(11)
    qkv = rng.standard_normal((B, L, 3 * N * H)).astype(np.float16)
    t = RoutineType([[B, L, N, H]] * 3, [F16] * 3, [[B, L, N, H]], [F16])
    st = (L * 3 * N * H, 3 * N * H, H, 1)
    views = [_view(st, i * N * H, (B, L, N, H)) for i in range(3)]
    routine = Routine(Routines.Attention, t, dict(scale=0.125, isCausal=causal, views=views))
    got, ks = R.run_gpu(routine, [qkv, qkv, qkv])
    q, k, v = [qkv[..., i * N * H:(i + 1) * N * H].reshape(B, L, N, H) for i in range(3)]
    want = R.run_oracle(attention_routine(B, L, L, N, causal), [q, k, v])
    np.testing.assert_allclose(got[0].astype(np.float64), want[0].astype(np.float64), rtol=1e-2, atol=3e-3)
    np.testing.assert_array_equal(R.run_oracle(routine, [qkv, qkv, qkv])[0], want[0])  # the checker reads views too
    # head-major keys and values, contiguous queries
    kh, vh = [np.ascontiguousarray(np.transpose(a, (0, 2, 1, 3))) for a in (k, v)]
    hm = _view((N * L * H, H, L * H, 1), 0, (B, L, N, H))
    routine = Routine(Routines.Attention, t, dict(scale=0.125, isCausal=causal, views=[None, hm, hm]))
    got2, _ = R.run_gpu(routine, [np.ascontiguousarray(q), kh, vh])
    np.testing.assert_array_equal(got2[0], got[0])


def test_strided_operands_the_kernel_cannot_load_are_refused():
    if WARM_ONLY:
        pytest.skip("nothing to compile")
    B, L, N, H = 1, 128, 1, 64
    t = RoutineType([[B, L, N, H]] * 3, [F16] * 3, [[B, L, N, H]], [F16])
    for bad in (_view((L * N * H, N * H, H, 1), 4, (B, L, N, H)), _view((L * N * H * 2, N * H * 2, H * 2, 2), 0, (B, L, N, H)),
                _view((L * 68, 68, 68, 1), 0, (B, L, N, H))):
        with pytest.raises(UnsupportedRoutineError):
            backend().prepareRoutineSync(Routine(Routines.Attention, t, dict(scale=0.125, isCausal=False, views=[bad, None, None])))


def test_shapes_outside_the_kernel_are_refused_not_faked():
    if WARM_ONLY:
        pytest.skip("nothing to compile")
    be = backend()
    t32 = RoutineType([[1, 128, 1, 64]] * 3, [DType.Float32] * 3, [[1, 128, 1, 64]], [DType.Float32])
    for routine in (attention_routine(1, 128, 128, 1, False, H=16), attention_routine(1, 128, 128, 1, False, H=96),
                    Routine(Routines.Attention, t32, dict(scale=0.125, isCausal=False))):
        with pytest.raises(UnsupportedRoutineError):
            be.prepareRoutineSync(routine)


def test_reference_attention_tables_on_the_fused_kernel():
    """test/nn.test.ts:275-390 on the fused kernel.  The tables use head sizes of 2 and 4; the operands are padded with
    zeros to 32 (dot products and the meaningful output columns are unchanged) and the scale is the table's own
    1/sqrt(H).  Two or three queries and keys: every tile is ragged."""
    def run(q, k, v, scale, causal):
        H0 = np.asarray(q).shape[-1]
        pad = lambda a: np.pad(np.asarray(a, np.float16), [(0, 0)] * 3 + [(0, 32 - H0)])  # noqa: E731
        q, k, v = pad(q), pad(k), pad(v)
        routine = attention_routine(q.shape[0], q.shape[1], k.shape[1], q.shape[2], causal, scale=scale, H=32)
        got, _ = R.run_gpu(routine, [q, k, v])
        out = got[0].astype(np.float64).reshape(q.shape)
        assert not out[..., H0:].any()
        return out[..., :H0]
    q = [[[[1, 0, 0, 0]], [[0, 1, 0, 0]]]]
    out = run(q, q, [[[[1, 2, 3, 4]], [[5, 6, 7, 8]]]], 0.5, False)
    np.testing.assert_allclose(out[0, 0, 0], [0.62245935 * a + 0.37754068 * b for a, b in zip((1, 2, 3, 4), (5, 6, 7, 8))], rtol=2e-3)
    e = [[[[1, 0]], [[0, 1]]]]
    out = run(e, e, e, 1.0, False)
    np.testing.assert_allclose(out[0, 0, 0], [0.7310586, 0.26894143], rtol=2e-3)
    out = run([[[[1, 0]], [[0.2, 0.2]], [[1, 1]]]], [[[[1, 0]], [[0, 1]], [[1, 1]]]], [[[[1, 0]], [[0, 1]], [[0, 0]]]], 1 / math.sqrt(2), True)
    np.testing.assert_allclose(out[0, 0, 0], [1, 0], atol=1e-3)
    np.testing.assert_allclose(out[0, 1, 0], [0.5, 0.5], rtol=2e-3)
    np.testing.assert_allclose(out[0, 2, 0], [1 / (2 + math.exp(math.sqrt(0.5)))] * 2, rtol=2e-3)


def test_gpt2_block_with_fused_attention():
    """Small block (d=128, 2 heads of 64): fused against the float64 block restatement and against the unfused program
    on the same GPU.  The front-end switch falls back to the reference's composition when the shapes do not fit."""
    batch, seq, d, heads, d_ff = 2, 128, 128, 2, 512
    fused = W.gpt2BlockProgram(batch, seq, d, heads, d_ff, fusedAttention=True)
    plain = W.gpt2BlockProgram(batch, seq, d, heads, d_ff)
    assert [r.name for r in fused.routines] == [Routines.Attention] and not plain.routines
    assert len(fused.kernels) == len(plain.kernels) - 7  # seven attention kernels out; q, k, v are views of the QKV output
    assert all(v is not None for v in fused.routines[0].params["views"])
    assert not W.gpt2BlockProgram(batch, seq, d, 8, d_ff, fusedAttention=True).routines  # heads of 16: composition kept
    assert W.gpt2BlockProgram(batch, 100, d, 4, d_ff, fusedAttention=True).routines     # heads of 32, a ragged length: fused
    if WARM_ONLY:
        from test_programs_gpu import warm
        warm(fused)
    arrs = block_inputs(batch, seq, d, d_ff, np.float16)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    arrays = [arrs[n] for n in order]
    (y,) = run_program(backend(), fused, arrays)
    (y0,) = run_program(backend(), plain, arrays)
    want = block_reference(arrs["x"].astype(np.float64), {n: arrs[n].astype(np.float64) for n in order[1:]}, heads)
    np.testing.assert_allclose(y.astype(np.float64).reshape(batch, seq, d), want, rtol=3e-2, atol=3e-2)
    np.testing.assert_allclose(y.astype(np.float64), y0.astype(np.float64), rtol=2e-2, atol=2e-2)
