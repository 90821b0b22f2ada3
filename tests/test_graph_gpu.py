"""A jit program replayed as one HIP graph: every replay must equal the eager run of the same program, also
with unrelated eager work and synchronisation between replays and after the inputs were overwritten in place."""
import numpy as np
import pytest

from gpu_util import WARM_ONLY, backend
from jaxjs_hip import workloads as W
from jaxjs_hip.alu import numpyDtype
from jaxjs_hip.graph import GraphedProgram
from jit_util import run_program
from test_jit import block_inputs

pytestmark = pytest.mark.gpu


def _eager(be, prog, arrays):
    return run_program(be, prog, arrays)


def _check_program(prog, make_arrays, rounds=3):
    be = backend()
    const_slots = []
    for c in prog.consts:
        k = c.kernel()
        s = be.malloc(k.bytes)
        be.dispatch(be.prepareKernelSync(k), [], [s])
        const_slots.append(s)
    arrays = make_arrays(0)
    in_slots = [be.malloc(a.nbytes, a.tobytes()) for a in arrays]
    g = GraphedProgram(be, prog, const_slots + in_slots)
    out_dtypes = {}
    for s in prog.steps:
        if s.kind == "execute" and s.routine is not None:
            out_dtypes.update(zip(s.outputs, s.routine.type.outputDtypes))
        elif s.kind == "execute":
            out_dtypes[s.output] = s.kernel.dtype
    try:
        for r in range(rounds):
            if r > 0:  # new input values, written into the slots the graph was captured with
                arrays = make_arrays(r)
                for slot, a in zip(in_slots, arrays):
                    be.dev.h2d(be.slotPointer(slot), a.tobytes())
            want = _eager(be, prog, arrays)  # eager work (allocations, launches, reads) between replays
            g.launch()
            g.launch()  # back-to-back replays are fine too: same inputs, same outputs
            for slot, oid, w in zip(g.outputs, prog.outputs, want):
                got = np.frombuffer(be.readSync(slot), dtype=numpyDtype(out_dtypes[oid]))
                np.testing.assert_array_equal(got.view(np.uint8), w.view(np.uint8), err_msg=f"replay {r}")
    finally:
        g.close()
        for s in const_slots + in_slots:
            be.decRef(s)


def test_row_softmax_argmax_graph():
    prog = W.rowSoftmaxArgmaxProgram(128, 777)
    if WARM_ONLY:
        pytest.skip("kernels are compiled by the program tests")
    _check_program(prog, lambda r: [np.random.default_rng(r).standard_normal((128, 777)).astype(np.float32)])
    assert len([s for s in prog.steps if s.kind == "execute"]) == 4


def test_gpt2_block_graph():
    batch, seq, d, heads, d_ff = 2, 64, 128, 2, 512
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff)
    if WARM_ONLY:
        pytest.skip("kernels are compiled by the program tests")
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)

    def arrays(r):
        a = block_inputs(batch, seq, d, d_ff, np.float16, seed=100 + r)
        return [a[n] for n in order]
    _check_program(prog, arrays)


def test_graph_replay_of_programs_with_routine_steps():
    """Routine steps (several launches, several outputs) are captured like kernels: LU + triangular solves (`solve`) and
    the block with the fused-attention routine replay bit for bit what the eager path gives."""
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    from jaxjs_hip.alu import DType
    from jaxjs_hip.jit import ShapedArray
    solve = J.jit(lambda x, y: L.solve(x, y), [ShapedArray((4, 40, 40), DType.Float32), ShapedArray((4, 40, 3), DType.Float32)])
    batch, seq, d, heads, d_ff = 2, 128, 128, 2, 512
    block = W.gpt2BlockProgram(batch, seq, d, heads, d_ff, fusedAttention=True)
    assert solve.routines and block.routines
    if WARM_ONLY:
        pytest.skip("kernels are compiled by the program tests")

    def systems(r):
        rng = np.random.default_rng(r)
        return [(rng.standard_normal((4, 40, 40)) + 6 * np.eye(40)).astype(np.float32), rng.standard_normal((4, 40, 3)).astype(np.float32)]
    _check_program(solve, systems)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)

    def arrays(r):
        a = block_inputs(batch, seq, d, d_ff, np.float16, seed=200 + r)
        return [a[n] for n in order]
    _check_program(block, arrays)


def test_graph_replay_of_a_k_split_folded_inside_the_launch():
    """An f32 matmul small enough that its k axis is cut over workgroups and folded inside the launch (per-tile counters
    that every launch must leave at zero): replays of the captured graph equal the eager run bit for bit."""
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    from jaxjs_hip.alu import DType
    from jaxjs_hip.jit import ShapedArray
    M, K, N = 256, 2048, 192
    prog = J.jit(lambda a, b: L.matmul(a, b), [ShapedArray((M, K), DType.Float32), ShapedArray((K, N), DType.Float32)])
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        for k in prog.kernels:
            for src in generate(k).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    info = be.prepareKernelSync(prog.kernels[0]).data.ks.info
    assert info.get("fused_fold") and info["splitk"] > 1, info

    def operands(r):
        rng = np.random.default_rng(300 + r)
        return [rng.uniform(-1, 1, (M, K)).astype(np.float32), rng.uniform(-1, 1, (K, N)).astype(np.float32)]
    _check_program(prog, operands)
