"""Helpers for replaying a traced JitProgram on a backend (the hip backend or the oracle one)."""
import numpy as np

from jaxjs_hip.alu import numpyDtype


def run_program(backend, prog, arrays, out_dtypes_shapes=None):
    """Realise the program's constants with their nullary kernels, upload `arrays`, execute, read back.
    Returns one flat typed numpy array per program output; every slot is released again."""
    const_slots = []
    for c in prog.consts:
        k = c.kernel()
        s = backend.malloc(k.bytes)
        backend.dispatch(backend.prepareKernelSync(k), [], [s])
        const_slots.append(s)
    in_slots = [backend.malloc(np.ascontiguousarray(a).nbytes, np.ascontiguousarray(a).tobytes()) for a in arrays]
    outs = prog.execute(backend, const_slots + in_slots)
    results = []
    out_dtypes = {}
    for s in prog.steps:
        if s.kind == "execute" and s.routine is not None:
            out_dtypes.update(zip(s.outputs, s.routine.type.outputDtypes))
        elif s.kind == "execute":
            out_dtypes[s.output] = s.kernel.dtype
    for slot, oid in zip(outs, prog.outputs):
        raw = backend.readSync(slot)
        if oid in out_dtypes:
            dt = numpyDtype(out_dtypes[oid])
        elif oid < len(prog.consts):  # a constant returned as it is
            dt = numpyDtype(prog.consts[oid].dtype)
        else:  # an input returned as it is
            dt = np.asarray(arrays[oid - len(prog.consts)]).dtype
        results.append(np.frombuffer(raw, dtype=dt).copy())
    for s in const_slots + in_slots + outs:
        backend.decRef(s)
    return results
