"""Helpers of the routine tests: build a Routine from arrays, run it through the CPU checker and through the
`hip` backend (C-ABI path)."""
import numpy as np
import pytest

from jaxjs_hip import DType
from jaxjs_hip.alu import byteWidth, numpyDtype
from jaxjs_hip.routine import Routine, Routines, RoutineType
from jaxjs_hip.shape import prod
from oracle.routines import runCpuRoutine

NP2DT = {np.dtype(np.float32): DType.Float32, np.dtype(np.int32): DType.Int32, np.dtype(np.uint32): DType.Uint32,
         np.dtype(np.float16): DType.Float16, np.dtype(np.float64): DType.Float64}


def routine_for(name, arrays, out_shapes, out_dtypes, params=None, in_dtypes=None):
    in_dtypes = in_dtypes or [NP2DT[np.asarray(a).dtype] for a in arrays]
    t = RoutineType([list(np.asarray(a).shape) for a in arrays], list(in_dtypes), [list(s) for s in out_shapes], list(out_dtypes))
    return Routine(name, t, params)


def _outputs(routine, raw):
    t = routine.type
    return [np.frombuffer(bytes(b), dtype=numpyDtype(dt)).reshape(shape).copy() for b, dt, shape in zip(raw, t.outputDtypes, t.outputShapes)]


def run_oracle(routine, arrays):
    t = routine.type
    bufs = [bytearray(prod(s) * byteWidth(dt)) for s, dt in zip(t.outputShapes, t.outputDtypes)]
    runCpuRoutine(routine, [np.ascontiguousarray(a).tobytes() for a in arrays], bufs)
    return _outputs(routine, bufs)


def run_gpu(routine, arrays, poison=True):
    """Prepare + dispatch on the GPU.  Output slots start filled with 0xA5 so that an element a routine fails to
    initialise shows up."""
    from gpu_util import WARM_ONLY, backend
    if WARM_ONLY:
        from jaxjs_hip.routinegen import generateRoutine
        from jaxjs_hip.runtime import compile_source
        for src in generateRoutine(routine).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    exe = be.prepareRoutineSync(routine)
    t = routine.type
    ins = [be.malloc(np.asarray(a).nbytes, np.ascontiguousarray(a).tobytes()) for a in arrays]
    sizes = [prod(s) * byteWidth(dt) for s, dt in zip(t.outputShapes, t.outputDtypes)]
    outs = [be.malloc(n, b"\xa5" * n if poison else None) for n in sizes]
    try:
        be.dispatch(exe, ins, outs)
        raw = [be.readSync(o) for o in outs]
    finally:
        for s in ins + outs:
            be.decRef(s)
    return _outputs(routine, raw), exe.data.ks


def bits_equal(a, b):
    """Same shape, type and bit patterns; NaNs count as one value (JavaScript has a single NaN, and which payload a
    typed-array store keeps is not specified)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.dtype.kind == "f":
        a, b = np.where(np.isnan(a), a.dtype.type(np.nan), a), np.where(np.isnan(b), b.dtype.type(np.nan), b)
    return a.tobytes() == b.tobytes()


# Routine constructors in the shapes the reference's front-end hands a backend.
def cholesky(a):
    return routine_for(Routines.Cholesky, [a], [a.shape], [NP2DT[a.dtype]])


def triangular_solve(a, b, unit_diagonal=False):
    return routine_for(Routines.TriangularSolve, [a, b], [b.shape], [NP2DT[b.dtype]], dict(unitDiagonal=unit_diagonal))


def lu(a):
    m, n = a.shape[-2:]
    batch = list(a.shape[:-2])
    return routine_for(Routines.LU, [a], [a.shape, batch + [min(m, n)], batch + [m]], [NP2DT[a.dtype], DType.Int32, DType.Int32])


def jacobi_eigh(a, max_sweeps=30, tolerance=1e-7):
    return routine_for(Routines.JacobiEigh, [a], [a.shape, a.shape], [NP2DT[a.dtype]] * 2, dict(maxSweeps=max_sweeps, tolerance=tolerance))


def factor_fft_size(n):
    """The front-end's factorisation (src/library/numpy-fft.ts:50-66): 4, 2, 3, 5, 7 first, then odd trial division."""
    factors = []
    for radix in (4, 2, 3, 5, 7):
        while n % radix == 0:
            factors.append(radix)
            n //= radix
    radix = 11
    while radix * radix <= n:
        while n % radix == 0:
            factors.append(radix)
            n //= radix
        radix += 2
    if n > 1:
        factors.append(n)
    return factors


def fft(re, im, inverse=False, factors=None):
    factors = factor_fft_size(re.shape[-1]) if factors is None else factors
    return routine_for(Routines.Fft, [re, im], [re.shape, re.shape], [NP2DT[re.dtype]] * 2, dict(factors=factors, inverse=inverse))


def scatter(updates, indices, op, shape, axis, out_dim, unique=False, dtype=None):
    in_dtypes = None
    if dtype is not None:
        in_dtypes = [dtype] + [NP2DT[np.asarray(i).dtype] for i in indices]
    out_dt = dtype or NP2DT[np.asarray(updates).dtype]
    return routine_for(Routines.Scatter, [updates] + list(indices), [shape], [out_dt],
                       dict(op=op, shape=list(shape), axis=list(axis), outDim=out_dim, uniqueIndices=unique), in_dtypes)
