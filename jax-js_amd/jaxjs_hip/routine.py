"""Routines: the non-fusable operations a backend is handed as a unit (reference: src/routine.ts).

`Routine{name, type, params}` mirrors src/routine.ts:20-29 and `Routines` the enum at :32-102.
Sort and Argsort have native GPU plans (`routinegen.py`, template `sort.hip.inc`) for 32-bit and
f16 element types.  For the other routines the `hip` backend does what the reference's Wasm
backend does for every routine (src/backend/wasm.ts:158-165, 216-220): copy the operands to the
host, run the host implementation, copy the outputs back.  Host implementations here cover Sort,
Argsort (also the checker of the native ones), Scatter, TriangularSolve and Cholesky (vectorised with numpy, same input/output contracts as
src/routine.ts:185-362); LU, JacobiEigh and Fft are not provided yet and raise
`UnsupportedRoutineError` at prepare time.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Any, List, Optional, Sequence

import numpy as np

from .alu import DType, numpyDtype


class Routines(str, Enum):
    Sort = "Sort"
    Argsort = "Argsort"
    Scatter = "Scatter"
    TriangularSolve = "TriangularSolve"
    Cholesky = "Cholesky"
    LU = "LU"
    JacobiEigh = "JacobiEigh"
    Fft = "Fft"

    def __str__(self):
        return self.value


class ScatterOp(str, Enum):
    Update = "update"
    Add = "add"


@dataclass
class RoutineType:
    inputShapes: List[List[int]]
    inputDtypes: List[DType]
    outputShapes: List[List[int]]
    outputDtypes: List[DType]


@dataclass
class Routine:
    name: Routines
    type: RoutineType
    params: Optional[dict] = None


SUPPORTED_ROUTINES = {Routines.Sort, Routines.Argsort, Routines.Scatter, Routines.TriangularSolve, Routines.Cholesky}


def _typed(bufs: Sequence, dtypes: Sequence[DType], shapes: Sequence[Sequence[int]], writable: bool):
    out = []
    for buf, dt, shape in zip(bufs, dtypes, shapes):
        a = np.frombuffer(buf, dtype=numpyDtype(dt))
        if writable and not a.flags.writeable:
            raise ValueError("routine outputs must be writable buffers")
        out.append(a.reshape(shape))
    return out


def runCpuRoutine(routine: Routine, inputs: Sequence, outputs: Sequence) -> None:
    """Run a routine on host buffers, fully initialising every output (src/routine.ts:130-160)."""
    t = routine.type
    ins = _typed(inputs, t.inputDtypes, t.inputShapes, False)
    outs = _typed(outputs, t.outputDtypes, t.outputShapes, True)
    name = routine.name
    if name == Routines.Sort:
        if ins[0].ndim == 0:
            raise ValueError("sort: cannot sort a scalar")
        outs[0][...] = np.sort(ins[0], axis=-1)  # NaNs last, like TypedArray.prototype.sort
    elif name == Routines.Argsort:
        if ins[0].ndim == 0:
            raise ValueError("argsort: cannot sort a scalar")
        order = np.argsort(ins[0], axis=-1, kind="stable")  # stable; NaNs sort to the end
        outs[1][...] = order.astype(outs[1].dtype)
        outs[0][...] = np.take_along_axis(ins[0], order, axis=-1)
    elif name == Routines.Scatter:
        _scatter(t, ins, outs[0], routine.params or {})
    elif name == Routines.TriangularSolve:
        _triangular_solve(ins[0], ins[1], outs[0], bool((routine.params or {}).get("unitDiagonal", False)))
    elif name == Routines.Cholesky:
        _cholesky(ins[0], outs[0])
    else:
        from .errors import UnsupportedRoutineError

        raise UnsupportedRoutineError(name, "hip")


def _scatter(t: RoutineType, ins: List[np.ndarray], out: np.ndarray, params: dict) -> None:
    """Zero-fill, then write/add each update at the coordinate its index arrays select; updates
    whose coordinate falls outside the output are dropped (src/routine.ts:226-296)."""
    out[...] = 0
    updates, indices = ins[0], ins[1:]
    if updates.size == 0:
        return
    op = ScatterOp(params["op"])
    out_shape, axes, out_dim = list(params["shape"]), list(params["axis"]), int(params["outDim"])
    accumulate = op != ScatterOp.Update and not params.get("uniqueIndices", False)
    ushape = list(updates.shape)
    index_rank = max(len(i.shape) for i in indices) if indices else 0
    coords = np.indices(ushape).reshape(len(ushape), -1)  # coordinate of every update element
    free_dims = [d for d in range(len(ushape)) if d < out_dim or d >= out_dim + index_rank]
    flat = np.zeros(coords.shape[1], dtype=np.int64)
    valid = np.ones(coords.shape[1], dtype=bool)
    strides = [int(np.prod(out_shape[d + 1:])) for d in range(len(out_shape))]
    free_iter = iter(free_dims)
    for axis, extent in enumerate(out_shape):
        if axis in axes:
            ia = indices[axes.index(axis)]
            first = out_dim + index_rank - ia.ndim
            sel = tuple(coords[first + j] if ia.shape[j] != 1 else np.zeros_like(coords[0]) for j in range(ia.ndim))
            c = ia[sel].astype(np.int64) if ia.ndim else np.full(coords.shape[1], int(ia), dtype=np.int64)
        else:
            c = coords[next(free_iter)].astype(np.int64)
        valid &= (c >= 0) & (c < extent)
        flat += np.where(valid, c, 0) * strides[axis]
    flat, vals = flat[valid], updates.reshape(-1)[valid]
    target = out.reshape(-1)
    if accumulate and t.inputDtypes[0] == DType.Bool:
        np.bitwise_or.at(target, flat, vals)
    elif accumulate:
        np.add.at(target, flat, vals)
    else:
        target[flat] = vals  # later updates win, as in the sequential reference loop


def _triangular_solve(a: np.ndarray, b: np.ndarray, x: np.ndarray, unit_diagonal: bool) -> None:
    """Back-substitution for upper-triangular `a @ x.T = b.T` (src/routine.ts:298-336)."""
    if a.ndim < 2 or b.ndim < 2:
        raise ValueError("triangular_solve: operands must be at least 2D")
    n = a.shape[-1]
    if a.shape[-2] != n or b.shape[-1] != n:
        raise ValueError(f"triangular_solve: incompatible shapes a={a.shape}, b={b.shape}")
    A = a.reshape(-1, n, n)
    B = b.reshape(A.shape[0], -1, n)
    X = np.zeros_like(B)
    for i in range(n - 1, -1, -1):
        s = B[:, :, i] - np.einsum("bj,btj->bt", A[:, i, i + 1:], X[:, :, i + 1:])
        X[:, :, i] = s if unit_diagonal else s / A[:, i, i][:, None]
    x[...] = X.reshape(x.shape)


def _cholesky(a: np.ndarray, out: np.ndarray) -> None:
    """Lower-triangular factor of each matrix, reading the lower triangle, zero above the diagonal
    (src/routine.ts:338-362).  Column by column so that non-PD inputs give NaNs rather than raising."""
    n = a.shape[-1]
    A = a.reshape(-1, n, n).astype(a.dtype)
    L = np.zeros_like(A)
    with np.errstate(invalid="ignore", divide="ignore"):
        for j in range(n):
            d = A[:, j, j] - np.sum(L[:, j, :j] ** 2, axis=-1)
            L[:, j, j] = np.sqrt(d)
            if j + 1 < n:
                s = A[:, j + 1:, j] - np.einsum("bik,bk->bi", L[:, j + 1:, :j], L[:, j, :j])
                L[:, j + 1:, j] = s / L[:, j, j][:, None]
    out[...] = L.reshape(out.shape)
