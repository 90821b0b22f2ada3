"""Kernel builders that lower array-level operations exactly the way the reference's front-end does.

The front-end itself is out of scope; these helpers restate the few lowerings the benchmark
configurations and the parity tests need, so that the backend is handed the same Kernels it would
receive from `Array.#naryCustom`, `Array.#unary` and `Array.#reduce` (src/frontend/array.ts:413-626)
or from the jit's fused groups (src/frontend/jit.ts:572-789).
"""

from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from .alu import AluExp, AluOp, AluVar, DType, Kernel, Reduction
from .shape import ShapeTracker, prod, unravelAlu


def mapKernel(shape: Sequence[int], inputs: Sequence[tuple], fn: Callable[..., AluExp]) -> Kernel:
    """Elementwise kernel over `shape`.  `inputs` is a list of (dtype, ShapeTracker); each tracker must
    have logical shape `shape` (broadcast beforehand).  Mirrors the non-reducing arm of
    `Array.#naryCustom` (src/frontend/array.ts:546-594): indices are `unravel(gidx)`."""
    shape = list(shape)
    idx = unravelAlu(shape, AluVar.gidx)
    src = [AluExp.globalView(dt, gid, st, idx) for gid, (dt, st) in enumerate(inputs)]
    return Kernel(len(inputs), prod(shape), fn(*src))


def reduceKernel(shape: Sequence[int], inputs: Sequence[tuple], fn: Callable[..., AluExp], op: AluOp,
                 epilogue: Optional[Callable[[AluExp], AluExp]] = None) -> Kernel:
    """Reduce the last axis of `shape`.  Mirrors `Array.#reduce` / the reducing arm of `#naryCustom`
    (src/frontend/array.ts:546-626): indices are `[unravel(gidx over shape[:-1])..., ridx]`."""
    shape = list(shape)
    idx = unravelAlu(shape[:-1], AluVar.gidx) + [AluVar.ridx]
    src = [AluExp.globalView(dt, gid, st, idx) for gid, (dt, st) in enumerate(inputs)]
    exp = fn(*src)
    re = Reduction(exp.dtype, op, shape[-1])
    if epilogue is not None:
        re = Reduction(exp.dtype, op, shape[-1], epilogue(AluVar.acc(exp.dtype)))
    return Kernel(len(inputs), prod(shape[:-1]), exp, re)


def matmulKernel(M: int, N: int, K: int, dtype: DType = DType.Float32, b_transposed: bool = False,
                 batch: Sequence[int] = ()) -> Kernel:
    """`np.matmul(A[...,M,K], B[...,K,N])` as the front-end lowers it (src/library/numpy.ts:1729-1747 ->
    src/library/lax.ts:84-129 -> Dot, src/frontend/array.ts:1045-1054): both operands are broadcast to
    `[..., M, N, K]` and multiplied under an Add reduction over K.  With `b_transposed` B is stored
    `[..., N, K]` (the `dot(x, W.T)` layout of an LLM linear layer)."""
    batch = list(batch)
    nb = len(batch)
    full = batch + [M, N, K]
    stA = ShapeTracker.fromShape(batch + [M, K]).reshape(batch + [M, 1, K]).expand(full)
    if b_transposed:
        stB = ShapeTracker.fromShape(batch + [N, K]).reshape(batch + [1, N, K]).expand(full)
    else:
        perm = list(range(nb)) + [nb + 1, nb]
        stB = ShapeTracker.fromShape(batch + [K, N]).permute(perm).reshape(batch + [1, N, K]).expand(full)
    return reduceKernel(full, [(dtype, stA), (dtype, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)


def matvecKernel(M: int, K: int, dtype: DType = DType.Float32, w_transposed: bool = False) -> Kernel:
    """`np.matvec(W[M,K], x[K])` (src/library/numpy.ts:1750-1754): W against x broadcast over rows.
    With `w_transposed` W is stored `[K, M]` and read through a transposed view."""
    if w_transposed:
        stW = ShapeTracker.fromShape([K, M]).permute([1, 0])
    else:
        stW = ShapeTracker.fromShape([M, K])
    stX = ShapeTracker.fromShape([K]).reshape([1, K]).expand([M, K])
    return reduceKernel([M, K], [(dtype, stW), (dtype, stX)], lambda w, x: AluExp.mul(w, x), AluOp.Add)
