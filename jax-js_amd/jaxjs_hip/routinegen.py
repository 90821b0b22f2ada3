"""Native launch plans for routines (the non-fusable operations, src/routine.ts:20-102).

Sort and Argsort along the last axis run on the GPU (template `sort.hip.inc`: keyed 64-bit words, bitonic
network, LDS tiles + global passes).  Routines without a native plan return None here and take the host path
the reference's Wasm backend takes for every routine (src/backend/wasm.ts:158-165, 216-220).
"""

from __future__ import annotations

from typing import Optional

from .alu import DType, byteWidth
from .kernelgen import KernelSource, LaunchStep, _prelude, fill, template
from .routine import Routine, Routines
from .shape import prod

_SORT_KINDS = {DType.Float32: (0, "float"), DType.Float16: (1, "jh_f16"), DType.Int32: (2, "int"),
               DType.Uint32: (3, "jh_u32"), DType.Bool: (2, "int")}
SORT_TILE = 8192  # 64 KB of LDS: rows up to 8192 elements never leave the CU


def _next_pow2(n: int) -> int:
    p = 1
    while p < n:
        p <<= 1
    return p


def generateRoutine(routine: Routine, numerics: str = "wasm") -> Optional[KernelSource]:
    if routine.name in (Routines.Sort, Routines.Argsort):
        return _gen_sort(routine, numerics)
    return None


def _gen_sort(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape, dtype = list(t.inputShapes[0]), t.inputDtypes[0]
    if len(shape) == 0:
        raise ValueError(f"{routine.name.value.lower()}: cannot sort a scalar")
    if dtype not in _SORT_KINDS:
        return None  # float64 keys do not fit the 32-bit key: host path
    n = shape[-1]
    rows = prod(shape[:-1])
    argsort = routine.name == Routines.Argsort
    if n == 0 or rows == 0:
        return KernelSource([], [], [], "sort", {}, dict(n=n, rows=rows))
    if n >= (1 << 30):
        return None
    P = max(_next_pow2(n), 2)
    tile = min(P, SORT_TILE)
    kind, ctype = _SORT_KINDS[dtype]
    threads = max(1, min(tile // 2, 1024))
    src = _prelude(numerics) + fill(template("sort.hip.inc"), dict(N=n, P=P, ROWS=rows, TILE=tile, ARGSORT=1 if argsort else 0,
                                                                   KIND=kind, T=ctype, THREADS=threads))
    tiles = rows * (P // tile)
    outs = [("out", 0), ("out", 1)] if argsort else [("out", 0), ("out", 0)]
    steps = [LaunchStep("jh_sort_local", (tiles, 1, 1), (threads, 1, 1), 0, [("in", 0), ("scratch", 0)] + outs)]
    pair_blocks = max(1, min((rows * (P // 2) + 255) // 256, 1 << 20))
    k = tile * 2
    while k <= P:
        j = k // 2
        while j >= tile:
            steps.append(LaunchStep("jh_sort_global", (pair_blocks, 1, 1), (256, 1, 1), 0, [("scratch", 0), ("const", k), ("const", j)]))
            j //= 2
        steps.append(LaunchStep("jh_sort_merge", (tiles, 1, 1), (threads, 1, 1), 0, [("in", 0), ("scratch", 0)] + outs + [("const", k)]))
        k *= 2
    scratch = [rows * P * 8] if P > tile else [8]
    need = {0: rows * n * byteWidth(dtype)}
    return KernelSource([src], steps, scratch, "sort", need, dict(n=n, rows=rows, P=P, tile=tile, argsort=argsort, launches=len(steps)))
