"""jax-js `hip` backend for AMD Instinct MI355X (gfx950).

`HipBackend` implements the reference's Backend interface (src/backend.ts:158-211) over a C-ABI
runtime; the IR classes mirror src/alu.ts and src/shape.ts.  Importing the package never touches
the GPU; constructing `HipBackend` does.
"""

from .alu import (AluExp, AluGroup, AluOp, AluVar, DType, Kernel, Reduction, accessorAluExp, accessorGlobal,
                  byteWidth, dtypedArray, isFloatDtype, numpyDtype, promoteTypes)
from .errors import HipRuntimeError, SlotError, UnsupportedOpError, UnsupportedRoutineError
from .routine import Routine, Routines, RoutineType, ScatterOp
from .shape import ShapeTracker, View, unravelAlu
from .tracing import isTracing, startTrace, stopTrace

devices = ["hip"]
_backends = {}


def init(*devicesToInit, **options):
    """Initialise backends and return the list of available ones (src/backend.ts:50-69)."""
    for d in devicesToInit or devices:
        if d != "hip":
            raise ValueError(f"Backend not found: {d}")
        if d not in _backends:
            from .backend import HipBackend

            _backends[d] = HipBackend(**options)
    return list(_backends)


def getBackend(device: str = "hip"):
    """Retrieve an initialised backend (src/backend.ts:145-152)."""
    if device not in _backends:
        raise RuntimeError(f"{device} backend not ready, call init() first")
    return _backends[device]
