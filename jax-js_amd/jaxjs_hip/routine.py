"""Routines: the non-fusable operations a backend is handed as a unit (reference: src/routine.ts).

`Routine{name, type, params}` mirrors src/routine.ts:20-29 and `Routines` the enum at :32-102.
This module only holds the descriptions; the launch plans that run them on the GPU are built in
`routinegen.py`.  There is no host implementation in the package: a routine/type combination without
a GPU plan raises `UnsupportedRoutineError` at prepare time.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum
from typing import List, Optional

from .alu import DType


class Routines(str, Enum):
    Sort = "Sort"
    Argsort = "Argsort"
    Scatter = "Scatter"
    TriangularSolve = "TriangularSolve"
    Cholesky = "Cholesky"
    LU = "LU"
    JacobiEigh = "JacobiEigh"
    Fft = "Fft"
    # Not in the reference's enum: fused scaled-dot-product attention (the front-end change src/library/nn.ts:478-583
    # would need in order to hand the whole QK^T -> mask -> softmax -> PV chain to a backend as one unit).
    # Inputs q [B,L,N,H], k and v [B,S,N,H]; output [B,L,N,H]; params {scale, isCausal}.
    Attention = "Attention"

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


SUPPORTED_ROUTINES = set(Routines)
