"""Serialisable launch plans: what the tuner and the code generator decide for one Kernel, as plain data.

A plan is everything a host in another language needs to run the Kernel through the C ABI -- HIP source
texts, launch steps, scratch sizes, compile options -- and nothing it would have to interpret.  The
JavaScript `HipBackend` (jax-js_amd/napi/hip_backend.js) consumes plans where the reference's TypeScript
backend would call its own port of `tuneHip` + `generate` in `prepareKernel` (src/backend.ts:192-195).
"""

from __future__ import annotations

import hashlib
from typing import Any, Dict

from .alu import Kernel, byteWidth
from .kernelgen import KernelSource, generate
from .routine import Routine
from .routinegen import generateRoutine
from .runtime import COMPILE_OPTIONS
from .shape import prod


def _common(ks: KernelSource) -> Dict[str, Any]:
    h = hashlib.sha256()
    for src in ks.sources:
        h.update(src.encode())
    for s in ks.steps:
        h.update(repr((s.name, s.grid, s.block, s.args)).encode())
    return dict(
        key=h.hexdigest(), klass=ks.klass,
        sources=list(ks.sources), compileOptions=list(COMPILE_OPTIONS), scratchBytes=[int(b) for b in ks.scratch_bytes],
        minInputBytes={str(g): int(b) for g, b in ks.min_input_bytes.items()},
        # args: ["in", i] / ["out", i] / ["scratch", i] are device pointers, ["const", v] a 64-bit integer by value
        steps=[dict(name=s.name, module=s.module, grid=list(s.grid), block=list(s.block), shared=int(s.shared),
                    args=[[kind, int(i)] for kind, i in s.args]) for s in ks.steps],
    )


def exportPlan(kernel: Kernel, numerics: str = "wasm", **tune_opts) -> Dict[str, Any]:
    ks = generate(kernel, numerics, **tune_opts)
    return dict(_common(ks), size=kernel.size, outputBytes=kernel.bytes)


def exportRoutinePlan(routine: Routine, numerics: str = "wasm") -> Dict[str, Any]:
    """The same for a Routine (src/routine.ts:20-29): several outputs, and launch steps that may take integer
    arguments by value.  Raises `UnsupportedRoutineError` when the routine has no GPU plan."""
    ks = generateRoutine(routine, numerics)
    t = routine.type
    return dict(_common(ks), routine=routine.name.value,
                inputBytes=[ks.min_input_bytes.get(i, prod(s) * byteWidth(d)) for i, (s, d) in enumerate(zip(t.inputShapes, t.inputDtypes))],
                outputBytes=[prod(s) * byteWidth(d) for s, d in zip(t.outputShapes, t.outputDtypes)])
