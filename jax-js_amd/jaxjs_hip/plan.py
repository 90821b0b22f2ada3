"""Serialisable launch plans: what the tuner and the code generator decide for one Kernel, as plain data.

A plan is everything a host in another language needs to run the Kernel through the C ABI -- HIP source
texts, launch steps, scratch sizes, compile options -- and nothing it would have to interpret.  The
JavaScript `HipBackend` (jax-js_amd/napi/hip_backend.js) consumes plans where the reference's TypeScript
backend would call its own port of `tuneHip` + `generate` in `prepareKernel` (src/backend.ts:192-195).
"""

from __future__ import annotations

import hashlib
from typing import Any, Dict

from .alu import Kernel
from .kernelgen import generate
from .runtime import COMPILE_OPTIONS


def exportPlan(kernel: Kernel, numerics: str = "wasm", **tune_opts) -> Dict[str, Any]:
    ks = generate(kernel, numerics, **tune_opts)
    h = hashlib.sha256()
    for src in ks.sources:
        h.update(src.encode())
    return dict(
        key=h.hexdigest(), klass=ks.klass, size=kernel.size, outputBytes=kernel.bytes,
        sources=list(ks.sources), compileOptions=list(COMPILE_OPTIONS), scratchBytes=[int(b) for b in ks.scratch_bytes],
        minInputBytes={str(g): int(b) for g, b in ks.min_input_bytes.items()},
        steps=[dict(name=s.name, module=s.module, grid=list(s.grid), block=list(s.block), shared=int(s.shared),
                    args=[[kind, int(i)] for kind, i in s.args]) for s in ks.steps],
    )
