"""A `Backend`-shaped wrapper around the CPU oracle (test infrastructure, not a product path).

It lets a whole `JitProgram` be replayed on the oracle exactly as it is replayed on the `hip` backend:
slots are host byte buffers, `dispatch` evaluates the Kernel with `oracle.run_kernel`.  Follows the
reference's CpuBackend (src/backend/cpu.ts:15-134) in behaviour: synchronous, reference-counted slots,
`SlotError`-like KeyError for unknown slots.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

from . import oracle
from . import routines as routine_oracle


class OracleBackend:
    type = "oracle"
    maxArgs = 64

    def __init__(self, mode: int = oracle.MODE_WASM):
        self.mode = mode
        self._slots: Dict[int, List] = {}  # slot -> [bytearray, refcount]
        self._next = 1

    def malloc(self, size: int, initialData: Optional[bytes] = None) -> int:
        if initialData is not None and len(initialData) != size:
            raise ValueError("initialData size does not match buffer size")
        buf = bytearray(initialData) if initialData is not None else bytearray(size)
        slot = self._next
        self._next += 1
        self._slots[slot] = [buf, 1]
        return slot

    def incRef(self, slot: int) -> None:
        self._slots[slot][1] += 1

    def decRef(self, slot: int) -> None:
        s = self._slots[slot]
        s[1] -= 1
        if s[1] == 0:
            del self._slots[slot]

    def readSync(self, slot: int, start: int = 0, count: Optional[int] = None) -> bytes:
        buf = self._slots[slot][0]
        end = len(buf) if count is None else start + count
        return bytes(buf[start:end])

    def prepareKernelSync(self, kernel):
        return kernel

    def prepareRoutineSync(self, routine):
        return routine

    def dispatch(self, exe, inputs: Sequence[int], outputs: Sequence[int]) -> None:
        if hasattr(exe, "type") and hasattr(exe, "name"):  # a Routine
            routine_oracle.runCpuRoutine(exe, [bytes(self._slots[s][0]) for s in inputs], [self._slots[s][0] for s in outputs])
            return
        kernel = exe
        out = oracle.run_kernel(kernel, [bytes(self._slots[s][0]) for s in inputs], self.mode)
        raw = np.ascontiguousarray(out).tobytes()
        dst = self._slots[outputs[0]][0]
        if len(raw) != len(dst):
            raise ValueError(f"output slot holds {len(dst)} bytes, kernel produces {len(raw)}")
        dst[:] = raw

    def live_slots(self) -> int:
        return len(self._slots)
