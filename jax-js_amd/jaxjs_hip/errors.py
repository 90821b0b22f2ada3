"""Exceptions of the Backend interface (reference: src/backend.ts:222-240)."""

from __future__ import annotations

import json


class SlotError(Exception):
    """Raised by every Backend method handed an unknown or already freed slot (src/backend.ts:222-226)."""

    def __init__(self, slot):
        super().__init__(f"Used a buffer that is invalid or already freed: {slot}")
        self.slot = slot


class UnsupportedOpError(Exception):
    """An op/dtype combination the backend cannot compile; raised at prepare time (src/backend.ts:228-234)."""

    def __init__(self, op, dtype, device, arg=None):
        msg = f"{op or ''}<{dtype}> not supported in {device} backend"
        if arg is not None:
            msg += f" with arg {json.dumps(arg, default=str)}"
        super().__init__(msg)


class UnsupportedRoutineError(Exception):
    """A routine the backend has no implementation for (src/backend.ts:236-240)."""

    def __init__(self, name, device):
        super().__init__(f"routine '{name}' is not supported in {device} backend")


class HipRuntimeError(RuntimeError):
    """A failure reported by the native runtime (compile error, launch failure, missing library)."""
