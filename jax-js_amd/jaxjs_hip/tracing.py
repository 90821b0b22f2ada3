"""Profiler hooks: the reference's global tracing state (src/tracing.ts:1-107) and the per-dispatch timestamps the
WebGPU backend feeds into it (src/backend/webgpu/tracing.ts).

`startTrace()` / `stopTrace()` switch collection on and off; while it is on, `HipBackend.dispatch` brackets every
executable with a pair of HIP events on the stream; `stopTrace()` runs the flush callbacks, which resolve the event
pairs into start/end times on the host's clock and hand them to `emitTrace(track, info, start, end)`.  The reference
ends in `performance.measure` with devtools metadata; here the same record goes to a sink the host chooses
(`setTraceSink`), by default the list `measures`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional, Tuple

from .alu import Kernel

_enabled = False
_flush: List[Callable[[], None]] = []
measures: List[dict] = []
_sink: Optional[Callable[[dict], None]] = None


def startTrace() -> None:
    global _enabled
    _enabled = True


def stopTrace() -> None:
    global _enabled
    _enabled = False
    for cb in list(_flush):
        cb()


def isTracing() -> bool:
    return _enabled


def onFlushTrace(cb: Callable[[], None]) -> None:
    _flush.append(cb)


def setTraceSink(sink: Optional[Callable[[dict], None]]) -> None:
    """Where `emitTrace` delivers its records (None: append to `measures`)."""
    global _sink
    _sink = sink


@dataclass
class TraceInfo:
    label: str
    color: str
    properties: List[Tuple[str, str]] = field(default_factory=list)


def humanSize(n: int) -> str:
    def prec3(x: float) -> str:  # Number.prototype.toPrecision(3) for 1 <= x < 1000
        return f"{x:.2f}" if x < 10 else (f"{x:.1f}" if x < 100 else f"{x:.0f}")
    if n >= 1e9:
        return prec3(n / 1e9) + "B"
    if n >= 1e6:
        return prec3(n / 1e6) + "M"
    if n >= 1e3:
        return prec3(n / 1e3) + "K"
    return str(n)


def traceSourceInfo(source) -> TraceInfo:
    """Label, colour and properties of a Kernel or Routine (src/tracing.ts:53-87)."""
    props: List[Tuple[str, str]] = []
    if isinstance(source, Kernel):
        label = f"Kernel[{humanSize(source.size)}]"
        props += [("exp", str(source.exp)), ("size", str(source.size)), ("nargs", str(source.nargs))]
        if source.reduction is None:
            color = "primary"
        else:
            color = "secondary"
            props.append(("reduction", f"{source.reduction.op}:{source.reduction.size}"))
    else:
        color = "tertiary"
        label = str(source.name)
        t = source.type
        props.append(("inputShapes", ", ".join("[" + ",".join(map(str, s)) + "]" for s in t.inputShapes)))
        props.append(("outputShapes", ", ".join("[" + ",".join(map(str, s)) + "]" for s in t.outputShapes)))
        props.append(("dtype", ", ".join(str(d) for d in t.inputDtypes)))
    return TraceInfo(label, color, props)


def emitTrace(track: str, info: TraceInfo, start: float, end: float) -> None:
    """One trace entry, shaped like the `performance.measure` call of src/tracing.ts:90-107 (times in milliseconds
    on the host's monotonic clock)."""
    rec = dict(name=info.label, start=start, end=end,
               detail=dict(devtools=dict(trackGroup="JAX Profiler", track=track, color=info.color,
                                         properties=list(info.properties))))
    if _sink is not None:
        _sink(rec)
    else:
        measures.append(rec)
