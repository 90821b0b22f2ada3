"""Profiler hook state and labels (src/tracing.ts:15-107), no device needed."""
from jaxjs_hip import AluOp, DType, ShapeTracker, tracing
from jaxjs_hip.lowering import mapKernel, reduceKernel
from jaxjs_hip.routine import Routine, Routines, RoutineType


def test_trace_state_and_flush_callbacks():
    calls = []
    tracing.onFlushTrace(lambda: calls.append(1))
    assert not tracing.isTracing()
    tracing.startTrace()
    assert tracing.isTracing() and calls == []
    tracing.stopTrace()
    assert not tracing.isTracing() and calls == [1]


def test_trace_source_info_and_emit():
    st = ShapeTracker.fromShape([1500, 8])
    k = mapKernel([1500, 8], [(DType.Float32, st)], lambda x: x)
    info = tracing.traceSourceInfo(k)
    assert info.label == "Kernel[12.0K]" and info.color == "primary" and dict(info.properties)["nargs"] == "1"
    r = reduceKernel([1500, 8], [(DType.Float32, st)], lambda x: x, AluOp.Max)
    info = tracing.traceSourceInfo(r)
    assert info.label == "Kernel[1.50K]" and info.color == "secondary" and ("reduction", "Max:8") in info.properties
    rt = Routine(Routines.Sort, RoutineType([[4, 10]], [DType.Float32], [[4, 10]], [DType.Float32]))
    info = tracing.traceSourceInfo(rt)
    assert info.label == "Sort" and info.color == "tertiary" and ("inputShapes", "[4,10]") in info.properties
    assert [tracing.humanSize(n) for n in (7, 999, 1000, 123456, 33554432, 2_500_000_000)] == ["7", "999", "1.00K", "123K", "33.6M", "2.50B"]
    got = []
    tracing.setTraceSink(got.append)
    try:
        tracing.emitTrace("hip", info, 1.0, 2.5)
    finally:
        tracing.setTraceSink(None)
    assert got == [dict(name="Sort", start=1.0, end=2.5, detail=dict(devtools=dict(
        trackGroup="JAX Profiler", track="hip", color="tertiary", properties=info.properties)))]
