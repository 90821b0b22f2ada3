"""The reference's backend contract test (src/backend/backend.test.ts) restated against `HipBackend`,
plus the ownership/error rules of the Backend interface (src/backend.ts:158-240).  Runs on a real MI355X
through the C-ABI library; expected values are the ones the reference's test asserts."""
import asyncio

import numpy as np
import pytest

from jaxjs_hip import (AluExp, AluOp, AluVar, DType, Kernel, Reduction, Routine, Routines, RoutineType, ScatterOp,
                       ShapeTracker, SlotError, accessorGlobal, unravelAlu)
from gpu_util import WARM_ONLY, backend

pytestmark = pytest.mark.gpu


def f32(*v):
    return np.array(v, dtype=np.float32)


def u8(a):
    return np.ascontiguousarray(a).tobytes()


@pytest.fixture(scope="module")
def be():
    if WARM_ONLY:
        pytest.skip("warm-up run")
    return backend()


def test_simple_operations(be):  # backend.test.ts:37-85
    shape = ShapeTracker.fromShape([3])
    a = be.malloc(12, u8(f32(1, 2, 3)))
    b = be.malloc(12, u8(f32(4, 5, 6)))
    c = be.malloc(12)
    try:
        g = AluVar.gidx
        x = accessorGlobal(DType.Float32, 0, shape, [g])
        y = accessorGlobal(DType.Float32, 1, shape.flip([True]), [g])
        exe1 = asyncio.run(be.prepareKernel(Kernel(2, 3, AluExp.mul(x, y))))
        be.dispatch(exe1, [a, b], [c])
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(c)), np.float32), f32(6, 10, 12))
        exe2 = asyncio.run(be.prepareKernel(Kernel(2, 3, AluExp.add(x, y))))
        be.dispatch(exe2, [a, b], [c])
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(c)), np.float32), f32(7, 7, 7))
        x = AluExp.globalView(DType.Float32, 0, shape, [g])
        y = AluExp.globalView(DType.Float32, 1, shape.flip([True]), [g])
        exe3 = asyncio.run(be.prepareKernel(Kernel(2, 3, AluExp.mul(x, y))))
        be.dispatch(exe3, [a, b], [c])
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(c)), np.float32), f32(6, 10, 12))
    finally:
        for s in (a, b, c):
            be.decRef(s)


def test_routines_initialize_outputs(be):  # backend.test.ts:88-116
    inp = be.malloc(16, u8(f32(4, 2, 2, 3)))
    out = be.malloc(16, u8(f32(9, 9, 9, 9)))
    try:
        r = Routine(Routines.Cholesky, RoutineType([[2, 2]], [DType.Float32], [[2, 2]], [DType.Float32]))
        exe = be.prepareRoutineSync(r)
        be.dispatch(exe, [inp], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(2, 0, 1, np.sqrt(np.float32(2))))
    finally:
        be.decRef(inp)
        be.decRef(out)


def test_scatter_clears_output(be):  # backend.test.ts:118-187
    upd = be.malloc(4, u8(f32(7)))
    i1 = be.malloc(4, u8(np.array([1], np.int32)))
    i2 = be.malloc(4, u8(np.array([2], np.int32)))
    eu, ei = be.malloc(0), be.malloc(0)
    out = be.malloc(16, u8(f32(9, 9, 9, 9)))
    params = dict(op=ScatterOp.Update, shape=[4], axis=[0], outDim=0, uniqueIndices=True)
    try:
        r = Routine(Routines.Scatter, RoutineType([[1], [1]], [DType.Float32, DType.Int32], [[4]], [DType.Float32]), params)
        exe = be.prepareRoutineSync(r)
        be.dispatch(exe, [upd, i1], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(0, 7, 0, 0))
        be.dispatch(exe, [upd, i2], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(0, 0, 7, 0))
        r0 = Routine(Routines.Scatter, RoutineType([[0], [0]], [DType.Float32, DType.Int32], [[4]], [DType.Float32]), params)
        be.dispatch(be.prepareRoutineSync(r0), [eu, ei], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(0, 0, 0, 0))
        assert len(be.readSync(eu)) == 0
    finally:
        for s in (upd, i1, i2, eu, ei, out):
            be.decRef(s)


def test_array_from_index_and_sync_ops(be):  # backend.test.ts:190-218
    a = be.malloc(800)
    try:
        exe = asyncio.run(be.prepareKernel(Kernel(0, 200, AluExp.cast(DType.Float32, AluVar.gidx))))
        be.dispatch(exe, [], [a])
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(a)), np.float32), np.arange(200, dtype=np.float32))
    finally:
        be.decRef(a)
    a = be.malloc(16)
    try:
        exe = be.prepareKernelSync(Kernel(0, 4, AluExp.cast(DType.Float32, AluVar.gidx)))
        be.dispatch(exe, [], [a])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(a), np.float32), f32(0, 1, 2, 3))
    finally:
        be.decRef(a)


def test_reads_a_buffer(be):  # backend.test.ts:220-246
    arr = f32(1, 1, 2, 3, 5, 7)
    a = be.malloc(24, u8(arr))
    try:
        np.testing.assert_array_equal(np.frombuffer(be.readSync(a), np.float32), arr)
        np.testing.assert_array_equal(np.frombuffer(be.readSync(a, 12, 8), np.float32), arr[3:5])
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(a)), np.float32), arr)
        np.testing.assert_array_equal(np.frombuffer(asyncio.run(be.read(a, 12, 8)), np.float32), arr[3:5])
        assert len(be.readSync(a, 0, 0)) == 0  # the completion fence form (src/frontend/array.ts:827)
    finally:
        be.decRef(a)


def test_performs_reduction(be):  # backend.test.ts:248-286
    a = be.malloc(24, u8(f32(1, 1, 2, 3, 5, 7)))
    out = be.malloc(12)
    try:
        st = ShapeTracker.fromShape([3, 2])
        exp = AluExp.globalView(DType.Float32, 0, st, [AluVar.gidx, AluVar.ridx])
        exe = be.prepareKernelSync(Kernel(1, 3, exp, Reduction(DType.Float32, AluOp.Add, 2)))
        be.dispatch(exe, [a], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(2, 5, 12))
        re = Reduction(DType.Float32, AluOp.Add, 2, AluExp.add(AluVar.acc(DType.Float32), AluExp.f32(1)))
        exe2 = be.prepareKernelSync(Kernel(1, 3, exp, re))
        be.dispatch(exe2, [a], [out])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.float32), f32(3, 6, 13))
    finally:
        be.decRef(a)
        be.decRef(out)


def test_bitwise_operations(be):  # backend.test.ts:288-373
    shape = ShapeTracker.fromShape([4])
    g = AluVar.gidx
    a = be.malloc(16, u8(np.array([0xFF00FF00, 0x0F0F0F0F, 0xAAAAAAAA, 7], np.uint32)))
    b = be.malloc(16, u8(np.array([0x00FF00FF, 0xF0F0F0F0, 0x55555555, 3], np.uint32)))
    c = be.malloc(16)
    sa = be.malloc(16, u8(np.array([1, 1, 1, 1], np.uint32)))
    sb = be.malloc(16, u8(np.array([0, 1, 8, 16], np.uint32)))
    ra = be.malloc(16, u8(np.array([256, 65536, 0xFFFF0000, 8], np.uint32)))
    try:
        x = accessorGlobal(DType.Uint32, 0, shape, [g])
        y = accessorGlobal(DType.Uint32, 1, shape, [g])
        for mode, want in (("and", [0, 0, 0, 3]), ("or", [0xFFFFFFFF] * 3 + [7]), ("xor", [0xFFFFFFFF] * 3 + [4])):
            be.dispatch(be.prepareKernelSync(Kernel(2, 4, AluExp.bitCombine(x, y, mode))), [a, b], [c])
            np.testing.assert_array_equal(np.frombuffer(be.readSync(c), np.uint32), np.array(want, np.uint32))
        be.dispatch(be.prepareKernelSync(Kernel(2, 4, AluExp.bitShift(x, y, "shl"))), [sa, sb], [c])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(c), np.uint32), np.array([1, 2, 256, 65536], np.uint32))
        be.dispatch(be.prepareKernelSync(Kernel(2, 4, AluExp.bitShift(x, y, "shr"))), [ra, sb], [c])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(c), np.uint32),
                                      np.array([256, 32768, 0x00FFFF00, 0], np.uint32))
    finally:
        for s in (a, b, c, sa, sb, ra):
            be.decRef(s)


def _matmul(M, N, K, gid_b, swap=False):
    stA = ShapeTracker.fromShape([M, K]).reshape([M, 1, K]).expand([M, N, K])
    stB = ShapeTracker.fromShape([K, N]).permute([1, 0]).reshape([1, N, K]).expand([M, N, K])
    idx = unravelAlu([M, N], AluVar.gidx) + [AluVar.ridx]
    ga = AluExp.globalView(DType.Float32, 0, stA, idx)
    gb = AluExp.globalView(DType.Float32, gid_b, stB, idx)
    exp = AluExp.mul(gb, ga) if swap else AluExp.mul(ga, gb)
    return Kernel(gid_b + 1, M * N, exp, Reduction(DType.Float32, AluOp.Add, K))


def test_matmul_64(be):  # backend.test.ts:375-409
    n = 64
    a = be.malloc(n * n * 4, u8(np.ones(n * n, np.float32)))
    b = be.malloc(n * n * 4)
    try:
        be.dispatch(be.prepareKernelSync(_matmul(n, n, n, 0)), [a], [b])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(b), np.float32), np.full(n * n, n, np.float32))
    finally:
        be.decRef(a)
        be.decRef(b)


def test_non_square_matmul(be):  # backend.test.ts:411-464
    M, N, K = 16, 48, 24
    a = be.malloc(M * K * 4, u8(np.ones(M * K, np.float32)))
    b = be.malloc(K * N * 4, u8(np.ones(K * N, np.float32)))
    c = be.malloc(M * N * 4)
    try:
        for swap in (False, True):
            be.dispatch(be.prepareKernelSync(_matmul(M, N, K, 1, swap)), [a, b], [c])
            np.testing.assert_array_equal(np.frombuffer(be.readSync(c), np.float32), np.full(M * N, K, np.float32))
    finally:
        for s in (a, b, c):
            be.decRef(s)


def test_row_dependent_contiguous_reduction(be):  # backend.test.ts:466-507
    M, N, K = 32, 128, 5
    m, k, n = np.meshgrid(np.arange(M), np.arange(K), np.arange(N), indexing="ij")
    inp = (m * 1000 + k * 10 + n).astype(np.float32)
    a = be.malloc(inp.nbytes, u8(inp))
    out = be.malloc(M * N * 4)
    try:
        mi, ni = unravelAlu([M, N], AluVar.gidx)
        exp = AluExp.globalView(DType.Float32, 0, ShapeTracker.fromShape([M, K, N]), [mi, AluVar.ridx, ni])
        be.dispatch(be.prepareKernelSync(Kernel(1, M * N, exp, Reduction(DType.Float32, AluOp.Add, K))), [a], [out])
        got = np.frombuffer(be.readSync(out), np.float32).reshape(M, N)
        mm, nn = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
        np.testing.assert_array_equal(got, (K * (mm * 1000 + nn) + 10 * K * (K - 1) // 2).astype(np.float32))
    finally:
        be.decRef(a)
        be.decRef(out)


def test_slot_ownership_and_errors(be):  # src/backend.ts:165-179, 222-226; src/backend/cpu.ts:22-24
    assert be.type == "hip" and 0 < be.maxArgs < float("inf")
    s = be.malloc(16)
    be.incRef(s)
    be.decRef(s)
    assert len(be.readSync(s)) == 16  # still alive: refcount was 2
    be.decRef(s)
    for call in (lambda: be.decRef(s), lambda: be.incRef(s), lambda: be.readSync(s)):
        with pytest.raises(SlotError):
            call()
    with pytest.raises(SlotError):
        asyncio.run(be.read(s))
    with pytest.raises(SlotError):
        be.readSync(123456789)
    with pytest.raises(ValueError, match="initialData size"):
        be.malloc(8, b"\0" * 4)
    z = be.malloc(0)
    assert len(be.readSync(z)) == 0
    be.decRef(z)
    exe = be.prepareKernelSync(Kernel(0, 4, AluExp.cast(DType.Float32, AluVar.gidx)))
    with pytest.raises(SlotError):
        be.dispatch(exe, [], [s])
    small = be.malloc(8)
    with pytest.raises(ValueError, match="output slot"):
        be.dispatch(exe, [], [small])
    be.decRef(small)
    # prepare is idempotent and cached by kernel structure
    assert be.prepareKernelSync(Kernel(0, 4, AluExp.cast(DType.Float32, AluVar.gidx))) is exe


def test_dispatch_refuses_undersized_inputs(be):
    st = ShapeTracker.fromShape([1024])
    k = Kernel(1, 1024, AluExp.globalView(DType.Float32, 0, st, [AluVar.gidx]))
    exe = be.prepareKernelSync(k)
    a, out = be.malloc(1024), be.malloc(4096)
    try:
        with pytest.raises(ValueError, match="kernel addresses"):
            be.dispatch(exe, [a], [out])
    finally:
        be.decRef(a)
        be.decRef(out)


def test_dispatch_order_and_buffer_reuse(be):
    """Operations run in dispatch order on one stream; freed buffers may be recycled immediately."""
    n = 1 << 16
    st = ShapeTracker.fromShape([n])
    inc = be.prepareKernelSync(Kernel(1, n, AluExp.add(AluExp.globalView(DType.Int32, 0, st, [AluVar.gidx]), AluExp.i32(1))))
    cur = be.malloc(n * 4, u8(np.zeros(n, np.int32)))
    for _ in range(50):
        nxt = be.malloc(n * 4)
        be.dispatch(inc, [cur], [nxt])
        be.decRef(cur)  # released while the kernel reading it may still be queued
        cur = nxt
    np.testing.assert_array_equal(np.frombuffer(be.readSync(cur), np.int32), np.full(n, 50, np.int32))
    be.decRef(cur)


def test_large_uploads_and_reads_through_the_pinned_staging_buffers(be):
    """Reads of 1 MiB and more are pipelined through two pinned 8 MiB buffers; uploads take the source's own memory
    (no host-side copy, read-only or not): sizes around the threshold and the chunk size, odd tails, partial reads at an
    offset, the source overwritten right after the call returns, and a kernel queued between upload and read."""
    rng = np.random.default_rng(5)
    M = 1 << 20
    sizes = [M - 4, M, M + 4, 8 * M - 4, 8 * M, 8 * M + 4, 16 * M, 20 * M + 12, 40 * M + 4]
    slots, keep = [], []
    for n in sizes:
        data = bytearray(rng.integers(0, 256, n, dtype=np.uint8).tobytes())
        keep.append(bytes(data))
        slots.append(be.malloc(n, data))
        data[:] = b"\x00" * n  # the call has returned: the library no longer reads the source
    for n, slot, want in zip(sizes, slots, keep):
        assert bytes(be.readSync(slot)) == want
        for start, count in ((4, n - 8), (n // 2 + 4, min(9 * M + 4, n - n // 2 - 4)), (n - 4, 4), (8, 0)):
            assert bytes(be.readSync(slot, start, count)) == want[start:start + count]
    n = sizes[-1] // 4
    st = ShapeTracker.fromShape([n])
    inc = be.prepareKernelSync(Kernel(1, n, AluExp.add(AluExp.globalView(DType.Int32, 0, st, [AluVar.gidx]), AluExp.i32(1))))
    out = be.malloc(n * 4)
    be.dispatch(inc, [slots[-1]], [out])  # queued behind the upload's last chunk
    np.testing.assert_array_equal(np.frombuffer(be.readSync(out), np.int32), np.frombuffer(keep[-1], np.int32) + 1)
    for s_ in slots + [out]:
        be.decRef(s_)


def test_read_is_asynchronous(be):
    """`read` (src/backend.ts:182-186) queues its copy behind the pending dispatches and yields to the event loop until it
    has landed: another coroutine runs, and dispatches more work, while the read is still pending; the bytes are those
    of the dispatches queued before the read (not of the later ones)."""
    n = 1 << 26
    heavy = be.prepareKernelSync(Kernel(0, n, AluExp.sin(AluExp.cast(DType.Float32, AluVar.gidx))))
    st = ShapeTracker.fromShape([1024])
    inc = be.prepareKernelSync(Kernel(1, 1024, AluExp.add(AluExp.globalView(DType.Int32, 0, st, [AluVar.gidx]), AluExp.i32(1))))
    big = be.malloc(n * 4)
    a = be.malloc(4096, u8(np.zeros(1024, np.int32)))
    b = be.malloc(4096)
    state = dict(turns=0, done=False, dispatched_while_pending=0)

    async def other_work():
        while not state["done"]:
            state["turns"] += 1
            if state["dispatched_while_pending"] < 3:  # the host keeps issuing work while the read is in flight
                be.dispatch(inc, [b], [a])
                state["dispatched_while_pending"] += 1
            await asyncio.sleep(0)

    async def main():
        for _ in range(300):  # tens of milliseconds of device work ahead of the read
            be.dispatch(heavy, [], [big])
        be.dispatch(inc, [a], [b])  # b = 1 everywhere
        task = asyncio.ensure_future(other_work())
        raw = await be.read(b)
        state["done"] = True
        await task
        part = await be.read(b, 8, 16)
        return raw, part

    try:
        raw, part = asyncio.run(main())
        assert state["turns"] > 1 and state["dispatched_while_pending"] == 3, state
        np.testing.assert_array_equal(np.frombuffer(raw, np.int32), np.ones(1024, np.int32))
        assert len(part) == 16
        np.testing.assert_array_equal(np.frombuffer(be.readSync(a), np.int32), np.full(1024, 2, np.int32))
        assert len(asyncio.run(be.read(be_zero := be.malloc(0)))) == 0
        be.decRef(be_zero)
        with pytest.raises(ValueError, match="outside buffer"):
            asyncio.run(be.read(a, 4000, 200))
    finally:
        for s in (big, a, b):
            be.decRef(s)


def test_routine_executables_are_cached_and_released(be):
    """prepareRoutineSync returns one executable per distinct routine (no scratch or module is allocated twice), and an
    executable that the cache lets go gives its scratch and code objects back; using it afterwards raises."""
    from jaxjs_hip.routine import Routine, Routines, RoutineType
    F = DType.Float32
    mk = lambda n: Routine(Routines.Cholesky, RoutineType([[n, n]], [F], [[n, n]], [F]))  # noqa: E731
    e1, e2 = be.prepareRoutineSync(mk(256)), be.prepareRoutineSync(mk(256))
    assert e1 is e2 and e1.data.scratch, "right-looking Cholesky owns a double-precision scratch copy"
    assert be.prepareRoutineSync(mk(192)) is not e1
    a = np.random.default_rng(3).standard_normal((256, 256))
    spd = (a @ a.T + 256 * np.eye(256)).astype(np.float32)
    x, y = be.malloc(spd.nbytes, u8(spd)), be.malloc(spd.nbytes)
    try:
        be.dispatch(e1, [x], [y])
        got = np.frombuffer(be.readSync(y), np.float32).reshape(256, 256)
        np.testing.assert_allclose(np.tril(got) @ np.tril(got).T, spd, rtol=1e-4, atol=1e-3)
        limit, be.cacheLimit = be.cacheLimit, 0
        try:
            k = Kernel(0, 4, AluExp.cast(DType.Float32, AluExp.add(AluVar.gidx, AluExp.i32(77))))
            fresh = be.prepareKernelSync(k)  # over the limit: everything prepared earlier is let go, never the one handed out
        finally:
            be.cacheLimit = limit
        assert e1.data.released and not fresh.data.released and not e1.data.scratch and not e1.data.modules
        with pytest.raises(ValueError, match="released"):
            be.dispatch(e1, [x], [y])
        e3 = be.prepareRoutineSync(mk(256))  # prepared again from the on-disk code objects
        assert e3 is not e1
        be.dispatch(e3, [x], [y])
        np.testing.assert_array_equal(np.frombuffer(be.readSync(y), np.float32).reshape(256, 256), got)
    finally:
        be.decRef(x)
        be.decRef(y)


def test_prepare_kernel_compiles_concurrently(be, monkeypatch):
    """`prepareKernel` awaited for many kernels at once (src/frontend/array.ts:792-797): the compilations overlap on
    worker threads, two requests for one kernel share one compilation, and the executables compute what the
    synchronous path's do."""
    import threading
    import jaxjs_hip.backend as B
    from jaxjs_hip import runtime
    monkeypatch.setattr(runtime, "DISK_CACHE", False)
    active, peak, calls, lock = [0], [0], [0], threading.Lock()
    orig = B.compile_source

    def counting(src, nm="kernel.hip", *a, **kw):
        with lock:
            active[0] += 1
            calls[0] += 1
            peak[0] = max(peak[0], active[0])
        try:
            return orig(src, nm, *a, **kw)
        finally:
            with lock:
                active[0] -= 1
    monkeypatch.setattr(B, "compile_source", counting)
    fresh = B.HipBackend(numerics="wasm")
    n = 4096
    st = ShapeTracker.fromShape([n])
    x = AluExp.globalView(DType.Float32, 0, st, [AluVar.gidx])
    kernels = [Kernel(1, n, AluExp.add(AluExp.mul(x, AluExp.f32(float(c))), AluExp.sin(x))) for c in range(2, 8)]

    async def main():
        return await asyncio.gather(*[fresh.prepareKernel(k) for k in kernels + kernels[:2]])
    exes = asyncio.run(main())
    assert calls[0] == len(kernels) and peak[0] >= 2, (calls, peak)
    assert exes[6] is exes[0] and exes[7] is exes[1] and len({id(e) for e in exes[:6]}) == 6
    assert fresh.prepareKernelSync(kernels[3]) is exes[3] and asyncio.run(fresh.prepareKernel(kernels[3])) is exes[3]
    data = np.linspace(-3, 3, n).astype(np.float32)
    a, o = fresh.malloc(n * 4, u8(data)), fresh.malloc(n * 4)
    try:
        fresh.dispatch(exes[5], [a], [o])
        got = np.frombuffer(fresh.readSync(o), np.float32)
        np.testing.assert_allclose(got, data * 7 + np.sin(data), rtol=1e-5, atol=1e-6)
    finally:
        fresh.decRef(a)
        fresh.decRef(o)
        fresh.clearCache()


def test_profiler_hook_emits_one_measure_per_dispatch(be):
    """startTrace / stopTrace (src/tracing.ts:15-36): every dispatch between them becomes one record shaped like the
    reference's `performance.measure` entries, in dispatch order, with device times that nest inside the host's."""
    import time
    from jaxjs_hip import tracing
    n = 1 << 22
    st = ShapeTracker.fromShape([n])
    k_map = Kernel(1, n, AluExp.exp(AluExp.globalView(DType.Float32, 0, st, [AluVar.gidx])))
    k_red = Kernel(1, 1, AluExp.globalView(DType.Float32, 0, st, [AluVar.ridx]), Reduction(DType.Float32, AluOp.Add, n))
    e_map, e_red = be.prepareKernelSync(k_map), be.prepareKernelSync(k_red)
    a, b, c = be.malloc(n * 4, u8(np.zeros(n, np.float32))), be.malloc(n * 4), be.malloc(4)
    seen = []
    tracing.setTraceSink(seen.append)
    try:
        be.dispatch(e_map, [a], [b])  # not traced
        t_before = time.perf_counter() * 1e3
        tracing.startTrace()
        assert tracing.isTracing()
        be.dispatch(e_map, [a], [b])
        be.dispatch(e_red, [b], [c])
        tracing.stopTrace()
        t_after = time.perf_counter() * 1e3
        assert not tracing.isTracing() and [r["name"] for r in seen] == ["Kernel[4.19M]", "Kernel[1]"]
        dev0, dev1 = seen[0]["detail"]["devtools"], seen[1]["detail"]["devtools"]
        assert dev0["trackGroup"] == "JAX Profiler" and dev0["track"] == "hip" and dev0["color"] == "primary"
        assert dev1["color"] == "secondary" and ("reduction", f"Add:{n}") in dev1["properties"]
        assert dict(dev0["properties"])["size"] == str(n) and dict(dev0["properties"])["nargs"] == "1"
        assert t_before <= seen[0]["start"] < seen[0]["end"] <= seen[1]["start"] + 0.05 and seen[1]["end"] <= t_after + 0.5
        assert 0.001 < seen[0]["end"] - seen[0]["start"] < 5.0
        assert np.frombuffer(be.readSync(c), np.float32)[0] == n  # the traced work ran: sum of exp(0)
        be.dispatch(e_map, [a], [b])  # after stopTrace: nothing more is recorded
        assert len(seen) == 2
    finally:
        tracing.setTraceSink(None)
        for s in (a, b, c):
            be.decRef(s)
