"""`HipBackend`: the `hip` device behind the reference's Backend interface.

Mirrors `interface Backend` (reference: src/backend.ts:158-211) member for member -- `type`,
`maxArgs`, `malloc`, `incRef`, `decRef`, `read`, `readSync`, `prepareKernel(Sync)`,
`prepareRoutine(Sync)`, `dispatch` -- with the same ownership and error rules:

* slots are caller-refcounted handles to untyped byte buffers; `malloc` returns refcount 1, the
  buffer is released when `decRef` reaches 0, any use of an unknown or freed slot raises
  `SlotError` (src/backend.ts:170-179, 222-226);
* `malloc(size, initialData)` requires `len(initialData) == size` (src/backend/cpu.ts:22-24);
  `malloc(0)` is legal;
* `prepareKernel*` is idempotent and cached per kernel structure (the role of
  `FpHash.hash(kernel)` in src/backend/wasm.ts:125-147); unsupported op/dtype pairs raise
  `UnsupportedOpError` here, not at dispatch;
* `dispatch` never blocks; work runs in dispatch order on one HIP stream and `read` of a slot
  observes every earlier dispatch (src/backend.ts:203-210).

Device memory, compilation and launches go through the C ABI of `include/jaxhip.h`; there is no
host fallback, neither for kernels nor for routines (the reference's Wasm backend runs routines on
the host, src/backend/wasm.ts:158-165, 216-220; here every routine is a plan of GPU launches and a
routine without one raises `UnsupportedRoutineError` at prepare time).
"""

from __future__ import annotations

import asyncio
import ctypes
import time
from collections import OrderedDict
from typing import Dict, List, Optional, Sequence

from . import tracing
from .alu import Kernel, byteWidth
from .errors import HipRuntimeError, SlotError, UnsupportedRoutineError
from .kernelgen import NUMERICS, KernelSource, generate
from .routine import Routine
from .runtime import Device, check, compile_source, pack_args


class Executable:
    """A prepared Kernel or Routine (src/backend.ts:213-220)."""

    def __init__(self, source, data):
        self.source = source
        self.data = data


class _Prepared:
    """Backend-private payload of an Executable for a Kernel."""

    def __init__(self, ks: KernelSource, functions: List[int], scratch: List[int], modules: List[int]):
        self.ks = ks
        self.functions = functions  # one per launch step
        self.scratch = scratch      # device pointers owned by this executable
        self.modules = modules
        # Per launch step: (argument cells, kernelParams array, [(cell, "in"|"out", index)] to fill per dispatch).
        # Scratch pointers and integer arguments are written once; a dispatch only stores the slot pointers, so a
        # plan of hundreds of small launches is not bound by building ctypes objects.
        self.bound = []
        for step in ks.steps:
            argv, cells = pack_args([0] * len(step.args))
            patch = []
            for c, (kind, i) in enumerate(step.args):
                if kind in ("in", "out"):
                    patch.append((c, kind, i))
                else:
                    cells[c] = scratch[i] if kind == "scratch" else int(i)
            self.bound.append((cells, argv, patch))
        # jh_launch's leading arguments per step, converted once
        self.launch_head = [(ctypes.c_void_p(fn), *step.grid, *step.block, step.shared) for step, fn in zip(ks.steps, functions)]
        self.released = False
        self.pins = 0               # holders that replay this executable without going through dispatch (HIP graphs)

    def rezero(self, dev) -> None:
        """Put the scratch buffers that every launch must find zero (the ticket counters of an in-launch fold) back to
        zero.  A launch that fails part-way may leave tickets drawn; without this every later launch of the executable
        would wait for a last ticket that never comes and leave its output unwritten."""
        for i in self.ks.zeroed_scratch:
            dev.sync()
            dev.h2d(self.scratch[i], bytes(self.ks.scratch_bytes[i]))

    def release(self, dev) -> None:
        """Give back what the executable owns on the device: its scratch buffers and its loaded code objects.  Waits for
        the stream first, so launches of it that are still queued finish on live code and memory."""
        if self.released:
            return
        if self.pins:
            raise ValueError("executable is pinned by a captured graph that still replays it")
        self.released = True
        dev.sync()
        for ptr in self.scratch:
            dev.free(ptr)
        for m in self.modules:
            dev.unload_module(m)
        self.scratch, self.modules, self.functions, self.bound, self.launch_head = [], [], [], [], []


_ALIGN = 256  # allocation granularity; also keeps every slot 128-bit-load aligned


def _freeze(v):
    if isinstance(v, dict):
        return tuple(sorted((str(k), _freeze(x)) for k, x in v.items()))
    if isinstance(v, (list, tuple)):
        return tuple(_freeze(x) for x in v)
    if isinstance(v, (int, float, str, bool, type(None))):
        return (type(v).__name__, v)
    return ("repr", repr(v))


def routineKey(routine: Routine) -> tuple:
    """Structural identity of a routine: name, operand shapes and dtypes, parameters."""
    t = routine.type
    return (str(routine.name), _freeze(t.inputShapes), tuple(str(d) for d in t.inputDtypes), _freeze(t.outputShapes),
            tuple(str(d) for d in t.outputDtypes), _freeze(routine.params))


class HipBackend:
    """MI355X backend.  `numerics="wasm"` evaluates transcendentals with the reference Wasm backend's polynomials,
    operation for operation (f32 maps within 2 ulp of the parity oracle); the default `"fast"` is the same except that
    `exp` and `reciprocal` run on the hardware's exp2 / rcp instructions (within rel 1e-5 of the oracle, the bar for f32
    maps), which is what keeps fused softmax-style rows bound by HBM instead of the VALU; `"native"` uses the device
    libm."""

    type = "hip"
    maxArgs = 64  # kernel parameters are plain pointers; same bound as the Wasm backend (src/backend/wasm.ts:38)

    def __init__(self, device: int = 0, numerics: str = "fast"):
        if numerics not in NUMERICS:
            raise ValueError(f"numerics must be one of {NUMERICS}")
        self.numerics = numerics
        self.dev = Device.get(device)
        from . import tuner

        tuner.set_compute_units(self.dev.info.compute_units)
        self._slots: Dict[int, dict] = {}
        self._next_slot = 1
        self._pool: Dict[int, List[int]] = {}   # rounded size -> free device pointers
        self._pool_bytes = 0
        self._pool_limit = 8 << 30
        self._exes: "OrderedDict[tuple, Executable]" = OrderedDict()
        self.cacheLimit = 4096
        self._preparing: Dict[tuple, "asyncio.Future"] = {}  # prepares in flight, by cache key
        self._compile_pool = None
        self._staging: Dict[int, List[int]] = {}  # capacity -> free pinned host buffers for asynchronous reads
        self.trace: Optional[list] = None       # when a list: (label, start_event, stop_event) per launch step
        self._trace_base = None                 # (event, host ms) pair fixing the profiler hook's time base
        self._trace_pending: list = []          # (TraceInfo, start event, stop event) per traced dispatch
        self._trace_registered = False
        self.capturing = False                  # a HIP graph is being recorded: no events, no synchronisation

    # -- memory -----------------------------------------------------------------------------------
    @staticmethod
    def _rounded(size: int) -> int:
        return max(_ALIGN, (size + _ALIGN - 1) // _ALIGN * _ALIGN)

    def _alloc(self, size: int) -> int:
        if size == 0:
            return 0
        r = self._rounded(size)
        free = self._pool.get(r)
        if free:
            self._pool_bytes -= r
            return free.pop()
        try:
            return self.dev.malloc(r)
        except HipRuntimeError:
            self._trim_pool(0)
            return self.dev.malloc(r)

    def _release(self, ptr: int, size: int) -> None:
        if not ptr:
            return
        r = self._rounded(size)
        # Reuse is safe without a fence: every consumer of the old contents was queued on the same
        # in-order stream before any later producer.
        self._pool.setdefault(r, []).append(ptr)
        self._pool_bytes += r
        if self._pool_bytes > self._pool_limit:
            self._trim_pool(self._pool_limit // 2)

    def _trim_pool(self, target: int) -> None:
        for r in sorted(self._pool, reverse=True):
            free = self._pool[r]
            while free and self._pool_bytes > target:
                self.dev.free(free.pop())
                self._pool_bytes -= r

    def malloc(self, size: int, initialData=None) -> int:
        size = int(size)
        if size < 0:
            raise ValueError("malloc size must be non-negative")
        if initialData is not None:
            mv = memoryview(initialData).cast("B")
            if len(mv) != size:
                raise ValueError("initialData size does not match buffer size")
        ptr = self._alloc(size)
        if initialData is not None and size:
            self.dev.h2d(ptr, initialData)
        slot = self._next_slot
        self._next_slot += 1
        self._slots[slot] = {"ptr": ptr, "size": size, "ref": 1}
        return slot

    def _get(self, slot: int) -> dict:
        s = self._slots.get(slot)
        if s is None:
            raise SlotError(slot)
        return s

    def incRef(self, slot: int) -> None:
        self._get(slot)["ref"] += 1

    def decRef(self, slot: int) -> None:
        s = self._get(slot)
        s["ref"] -= 1
        if s["ref"] == 0:
            del self._slots[slot]
            self._release(s["ptr"], s["size"])

    def readSync(self, slot: int, start: Optional[int] = None, count: Optional[int] = None) -> bytearray:
        s = self._get(slot)
        start = 0 if start is None else int(start)
        count = s["size"] - start if count is None else int(count)
        if start < 0 or count < 0 or start + count > s["size"]:
            raise ValueError(f"read range [{start}, {start + count}) outside buffer of {s['size']} bytes")
        return self.dev.d2h(s["ptr"], start, count)

    async def read(self, slot: int, start: Optional[int] = None, count: Optional[int] = None) -> bytearray:
        """Asynchronous read (src/backend.ts:182-186; the staging-buffer map of src/backend/webgpu/reader.ts): the copy
        into pinned host memory is queued behind every earlier dispatch and the coroutine yields to the event loop until
        its completion event has passed, so a caller that awaits a result keeps preparing and dispatching other work
        meanwhile.  The slot may be released while the copy is in flight: a later owner of the memory can only write it
        through work queued on the same in-order stream, after the copy."""
        s = self._get(slot)
        start = 0 if start is None else int(start)
        count = s["size"] - start if count is None else int(count)
        if start < 0 or count < 0 or start + count > s["size"]:
            raise ValueError(f"read range [{start}, {start + count}) outside buffer of {s['size']} bytes")
        cap, host = self._staging_take(count)
        ev = self.dev.d2h_async(host, s["ptr"], start, count)
        try:
            while not self.dev.event_done(ev):
                await asyncio.sleep(0)
            return bytearray(ctypes.string_at(host, count)) if count else bytearray()
        finally:
            # leaving early (cancellation) must not hand the buffer on while the copy may still land in it
            self.dev.lib.jh_event_sync(ctypes.c_void_p(ev))
            self.dev.destroy_event(ev)
            self._staging_give(cap, host)

    def _staging_take(self, nbytes: int):
        """A pinned staging buffer of at least `nbytes` (power-of-two classes from 4 KiB, a few kept per class)."""
        if nbytes == 0:
            return 0, 0
        cap = max(4096, 1 << (nbytes - 1).bit_length())
        free = self._staging.get(cap)
        return cap, (free.pop() if free else self.dev.host_alloc(cap))

    def _staging_give(self, cap: int, host: int) -> None:
        if not host:
            return
        free = self._staging.setdefault(cap, [])
        if len(free) < 4 and cap <= (64 << 20):
            free.append(host)
        else:
            self.dev.host_free(host)

    def live_slots(self) -> int:
        """Slots currently allocated through this backend object (leak checks)."""
        return len(self._slots)

    def slotPointer(self, slot: int) -> int:
        """Device address of a slot (for the benchmark harness)."""
        return self._get(slot)["ptr"]

    # -- kernels ----------------------------------------------------------------------------------
    def _build(self, source, ks: KernelSource, blobs=None) -> Executable:
        if blobs is None:
            blobs = [compile_source(src, f"{ks.klass}.hip") for src in ks.sources]
        modules = [self.dev.load_module(b) for b in blobs]
        functions = [self.dev.function(modules[s.module], s.name) for s in ks.steps]
        scratch = [self.dev.malloc(self._rounded(b)) for b in ks.scratch_bytes]
        for i in ks.zeroed_scratch:
            self.dev.h2d(scratch[i], bytes(ks.scratch_bytes[i]))
        return Executable(source, _Prepared(ks, functions, scratch, modules))

    def _cached(self, key: tuple):
        exe = self._exes.get(key)
        if exe is not None:
            self._exes.move_to_end(key)
        return exe

    def _remember(self, key: tuple, exe: Executable) -> Executable:
        """Keep at most `cacheLimit` prepared executables; the least recently prepared one is released (scratch freed,
        code objects unloaded) when the limit is passed.  Dispatching a released executable raises."""
        self._exes[key] = exe
        if len(self._exes) > self.cacheLimit:
            # oldest first; an executable that a captured graph replays is passed over (the graph launches its code
            # objects and writes its scratch without coming through dispatch)
            for k in [k for k, e in self._exes.items() if not e.data.pins and e is not exe][:len(self._exes) - self.cacheLimit]:
                self._exes.pop(k).data.release(self.dev)
        return exe

    def clearCache(self) -> None:
        """Release every prepared executable (device scratch and loaded code objects) except those pinned by a captured
        graph, which stay prepared until the graph is closed."""
        for k in [k for k, e in self._exes.items() if not e.data.pins]:
            self._exes.pop(k).data.release(self.dev)

    def pin(self, exe: Executable) -> None:
        """Keep `exe` prepared until `unpin`: for holders that launch it outside `dispatch` (a captured graph)."""
        if exe.data.released:
            raise ValueError("executable was released (evicted from the backend's cache): prepare it again")
        exe.data.pins += 1

    def unpin(self, exe: Executable) -> None:
        exe.data.pins -= 1

    def prepareKernelSync(self, kernel: Kernel, **tune_opts) -> Executable:
        key = (kernel.key(), self.numerics, tuple(sorted(tune_opts.items())))
        exe = self._cached(key)
        if exe is not None:
            return exe
        return self._remember(key, self._build(kernel, generate(kernel, self.numerics, **tune_opts)))

    async def _prepare_async(self, key: tuple, source, make_plan) -> Executable:
        """Asynchronous prepare (src/backend.ts:192-203; `createComputePipelineAsync` in src/backend/webgpu.ts:705-744):
        source generation runs here, the hiprtc compilations run on worker threads (the C call releases the
        interpreter lock), so a caller that awaits many kernels at once (src/frontend/array.ts:792-797) gets them
        compiled side by side.  Idempotent: concurrent requests for one kernel share one compilation."""
        exe = self._cached(key)
        if exe is not None:
            return exe
        pending = self._preparing.get(key)
        if pending is not None:
            return await asyncio.shield(pending)
        loop = asyncio.get_running_loop()
        fut = loop.create_future()
        self._preparing[key] = fut
        try:
            ks = make_plan()
            if self._compile_pool is None:
                from concurrent.futures import ThreadPoolExecutor
                self._compile_pool = ThreadPoolExecutor(max_workers=8, thread_name_prefix="jaxhip-compile")
            blobs = await asyncio.gather(*[loop.run_in_executor(self._compile_pool, compile_source, src, f"{ks.klass}.hip")
                                           for src in ks.sources])
            exe = self._cached(key) or self._remember(key, self._build(source, ks, blobs))
            fut.set_result(exe)
            return exe
        except BaseException as e:
            fut.set_exception(e)
            fut.exception()  # mark as retrieved: waiters, if any, re-raise it themselves
            raise
        finally:
            del self._preparing[key]

    async def prepareKernel(self, kernel: Kernel, **tune_opts) -> Executable:
        key = (kernel.key(), self.numerics, tuple(sorted(tune_opts.items())))
        return await self._prepare_async(key, kernel, lambda: generate(kernel, self.numerics, **tune_opts))

    def prepareRoutineSync(self, routine: Routine) -> Executable:
        from .routine import SUPPORTED_ROUTINES
        from .routinegen import generateRoutine

        if routine.name not in SUPPORTED_ROUTINES:
            raise UnsupportedRoutineError(routine.name, "hip")
        # Cached like kernels (the role FpHash plays in src/backend/wasm.ts:125-147): one executable, one set of
        # scratch buffers and loaded code objects per distinct routine, however often a program prepares it.
        key = ("routine", routineKey(routine), self.numerics)
        exe = self._cached(key)
        if exe is not None:
            return exe
        ks = generateRoutine(routine, self.numerics)  # raises UnsupportedRoutineError when there is no GPU plan
        return self._remember(key, self._build(routine, ks))

    async def prepareRoutine(self, routine: Routine) -> Executable:
        from .routine import SUPPORTED_ROUTINES
        from .routinegen import generateRoutine

        if routine.name not in SUPPORTED_ROUTINES:
            raise UnsupportedRoutineError(routine.name, "hip")
        key = ("routine", routineKey(routine), self.numerics)
        return await self._prepare_async(key, routine, lambda: generateRoutine(routine, self.numerics))

    def _dispatch_routine(self, exe: Executable, ins, outs) -> None:
        """Launch a routine's native plan (several kernels on the one in-order stream)."""
        routine: Routine = exe.source
        prep: _Prepared = exe.data
        t = routine.type
        if prep.released:
            raise ValueError("executable was released (evicted from the backend's cache): prepare it again")
        from .alu import byteWidth
        from .shape import prod

        if len(ins) != len(t.inputShapes) or len(outs) != len(t.outputShapes):
            raise ValueError(f"{routine.name.value} takes {len(t.inputShapes)} inputs and {len(t.outputShapes)} outputs")
        for what, slots, shapes, dtypes in (("input", ins, t.inputShapes, t.inputDtypes), ("output", outs, t.outputShapes, t.outputDtypes)):
            for i, (s, shape, dt) in enumerate(zip(slots, shapes, dtypes)):
                need = prod(shape) * byteWidth(dt)
                if what == "input" and i in prep.ks.min_input_bytes:  # an operand passed as a view of a larger buffer
                    need = prep.ks.min_input_bytes[i]
                if s["size"] < need:
                    raise ValueError(f"{what} {i} holds {s['size']} bytes, the routine addresses {need}")
        jh_launch = self.dev.lib.jh_launch
        for head, (cells, argv, patch) in zip(prep.launch_head, prep.bound):
            for c, kind, i in patch:
                cells[c] = (ins if kind == "in" else outs)[i]["ptr"]
            rc = jh_launch(*head, argv)
            if rc:
                check(rc, "jh_launch")

    # -- profiler hook (src/backend/webgpu/tracing.ts: a timestamp pair around every pass) -----------
    def _trace_begin(self):
        """While tracing is on: an event ahead of the executable's launches; the first one also fixes the time base
        (a synchronised event paired with the host clock) and registers the flush."""
        if self._trace_base is None:
            self.dev.sync()
            ev = self.dev.event()
            self.dev.record(ev)
            self.dev.sync()
            self._trace_base = (ev, time.perf_counter() * 1e3)
            if not self._trace_registered:
                tracing.onFlushTrace(self._trace_flush)
                self._trace_registered = True
        e0 = self.dev.event()
        self.dev.record(e0)
        return e0

    def _trace_end(self, exe: Executable, e0) -> None:
        e1 = self.dev.event()
        self.dev.record(e1)
        self._trace_pending.append((tracing.traceSourceInfo(exe.source), e0, e1))

    def _trace_flush(self) -> None:
        """Resolve the pending event pairs into host-clock times and emit them (run by `stopTrace`)."""
        if self._trace_base is None:
            return
        base_ev, base_ms = self._trace_base
        self.dev.sync()
        for info, e0, e1 in self._trace_pending:
            t0 = base_ms + self.dev.elapsed_ms(base_ev, e0)
            t1 = base_ms + self.dev.elapsed_ms(base_ev, e1)
            tracing.emitTrace("hip", info, t0, t1)
            self.dev.destroy_event(e0)
            self.dev.destroy_event(e1)
        self.dev.destroy_event(base_ev)
        self._trace_pending, self._trace_base = [], None

    def dispatch(self, exe: Executable, inputs: Sequence[int], outputs: Sequence[int], repeat: int = 1) -> None:
        if tracing.isTracing() and not self.capturing:
            e0 = self._trace_begin()
            try:
                self._dispatch(exe, inputs, outputs, repeat)
            finally:
                self._trace_end(exe, e0)
            return
        self._dispatch(exe, inputs, outputs, repeat)

    def _dispatch(self, exe: Executable, inputs: Sequence[int], outputs: Sequence[int], repeat: int = 1) -> None:
        ins = [self._get(s) for s in inputs]
        outs = [self._get(s) for s in outputs]
        if isinstance(exe.source, Routine):
            self._dispatch_routine(exe, ins, outs)
            return

        kernel: Kernel = exe.source
        prep: _Prepared = exe.data
        if prep.released:
            raise ValueError("executable was released (evicted from the backend's cache): prepare it again")
        if len(outs) != 1:
            raise ValueError("a Kernel has exactly one output")
        if len(ins) < kernel.nargs:
            raise ValueError(f"kernel takes {kernel.nargs} inputs, got {len(ins)}")
        if outs[0]["size"] < kernel.bytes:
            raise ValueError(f"output slot holds {outs[0]['size']} bytes, kernel writes {kernel.bytes}")
        # The generated code relies on the extents the index analysis saw: refuse a launch whose
        # buffers are smaller instead of letting a wave read past an allocation.
        for gid, need in prep.ks.min_input_bytes.items():
            if ins[gid]["size"] < need:
                raise ValueError(f"input {gid} holds {ins[gid]['size']} bytes, kernel addresses {need}")
        if kernel.size == 0:
            return
        for step, fn, head, (cells, argv, patch) in zip(prep.ks.steps, prep.functions, prep.launch_head, prep.bound):
            for c, kind, i in patch:
                cells[c] = ins[i]["ptr"] if kind == "in" else outs[0]["ptr"]
            if self.trace is None and repeat == 1:
                rc = self.dev.lib.jh_launch(*head, argv)
                if rc:
                    if prep.ks.zeroed_scratch and not self.capturing:
                        prep.rezero(self.dev)
                    check(rc, "jh_launch")
            elif self.trace is not None:
                e0, e1 = self.dev.event(), self.dev.event()
                self.dev.record(e0)
                self.dev.launch(fn, step.grid, step.block, step.shared, argv, repeat)
                self.dev.record(e1)
                self.trace.append((f"{prep.ks.klass}:{step.name}", e0, e1))
            else:
                self.dev.launch(fn, step.grid, step.block, step.shared, argv, repeat)

    def dispatchStaticScratch(self, exe: Executable, inputs: Sequence[int], outputs: Sequence[int]) -> None:
        """`dispatch` of a Kernel through `jh_launch_static_scratch`: launch steps that take a scratch buffer get the
        library's static one instead of the buffer allocated with the executable, so nothing is allocated on the way.
        For callers that must not allocate; results are bit-identical to `dispatch` (same kernels, same fold order)."""
        ins = [self._get(s) for s in inputs]
        outs = [self._get(s) for s in outputs]
        kernel, prep = exe.source, exe.data
        if isinstance(kernel, Routine) or prep.released or len(outs) != 1:
            raise ValueError("dispatchStaticScratch takes a live prepared Kernel and one output")
        if len(ins) < kernel.nargs or outs[0]["size"] < kernel.bytes:
            raise ValueError("inputs or output do not fit the kernel")
        for gid, need in prep.ks.min_input_bytes.items():
            if ins[gid]["size"] < need:
                raise ValueError(f"input {gid} holds {ins[gid]['size']} bytes, kernel addresses {need}")
        if len(prep.ks.scratch_bytes) > 1:
            raise ValueError("a kernel with several scratch buffers cannot share the one static buffer")
        if kernel.size == 0:
            return
        lib = self.dev.lib
        for step, head, (cells, argv, patch) in zip(prep.ks.steps, prep.launch_head, prep.bound):
            for c, kind, i in patch:
                cells[c] = ins[i]["ptr"] if kind == "in" else outs[0]["ptr"]
            where = [c for c, (kind, _) in enumerate(step.args) if kind == "scratch"]
            if where:
                rc = lib.jh_launch_static_scratch(*head, argv, where[0], prep.ks.scratch_bytes[0])
                cells[where[0]] = prep.scratch[0]  # the cell was overwritten: restore it for ordinary dispatches
            else:
                rc = lib.jh_launch(*head, argv)
            if rc:
                check(rc, "jh_launch_static_scratch")

    def sync(self) -> None:
        """Completion fence (what `read(slot, 0, 0)` stands for in src/frontend/array.ts:827)."""
        self.dev.sync()
