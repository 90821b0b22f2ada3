"""A compiled jit program captured into a HIP graph.

`JitProgram.execute` (src/frontend/jit.ts:111-162) is a fixed list of kernel dispatches over buffers whose
sizes are known at compile time.  `GraphedProgram` allocates every intermediate and output once, records the
dispatches into one graph (`jh_graph_begin/end`) and replays them with a single `jh_graph_launch`: no host
work per kernel, no allocator traffic per call.  Inputs are bound at capture time: write new data into the
same input slots (or capture again) to run on other values.
"""

from __future__ import annotations

from typing import Dict, List, Sequence

from .jit import JitProgram


class GraphedProgram:
    def __init__(self, backend, prog: JitProgram, inputs: Sequence[int]):
        if len(inputs) != prog.nargs:
            raise ValueError(f"jit program takes {prog.nargs} inputs, got {len(inputs)}")
        self.backend, self.prog = backend, prog
        self._slots: Dict[int, int] = {i: s for i, s in enumerate(inputs)}
        self._owned: List[int] = []
        for s in inputs:
            backend.incRef(s)
            self._owned.append(s)
        steps = [s for s in prog.steps if s.kind == "execute"]
        # compile + load before any capture; a routine step is several launches and outputs, recorded the same way
        exes = [backend.prepareRoutineSync(s.routine) if s.routine is not None else backend.prepareKernelSync(s.kernel) for s in steps]
        # The graph launches these executables' code objects and writes their scratch buffers without going through
        # dispatch: pin them so that neither cache eviction nor clearCache() can release them under a replay.
        self._exes = []
        for exe in exes:
            backend.pin(exe)
            self._exes.append(exe)
        sizes = {s.output: s.size for s in prog.steps if s.kind == "malloc"}
        for s in steps:
            for o in (s.outputs if s.routine is not None else [s.output]):
                slot = backend.malloc(sizes[o])
                self._slots[o] = slot
                self._owned.append(slot)

        def issue():
            for s, exe in zip(steps, exes):
                outs = s.outputs if s.routine is not None else [s.output]
                backend.dispatch(exe, [self._slots[i] for i in s.inputs], [self._slots[o] for o in outs])

        issue()  # one eager pass: every code object is resident before the capture starts
        backend.dev.sync()
        self._graph = None
        trace, backend.trace = backend.trace, None  # event records are not part of the graph
        backend.capturing = True                    # nor is the profiler hook's event pair (it synchronises)
        try:
            backend.dev.graph_begin()
            try:
                issue()
            finally:
                self._graph = backend.dev.graph_end()
        finally:
            backend.trace, backend.capturing = trace, False
        self.outputs = [self._slots[o] for o in prog.outputs]
        self.kernels = len(steps)

    def launch(self) -> None:
        """Queue one replay of the whole program (asynchronous, in order with everything else)."""
        if self._graph is None:
            raise ValueError("the graphed program was closed")
        if any(exe.data.released for exe in self._exes):
            raise ValueError("an executable of this graph was released: capture the program again")
        self.backend.dev.graph_launch(self._graph)

    def close(self) -> None:
        if self._graph is not None:
            self.backend.dev.sync()
            self.backend.dev.graph_destroy(self._graph)
            self._graph = None
            for exe in self._exes:
                self.backend.unpin(exe)
            self._exes = []
            for s in self._owned:
                self.backend.decRef(s)
            self._owned = []
