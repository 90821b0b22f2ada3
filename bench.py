#!/usr/bin/env python3
"""Benchmark of the jax-js `hip` backend on one MI355X.

Headline workload (`config.workload`): dense f16 GEMM 8192^3 (f32 accumulation, f16 result) lowered the
way `np.matmul` lowers it, one dispatch per step, operands resident in HBM.  `value` is TFLOP/s with
FLOPs = 2*M*N*K (the reference's own convention, website/src/routes/bench/matmul/+page.svelte:16).
`roofline` is priced against the dense f16 MFMA peak; `cpu_baseline` times a single-core C restatement of
the reference Wasm backend's tiled f32 matmul loop on a slice of the same problem (the Wasm backend has
no f16 and is single-threaded in Node).  `extra` carries the other configurations: f16 matvec in both
layouts and the four fused row-reduce kernels of the softmax/argmax configuration (HBM-bound, GB/s),
an f32 elementwise map, the f32 1024^3 matmul and a GEMM sweep.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "jax-js_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

USE_GRAPHS = True  # --no-graphs clears it

PEAK_HBM_GBS = 8000.0
PEAK_F16_TFLOPS = 2500.0
PEAK_F32_MATRIX_TFLOPS = 157.3
# HBM bytes per launch of the 8192^3 f16 GEMM kernel from rocprofv3 FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 (factors from a
# copy kernel of known size); the counters are collected in separate profiler runs, not in the timed run.
GEMM_8192_HBM_BYTES = 1.750e9


def timed(be, exe, ins, out, steps, warmup):
    """W untimed + K timed dispatches; wall clock around a device fence and HIP events on the stream."""
    dev = be.dev
    for _ in range(warmup):
        be.dispatch(exe, ins, [out])
    dev.sync()
    e0, e1 = dev.event(), dev.event()
    t0 = time.perf_counter()
    dev.record(e0)
    for _ in range(steps):
        be.dispatch(exe, ins, [out])
    dev.record(e1)
    dev.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = dev.elapsed_ms(e0, e1) / steps
    dev.destroy_event(e0)
    dev.destroy_event(e1)
    return wall_ms, ev_ms


def timed_rotating(be, exe, ins_sets, out, steps, warmup):
    """`timed` over several sets of input slots taken in turn, one set per dispatch: with more bytes in the sets together
    than the 256 MB memory-side cache holds, every launch reads its operands from HBM itself (a decode loop walking a
    model's weights), not from what the previous launch of the same buffers left in that cache."""
    dev = be.dev
    n = len(ins_sets)
    for i in range(warmup):
        be.dispatch(exe, ins_sets[i % n], [out])
    dev.sync()
    e0, e1 = dev.event(), dev.event()
    t0 = time.perf_counter()
    dev.record(e0)
    for i in range(steps):
        be.dispatch(exe, ins_sets[i % n], [out])
    dev.record(e1)
    dev.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = dev.elapsed_ms(e0, e1) / steps
    dev.destroy_event(e0)
    dev.destroy_event(e1)
    return wall_ms, ev_ms


def settle(be, exe, ins, out, batch=10, limit=120, tol=0.004):
    """Launch the kernel in batches until two consecutive batches take the same time (within `tol`), at most
    `limit` launches.  After the host-side set-up (input generation, upload, compilation) the first launches of a
    kernel that runs the chip at its power limit see the clock first dip and then settle: launches 4-10 measured
    10-25 % slower than the steady state.  Returns the number of launches issued."""
    dev = be.dev
    prev, done = None, 0
    while done < limit:
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        for _ in range(batch):
            be.dispatch(exe, ins, [out])
        dev.record(e1)
        dev.sync()
        ms = dev.elapsed_ms(e0, e1) / batch
        dev.destroy_event(e0)
        dev.destroy_event(e1)
        done += batch
        if prev is not None and abs(ms - prev) <= tol * prev:
            break
        prev = ms
    return done


def timed_per_step(be, exe, ins, out, steps, warmup):
    """W untimed + K timed dispatches with a HIP event between consecutive steps: wall-clock ms per step over the K
    steps (device fence on both sides) and the list of the K per-step event times."""
    dev = be.dev
    for _ in range(warmup):
        be.dispatch(exe, ins, [out])
    dev.sync()
    evs = [dev.event() for _ in range(steps + 1)]
    t0 = time.perf_counter()
    dev.record(evs[0])
    for i in range(steps):
        be.dispatch(exe, ins, [out])
        dev.record(evs[i + 1])
    dev.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per = [dev.elapsed_ms(evs[i], evs[i + 1]) for i in range(steps)]
    for e in evs:
        dev.destroy_event(e)
    return wall_ms, per


def upload(be, arr):
    a = np.ascontiguousarray(arr)
    return be.malloc(a.nbytes, a.tobytes())


def cpu_baseline_matmul(n, seconds=12.0):
    """Single-core Wasm-loop restatement on an M-row slice of the n^3 problem, f32 stand-in for f16."""
    from oracle import oracle
    from jaxjs_hip import hostrand

    L = oracle.lib()
    rows = 32
    B = hostrand.uniform(1004 + 1, (n, n), dtype=np.float32, stream=1)
    done_flops, spent = 0.0, 0.0
    sample_rows = 0
    while spent < seconds:
        A = hostrand.uniform(1004, (rows, n), dtype=np.float32)
        C = np.empty((rows, n), dtype=np.float32)
        t0 = time.perf_counter()
        rc = L.jo_wasm_matmul_f32(A.ctypes.data_as(ctypes.c_void_p), B.ctypes.data_as(ctypes.c_void_p),
                                  C.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(rows), ctypes.c_int64(n), ctypes.c_int64(n))
        dt = time.perf_counter() - t0
        assert rc == 0
        spent += dt
        done_flops += 2.0 * rows * n * n
        sample_rows += rows
        rate = done_flops / spent
        rows = int(min(512, max(32, (seconds - spent) * rate / (2.0 * n * n) // 32 * 32)))
        if seconds - spent < 0.5:
            break
    return dict(value=done_flops / spent / 1e12, unit="TFLOP/s", cores=1, kind="port",
                sample=f"{sample_rows} of {n} output rows of the same {n}^3 problem in f32 (Wasm has no f16), "
                       f"{spent:.1f} s on one host core; {os.cpu_count()} cores present")


def cpu_baseline_secondary():
    """CPU figures beside the secondary workloads (one host core, reported only): the Wasm K-SIMD matvec loop
    restated in C on the full f32 stand-in of W[11008,4096], and the Wasm-mode evaluation of the fused
    sum(exp(x-m)*sigmoid(x)) row kernel on 64 of the 8192 rows."""
    from oracle import oracle
    from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker, hostrand
    from jaxjs_hip.lowering import reduceKernel

    L = oracle.lib()
    M, K = 11008, 4096
    W = hostrand.normal(1003, (M, K), 0.02, np.float32)
    x = hostrand.normal(1003, (K,), 1.0, np.float32, stream=1)
    y = np.empty(M, np.float32)
    best = 1e9
    for _ in range(5):
        t0 = time.perf_counter()
        rc = L.jo_wasm_matvec_f32(W.ctypes.data_as(ctypes.c_void_p), x.ctypes.data_as(ctypes.c_void_p),
                                  y.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(M), ctypes.c_int64(K))
        best = min(best, time.perf_counter() - t0)
        assert rc == 0
    out = {"matvec_f32_W[11008,4096]": {"ms": round(best * 1e3, 3), "GB/s": round((M * K * 4 + K * 4 + M * 4) / best / 1e9, 2),
                                          "kind": "port", "cores": 1}}
    rows, Lc = 64, 4096
    X = hostrand.normal(1002, (rows, Lc), 1.0, np.float32)
    f = DType.Float32
    st = ShapeTracker.fromShape([rows, Lc])
    stm = ShapeTracker.fromShape([rows]).reshape([rows, 1]).expand([rows, Lc])

    def body(v, mm):
        sig = AluExp.reciprocal(AluExp.add(AluExp.exp(AluExp.sub(AluExp.f32(0), v)), AluExp.f32(1)))
        return AluExp.mul(AluExp.exp(AluExp.add(v, AluExp.sub(AluExp.f32(0), mm))), sig)
    k = reduceKernel([rows, Lc], [(f, st), (f, stm)], body, AluOp.Add)
    m = X.max(axis=1)
    t0 = time.perf_counter()
    oracle.run_kernel(k, [X, m], oracle.MODE_WASM)
    dt = time.perf_counter() - t0
    out["c2_sum_exp_sigmoid"] = {"ms_for_64_of_8192_rows": round(dt * 1e3, 2), "GB/s": round(rows * Lc * 4 / dt / 1e9, 3),
                                 "kind": "port (interpreter of the kernel, Wasm numerics)", "cores": 1}
    return out


def bench_program_gpt2(be, hostrand, timed):
    """GPT-2-small block forward (batch 8, seq 1024, d 768, 12 heads, d_ff 3072, f16) as the traced jit program:
    every Kernel timed alone on the program's own buffers, and the whole program timed back to back."""
    from jaxjs_hip import workloads as W

    batch, seq, d, heads, d_ff = 8, 1024, 768, 12, 3072
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff)
    shapes = W.gpt2BlockShapes(batch, seq, d, d_ff)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    bufs = {}
    for i, c in enumerate(prog.consts):
        k = c.kernel()
        bufs[i] = be.malloc(k.bytes)
        be.dispatch(be.prepareKernelSync(k), [], [bufs[i]])
    for j, name in enumerate(order):
        if name in ("ln1_g", "ln2_g"):
            arr = np.ones(shapes[name], np.float16)
        elif name in ("ln1_b", "ln2_b"):
            arr = np.zeros(shapes[name], np.float16)
        else:
            arr = hostrand.normal(1005, shapes[name], 0.02, np.float16, stream=j)
        bufs[len(prog.consts) + j] = upload(be, arr)
    steps = [s for s in prog.steps if s.kind == "execute"]
    exes = []
    for s in steps:
        bufs[s.output] = be.malloc(s.kernel.bytes)
        exes.append(be.prepareKernelSync(s.kernel))

    def whole():
        for s, ex in zip(steps, exes):
            be.dispatch(ex, [bufs[i] for i in s.inputs], [bufs[s.output]])

    dev = be.dev
    for _ in range(5):
        whole()
    dev.sync()
    e0, e1 = dev.event(), dev.event()
    reps = 10
    dev.record(e0)
    for _ in range(reps):
        whole()
    dev.record(e1)
    dev.sync()
    total_ms = dev.elapsed_ms(e0, e1) / reps
    dev.destroy_event(e0)
    dev.destroy_event(e1)
    # The same program captured once into a HIP graph and replayed with one launch call per forward.
    graph_ms = None
    if USE_GRAPHS:
        from jaxjs_hip.graph import GraphedProgram
        gp = GraphedProgram(be, prog, [bufs[i] for i in range(prog.nargs)])
        for _ in range(5):
            gp.launch()
        dev.sync()
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        for _ in range(reps):
            gp.launch()
        dev.record(e1)
        dev.sync()
        graph_ms = dev.elapsed_ms(e0, e1) / reps
        dev.destroy_event(e0)
        dev.destroy_event(e1)
        gp.close()
    kernels = []
    for s, ex in zip(steps, exes):
        _, est = timed(be, ex, [bufs[i] for i in s.inputs], bufs[s.output], 3, 2)
        n_steps = int(min(max(3.0 / max(est, 1e-4), 5), 2000))
        _, ms = timed(be, ex, [bufs[i] for i in s.inputs], bufs[s.output], n_steps, max(n_steps // 2, 3))
        k = s.kernel
        row = {"class": ex.data.ks.klass, "out_elems": k.size, "reduce": k.reduction.size if k.reduction is not None else 0,
               "ms": round(ms, 5)}
        if ex.data.ks.klass.startswith("gemm"):
            row["TFLOP/s"] = round(2.0 * k.size * k.reduction.size / (ms * 1e-3) / 1e12, 1)
        kernels.append(row)
    for sl in bufs.values():
        be.decRef(sl)
    flops = 1.417e11
    return {"kernels_in_program": len(steps), "ms": round(total_ms, 4), "ms_as_hip_graph": None if graph_ms is None else round(graph_ms, 4), "sum_of_kernel_ms": round(sum(r["ms"] for r in kernels), 4),
            "model_flops": flops, "TFLOP/s": round(flops / (total_ms * 1e-3) / 1e12, 1), "per_kernel": kernels}


def bench_program_gpt2_fused(be, hostrand, timed):
    """The same block traced with the backend's fused `Attention` routine in place of the reference's seven attention
    kernels (a front-end switch, not the reference's composition): whole program eager and as a HIP graph, and the
    attention launch alone (causal: FLOP counted for the visible half of the score matrix plus the diagonal blocks)."""
    from jaxjs_hip import workloads as W
    from jaxjs_hip.graph import GraphedProgram

    batch, seq, d, heads, d_ff = 8, 1024, 768, 12, 3072
    prog = W.gpt2BlockProgram(batch, seq, d, heads, d_ff, fusedAttention=True)
    shapes = W.gpt2BlockShapes(batch, seq, d, d_ff)
    order = ["x"] + list(W.GPT2_BLOCK_PARAMS)
    ins = []
    for j, name in enumerate(order):
        if name in ("ln1_g", "ln2_g"):
            arr = np.ones(shapes[name], np.float16)
        elif name in ("ln1_b", "ln2_b"):
            arr = np.zeros(shapes[name], np.float16)
        else:
            arr = hostrand.normal(1005, shapes[name], 0.02, np.float16, stream=j)
        ins.append(upload(be, arr))
    assert not prog.consts
    prepared = prog.prepare(be)
    dev = be.dev

    def measure(fn, reps=10):
        for _ in range(5):
            fn()
        dev.sync()
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        for _ in range(reps):
            fn()
        dev.record(e1)
        dev.sync()
        ms = dev.elapsed_ms(e0, e1) / reps
        dev.destroy_event(e0)
        dev.destroy_event(e1)
        return ms

    def eager():
        for o in prog.execute(be, ins, prepared):
            be.decRef(o)

    eager_ms = measure(eager)
    graph_ms = None
    if USE_GRAPHS:
        gp = GraphedProgram(be, prog, ins)
        graph_ms = measure(gp.launch)
        gp.close()
    # the attention launch alone, on operands of the block's shape
    step = next(s for s in prog.steps if s.kind == "execute" and s.routine is not None)
    # (q, k and v reach the routine as three strided windows of the QKV projection's [batch, seq, 3d] output)
    assert all(v is not None for v in step.routine.params["views"]) and len(set(step.inputs)) == 1
    qkv = upload(be, hostrand.normal(1006, (batch, seq, 3 * d), 1.0, np.float16))
    out = be.malloc(batch * seq * d * 2)
    exe = be.prepareRoutineSync(step.routine)
    attn_ms = measure(lambda: be.dispatch(exe, [qkv, qkv, qkv], [out]), reps=50)
    for sl in ins + [qkv, out]:
        be.decRef(sl)
    H = d // heads
    full = 4.0 * batch * heads * seq * seq * H
    return {"steps_in_program": sum(1 for s in prog.steps if s.kind == "execute"), "ms": round(eager_ms, 4), "ms_as_hip_graph": None if graph_ms is None else round(graph_ms, 4),
            "TFLOP/s": round(1.417e11 / (eager_ms * 1e-3) / 1e12, 1),
            "attention_alone": {"ms": round(attn_ms, 5), "TFLOP/s_full_matrix_convention": round(full / (attn_ms * 1e-3) / 1e12, 1),
                                "TFLOP/s_causal_half": round(full / 2 / (attn_ms * 1e-3) / 1e12, 1)}}


def bench_reference_matmul_matvec_cases(be, timed):
    """The cases of the reference's own matmul and matvec benches on this backend (bench/matmul-wasm.bench.ts:5-46,
    bench/matmul-webgpu.bench.ts:11, bench/matvec-wasm.bench.ts:5-53, bench/matvec-webgpu.bench.ts:11): f32 n x n against
    n x n (and against the transpose), n x n (and its transpose) against a vector, with the operand values of the Wasm
    benches.  `ms_sync` is one dispatch + fence per iteration as there (best of 5); `ms` is the kernel back to back."""
    from jaxjs_hip import DType
    from jaxjs_hip.lowering import matmulKernel, matvecKernel

    out = {}

    def one(kernel, arrays):
        exe = be.prepareKernelSync(kernel)
        ins = [upload(be, a) for a in arrays]
        o = be.malloc(kernel.bytes)
        be.dispatch(exe, ins, [o])
        be.dev.sync()
        best = float("inf")
        for _ in range(5):
            t0 = time.perf_counter()
            be.dispatch(exe, ins, [o])
            be.dev.sync()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        _, est = timed(be, exe, ins, o, 5, 3)
        n_steps = int(min(max(5.0 / max(est, 1e-4), 20), 2000))
        _, ms = timed(be, exe, ins, o, n_steps, max(n_steps // 4, 3))
        for s_ in ins + [o]:
            be.decRef(s_)
        return {"class": exe.data.ks.klass, "ms_sync": round(best, 4), "ms": round(ms, 5)}

    def matrix(n):
        return ((np.arange(n * n, dtype=np.int64) % 7) - 3).astype(np.float32).reshape(n, n)

    for n in (64, 128, 256, 512, 1024, 2048, 4096):
        a = matrix(n)
        for tag, bt in ((f"matmul {n}x{n}", False), (f"matmul {n}x{n} @ transpose", True)):
            row = one(matmulKernel(n, n, n, DType.Float32, b_transposed=bt), [a, a])
            row["TFLOP/s"] = round(2.0 * n ** 3 / (row["ms"] * 1e-3) / 1e12, 2)
            out[tag] = row
    for n in (512, 1024, 2048, 4096):
        a = matrix(n)
        x = ((np.arange(n, dtype=np.int64) % 5) - 2).astype(np.float32)
        for tag, wt in ((f"matvec {n}x{n} @ vector", False), (f"matvec {n}x{n}.T @ vector", True)):
            row = one(matvecKernel(n, n, DType.Float32, w_transposed=wt), [a, x])
            row["GB/s"] = round((n * n + 2 * n) * 4 / (row["ms"] * 1e-3) / 1e9, 1)
            out[tag] = row
    return out


def bench_reference_routine_cases(be):
    """The cases of the reference's own routine benches on this backend (bench/fft.bench.ts:6-13, sort.bench.ts:15-16,
    cholesky-webgpu.bench.ts:16): one dispatch + fence per iteration as there, best of 5; operands resident."""
    from jaxjs_hip import DType
    from jaxjs_hip.library import factorFftSize
    from jaxjs_hip.routine import Routine, Routines, RoutineType

    F = DType.Float32
    out = {}

    def best_ms(routine, arrays, out_bytes, reps=5):
        exe = be.prepareRoutineSync(routine)
        ins = [upload(be, a) for a in arrays]
        outs = [be.malloc(b) for b in out_bytes]
        be.dispatch(exe, ins, outs)
        be.dev.sync()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            be.dispatch(exe, ins, outs)
            be.dev.sync()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        for s in ins + outs:
            be.decRef(s)
        return round(best, 4)

    for name, shape, phase in (("256", (256,), 0.0), ("1024", (1024,), 0.01), ("1000", (1000,), 0.02), ("64x256", (64, 256), 0.03),
                               ("100k", (100_000,), 0.04), ("1m", (1_000_000,), 0.05)):
        i = np.arange(int(np.prod(shape)), dtype=np.float64)
        mk = lambda ph: (np.sin((i + 1) * (0.013 + ph)) + 0.25 * np.cos((i + 3) * (0.037 + ph))).astype(np.float32).reshape(shape)  # noqa: E731
        rt = Routine(Routines.Fft, RoutineType([list(shape)] * 2, [F, F], [list(shape)] * 2, [F, F]),
                     dict(factors=factorFftSize(shape[-1]), inverse=False))
        out[f"fft {name}"] = {"ms": best_ms(rt, [mk(phase), mk(phase + 0.01)], [i.size * 4] * 2)}
    rng = np.random.default_rng(0)
    x = rng.random((32768, 1024), dtype=np.float32)
    out["sort 32768x1024"] = {"ms": best_ms(Routine(Routines.Sort, RoutineType([[32768, 1024]], [F], [[32768, 1024]], [F])), [x], [x.nbytes])}
    out["argsort 32768x1024"] = {"ms": best_ms(Routine(Routines.Argsort, RoutineType([[32768, 1024]], [F], [[32768, 1024]] * 2, [F, DType.Int32])),
                                               [x], [x.nbytes] * 2)}
    for n in (128, 256, 512, 1024, 2048):
        a = rng.standard_normal((n, n)).astype(np.float32)
        spd = (a.T @ a + n * np.eye(n, dtype=np.float32)).astype(np.float32)
        out[f"cholesky {n}x{n}"] = {"ms": best_ms(Routine(Routines.Cholesky, RoutineType([[n, n]], [F], [[n, n]], [F])), [spd], [spd.nbytes])}

    # Traced programs (bench/svd.bench.ts:11-15, bench/argreduce.bench.ts:16-48): one eager execution + fence per
    # iteration, best of 3; constants and inputs resident.
    from jaxjs_hip import jit as J
    from jaxjs_hip import library as L
    from jaxjs_hip.jit import ShapedArray

    def best_prog_ms(fn, arrays, reps=3):
        prog = J.jit(fn, [ShapedArray(tuple(a.shape), F) for a in arrays])
        const_slots = []
        for c in prog.consts:
            k = c.kernel()
            slot = be.malloc(k.bytes)
            be.dispatch(be.prepareKernelSync(k), [], [slot])
            const_slots.append(slot)
        ins = const_slots + [upload(be, a) for a in arrays]
        prepared = prog.prepare(be)
        best = float("inf")
        for it in range(reps + 1):
            t0 = time.perf_counter()
            outs = prog.execute(be, ins, prepared)
            be.dev.sync()
            if it:
                best = min(best, (time.perf_counter() - t0) * 1e3)
            for o in outs:
                be.decRef(o)
        for sl in ins:
            be.decRef(sl)
        return round(best, 4)

    for name, shape in (("128x128", (128, 128)), ("1024x128", (1024, 128)), ("32768x256", (32768, 256))):
        a = rng.standard_normal(shape).astype(np.float32)
        out[f"svdvals {name}"] = {"ms": best_prog_ms(lambda x: L.svdvals(x), [a])}
        out[f"thin svd {name}"] = {"ms": best_prog_ms(lambda x: L.svd(x), [a])}
    v10k, m2d = rng.random(10000, dtype=np.float32), rng.random((100, 1000), dtype=np.float32)
    out["argmax 10k elements"] = {"ms": best_prog_ms(lambda x: L.argmax(x, 0), [v10k])}
    out["argmax along axis (100x1000)"] = {"ms": best_prog_ms(lambda x: L.argmax(x, 1), [m2d])}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the headline GEMM")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-settle", action="store_true", help="skip the clock-settling launches before the warm-up steps")
    ap.add_argument("--no-graphs", action="store_true", help="skip the HIP-graph replays of the C5 programs (for runs under a profiler "
                                                             "whose graph-launch tracing is not to be relied on)")
    ap.add_argument("--only", choices=["all", "gemm", "copy", "hbm", "matvec", "attention"], default="all",
                    help="gemm: headline kernel only; copy: a plain f32 copy kernel of known size (counter calibration); "
                         "hbm: headline + the HBM-bound secondary workloads only (matvecs, row kernels, map); "
                         "matvec: the two f16 matvec layouts under the launch plans compared in profiles/ (each as its own "
                         "named kernel, cache-resident and cold), nothing else; attention: the GPT-2 block with the fused "
                         "attention routine and that launch (`jh_attention`) alone, nothing else")
    args = ap.parse_args()
    global USE_GRAPHS
    USE_GRAPHS = not args.no_graphs
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker, getBackend, hostrand, init
    from jaxjs_hip.lowering import mapKernel, matmulKernel, matvecKernel, reduceKernel

    init("hip")
    be = getBackend("hip")
    n = args.size
    if args.only == "gemm":
        args.no_extra = True
    if args.only == "copy":
        # 8192x4096 f32 copied once per step: 134,217,728 bytes read and as many written per launch.
        rows, L = 8192, 4096
        X = hostrand.normal(1002, (rows, L), 1.0, np.float32)
        kcopy = mapKernel([rows, L], [(DType.Float32, ShapeTracker.fromShape([rows, L]))], lambda v: v)
        ex = be.prepareKernelSync(kcopy)
        src, dst = upload(be, X), be.malloc(kcopy.bytes)
        w_ms, e_ms = timed(be, ex, [src], dst, args.steps, args.warmup)
        print(json.dumps({"workload": "copy f32 [8192,4096]", "bytes_read": rows * L * 4, "bytes_written": rows * L * 4,
                          "ms": e_ms, "GBps": 2 * rows * L * 4 / (e_ms * 1e-3) / 1e9}))
        return

    if args.only == "matvec":
        # The decode matvec W[11008,4096] . x and its transposed layout, each under the default plan and under the plan
        # it replaced, so that a profiler's per-kernel rows (durations, counters) can be compared.  "cold": four copies
        # of W taken in turn (360 MB > the 256 MB memory-side cache), "warm": one W re-read by every launch.
        M, K = 11008, 4096
        W = hostrand.normal(1003, (M, K), 0.02, np.float16)
        x = hostrand.normal(1003, (K,), 1.0, np.float16, stream=1)
        mv_bytes = M * K * 2 + K * 2 + M * 2
        rows = {}
        for layout, kern, w_host in (("W", matvecKernel(M, K, DType.Float16), W),
                                     ("WT", matvecKernel(M, K, DType.Float16, w_transposed=True), np.ascontiguousarray(W.T))):
            plans = ([("batched_nt", {}), ("one_load_in_flight", dict(row_unroll=1, row_nt=0))] if layout == "W" else
                     [("wide_strips_two_launches", {}), ("line_strips_one_launch", dict(col_strip=(8, 1024, 8), col_nt=0))])
            xs = upload(be, x)
            ws = [upload(be, w_host) for _ in range(4)]
            o = be.malloc(kern.bytes)
            for plan, opts in plans:
                for temp, use in (("warm", ws[:1]), ("cold", ws)):
                    name = f"jh_mv_{layout}_{plan}_{temp}"
                    ex = be.prepareKernelSync(kern, name=name, **opts)
                    sets = [[w, xs] for w in use]
                    n_launch = max(args.steps, 1) * 20  # 400 by default; fewer under a profiler that serialises dispatches
                    _, e1 = timed_rotating(be, ex, sets, o, n_launch, n_launch)
                    _, e2 = timed_rotating(be, ex, sets, o, n_launch, 0)
                    ms = min(e1, e2)
                    rows[name] = {"class": ex.data.ks.klass, "plan": {k_: v for k_, v in ex.data.ks.info.items() if k_ != "stage2"}, "us": round(ms * 1e3, 2),
                                  "GB/s": round(mv_bytes / (ms * 1e-3) / 1e9, 1), "frac_of_peak": round(mv_bytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
            for s_ in ws + [xs, o]:
                be.decRef(s_)
        print(json.dumps({"workload": "f16 matvec [11008,4096], both layouts, plans compared", "bytes_per_launch": mv_bytes, "rows": rows}))
        return

    if args.only == "attention":
        print(json.dumps({"workload": "GPT-2-small block, batch 8 x 1024 tokens, f16, fused attention routine (causal, 12 heads of 64)",
                          **bench_program_gpt2_fused(be, hostrand, timed)}))
        return

    # ---- headline: f16 GEMM n^3 -----------------------------------------------------------------
    A = hostrand.uniform(1004, (n, n), dtype=np.float16)
    B = hostrand.uniform(1005, (n, n), dtype=np.float16, stream=1)
    kern = matmulKernel(n, n, n, DType.Float16)
    exe = be.prepareKernelSync(kern, name=f"jh_gemm_f16_{n}_headline")
    a, b = upload(be, A), upload(be, B)
    c = be.malloc(kern.bytes)
    settled = 0 if args.no_settle else settle(be, exe, [a, b], c)
    wall_ms, per_step = timed_per_step(be, exe, [a, b], c, args.steps, args.warmup)
    ev_ms = sum(per_step) / len(per_step)
    med_ms = float(np.median(per_step))
    flops = 2.0 * n * n * n
    value = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (ev_ms * 1e-3) / 1e12
    result = {
        "metric": "matmul TFLOP/s + f16 matvec HBM GB/s (% MI355X roofline) vs Wasm CPU",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"dense GEMM f16 {n}x{n}x{n}, f32 accumulate, np.matmul lowering (B stored [K,N])",
                   "kernel_class": exe.data.ks.klass, "tile": exe.data.ks.info},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_F16_TFLOPS, 4), "traffic": GEMM_8192_HBM_BYTES if n == 8192 else None,
                     # per-step HIP-event times of the K timed steps: `achieved` is from their mean
                     "kernel_ms_mean": round(ev_ms, 4), "kernel_ms_median": round(med_ms, 4),
                     "kernel_ms_min": round(min(per_step), 4), "kernel_ms_max": round(max(per_step), 4),
                     "achieved_at_median": round(flops / (med_ms * 1e-3) / 1e12, 2)},
        # launches issued before the W warm-up steps until the clock had settled (see settle()); 0 with --no-settle
        "settle_launches": settled,
    }
    for s in (a, b, c):
        be.decRef(s)
    del A, B

    extra = {}
    if not args.no_extra:
        steps, warm = max(args.steps, 20), max(args.warmup, 5)

        def run(name, kernel, bufs, work, unit, peak, cold=None):
            """One `extra` row.  `cold=(i, n)`: a second row, `name [cold]`, in which operand i exists n times and the
            copies are taken in turn, so that the launches together read more than the 256 MB memory-side cache holds and
            every one of them fetches the operand from HBM; the first row, which re-reads one buffer, is then named
            `name [cache-resident]`."""
            # the entry point carries the workload's name, so a profiler's per-kernel rows can be told apart
            ex = be.prepareKernelSync(kernel, name="jh_" + re.sub(r"[^A-Za-z0-9]+", "_", name).strip("_"))
            slots = [upload(be, x) for x in bufs]
            sets = [slots]
            if cold is not None:
                for _ in range(cold[1] - 1):
                    other = list(slots)
                    other[cold[0]] = upload(be, bufs[cold[0]])
                    sets.append(other)
            o = be.malloc(kernel.bytes)
            # The clocks idle down while the host prepares inputs: warm up for ~30 ms of device work and time
            # at least ~5 ms of it, so a 15 us kernel is not measured on a ramping clock.
            _, est = timed(be, ex, slots, o, 3, warm)
            n_warm = int(min(max(30.0 / max(est, 1e-4), warm), 20000))
            n_steps = int(min(max(5.0 / max(est, 1e-4), steps), 5000))
            for label, use in ((" [cache-resident]" if cold else "", sets[:1]), (" [cold]", sets if cold else None)):
                if use is None:
                    continue
                # Memory clocks can take longer than the warm-up to come back after a long host-side pause (input
                # generation): two timed blocks, the faster one is reported ("timing" says so).
                w_ms, e_ms = timed_rotating(be, ex, use, o, n_steps, n_warm)
                w2, e2 = timed_rotating(be, ex, use, o, n_steps, 0)
                if e2 < e_ms:
                    w_ms, e_ms = w2, e2
                rate = work / (e_ms * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
                extra[name + label] = {"class": ex.data.ks.klass, "ms": round(e_ms, 5), "wall_ms": round(w_ms, 5),
                                       "achieved": round(rate, 2), "unit": unit, "frac_of_peak": round(rate / peak, 4),
                                       "timing": f"faster of 2 blocks of {n_steps} launches"}
                if cold:
                    extra[name + label]["operands"] = ("one set of buffers re-read by every launch (served by the memory-side cache)"
                                                       if len(use) == 1 else
                                                       f"{cold[1]} copies of operand {cold[0]} taken in turn ({cold[1] * bufs[cold[0]].nbytes >> 20} MiB > 256 MiB cache)")
            for s in {x for ss in sets for x in ss} | {o}:
                be.decRef(s)

        M, K = 11008, 4096
        W = hostrand.normal(1003, (M, K), 0.02, np.float16)
        x = hostrand.normal(1003, (K,), 1.0, np.float16, stream=1)
        mv_bytes = M * K * 2 + K * 2 + M * 2
        run("matvec_f16_W[11008,4096]", matvecKernel(M, K, DType.Float16), [W, x], mv_bytes, "GB/s", PEAK_HBM_GBS, cold=(0, 4))
        run("matvec_f16_W^T[4096,11008]", matvecKernel(M, K, DType.Float16, w_transposed=True),
            [np.ascontiguousarray(W.T), x], mv_bytes, "GB/s", PEAK_HBM_GBS, cold=(0, 4))
        del W

        rows, L = 8192, 4096
        X = hostrand.normal(1002, (rows, L), 1.0, np.float32)
        st = ShapeTracker.fromShape([rows, L])
        stm = ShapeTracker.fromShape([rows]).reshape([rows, 1]).expand([rows, L])
        f = DType.Float32
        kmax = reduceKernel([rows, L], [(f, st)], lambda v: v, AluOp.Max)
        m = X.max(axis=1)

        def body(v, mm):
            xm = AluExp.add(v, AluExp.sub(AluExp.f32(0), mm))
            sig = AluExp.reciprocal(AluExp.add(AluExp.exp(AluExp.sub(AluExp.f32(0), v)), AluExp.f32(1)))
            return AluExp.mul(AluExp.exp(xm), sig)

        ksum = reduceKernel([rows, L], [(f, st), (f, stm)], body, AluOp.Add)
        star = ShapeTracker.fromShape([L]).reshape([1, L]).expand([rows, L])
        karg = reduceKernel(
            [rows, L], [(f, st), (f, stm), (DType.Int32, star)],
            lambda v, mm, rev: AluExp.mul(AluExp.cast(DType.Int32, AluExp.cmpne(v, mm).not_()), rev), AluOp.Max,
            epilogue=lambda acc: AluExp.sub(AluExp.i32(L), acc))
        rev = np.arange(L, 0, -1, dtype=np.int32)
        xb = rows * L * 4
        run("c2_rowmax_f32[8192,4096]", kmax, [X], xb + rows * 4, "GB/s", PEAK_HBM_GBS, cold=(0, 3))
        run("c2_sum_exp_sigmoid", ksum, [X, m], xb + 2 * rows * 4, "GB/s", PEAK_HBM_GBS, cold=(0, 3))
        for label in (" [cache-resident]", " [cold]"):
            extra["c2_sum_exp_sigmoid" + label]["numerics"] = be.numerics
        # the same kernel under the other two numerics modes (second and third backend objects on the same device)
        from jaxjs_hip.backend import HipBackend
        main_be = be
        for mode in ("wasm", "native"):
            be = HipBackend(numerics=mode)
            run(f"c2_sum_exp_sigmoid[numerics={mode}]", ksum, [X, m], xb + 2 * rows * 4, "GB/s", PEAK_HBM_GBS)
            be.clearCache()
        be = main_be
        run("c2_argmax", karg, [X, m, rev], xb + 2 * rows * 4 + L * 4, "GB/s", PEAK_HBM_GBS, cold=(0, 3))
        kmap = mapKernel([rows, L], [(f, st)], lambda v: AluExp.mul(AluExp.exp(v), AluExp.f32(0.5)))
        run("map_exp_f32[8192,4096]", kmap, [X], 2 * xb, "GB/s", PEAK_HBM_GBS, cold=(0, 3))
        del X
        if args.only == "hbm":
            result["extra"] = extra
            result["cpu_baseline"] = None
            print(json.dumps(result))
            return

        for (mm, nn, kk, dt, tag, peak) in [
            (1024, 1024, 1024, DType.Float32, "c1_matmul_f32_1024", PEAK_F32_MATRIX_TFLOPS),
            (2048, 2048, 2048, DType.Float16, "gemm_f16_2048", PEAK_F16_TFLOPS),
            (4096, 4096, 4096, DType.Float16, "gemm_f16_4096", PEAK_F16_TFLOPS),
            (8000, 8000, 8000, DType.Float16, "gemm_f16_8000 (edge tiles)", PEAK_F16_TFLOPS),
            (128, 14336, 4096, DType.Float16, "gemm_f16_skinny_128x14336x4096", PEAK_F16_TFLOPS),
            (4096, 4096, 4096, DType.Float32, "gemm_f32_4096", PEAK_F32_MATRIX_TFLOPS),
        ]:
            npdt = np.float16 if dt == DType.Float16 else np.float32
            Am = hostrand.uniform(1004, (mm, kk), dtype=npdt)
            Bm = hostrand.uniform(1005, (kk, nn), dtype=npdt, stream=1)
            run(tag, matmulKernel(mm, nn, kk, dt), [Am, Bm], 2.0 * mm * nn * kk, "TFLOP/s", peak)
        # A linear layer on a few tokens and matmul against a vocabulary of 50257 columns: HBM-bound on B / rows and row
        # pitches off the 16-byte grid; reported in GB/s of algorithmic bytes and TFLOP/s respectively.
        for mm in (4, 16, 64):
            Am = hostrand.uniform(1004, (mm, 4096), dtype=np.float16)
            Bm = hostrand.uniform(1005, (4096, 14336), dtype=np.float16, stream=1)
            run(f"gemm_f16_{mm}x14336x4096", matmulKernel(mm, 14336, 4096, DType.Float16), [Am, Bm],
                2.0 * (mm * 4096 + 4096 * 14336 + mm * 14336), "GB/s", PEAK_HBM_GBS)
        Am = hostrand.uniform(1004, (8192, 768), dtype=np.float16)
        Bm = hostrand.uniform(1005, (768, 50257), dtype=np.float16, stream=1)
        run("gemm_f16_8192x50257x768", matmulKernel(8192, 50257, 768, DType.Float16), [Am, Bm], 2.0 * 8192 * 50257 * 768, "TFLOP/s", PEAK_F16_TFLOPS)
        Am = hostrand.uniform(1004, (8192, 8192), dtype=np.float16)
        Bm = hostrand.uniform(1005, (8192, 8192), dtype=np.float16, stream=1)
        run("gemm_f16_8192_NT(B stored [N,K])", matmulKernel(8192, 8192, 8192, DType.Float16, b_transposed=True), [Am, Bm],
            2.0 * 8192 ** 3, "TFLOP/s", PEAK_F16_TFLOPS)
        del Am, Bm
        for (mm, nn, kk, tag) in [(2048, 2048, 2048, "gemm_f32_2048"), (8192, 8192, 8192, "gemm_f32_8192"),
                                  (128, 14336, 4096, "gemm_f32_skinny_128x14336x4096")]:
            Am = hostrand.uniform(1004, (mm, kk), dtype=np.float32)
            Bm = hostrand.uniform(1005, (kk, nn), dtype=np.float32, stream=1)
            run(tag, matmulKernel(mm, nn, kk, DType.Float32), [Am, Bm], 2.0 * mm * nn * kk, "TFLOP/s", PEAK_F32_MATRIX_TFLOPS)
        del Am, Bm

        extra["c5_gpt2_block_b8_l1024_f16"] = bench_program_gpt2(be, hostrand, timed)
        extra["c5_gpt2_block_b8_l1024_f16_fused_attention"] = bench_program_gpt2_fused(be, hostrand, timed)

        # Convolution through the view algebra: the traced reduce Kernel is recognised as an implicit GEMM (f16 stride-1
        # windows: image patch resident in LDS; f32: gather loaders).
        from jaxjs_hip import jit as J, library as Lb
        from jaxjs_hip.jit import ShapedArray
        for cdt, npdt, tag in ((DType.Float16, np.float16, "f16"), (DType.Float32, np.float32, "f32")):
            cx, cw = (32, 64, 56, 56), (64, 64, 3, 3)
            cprog = J.jit(lambda a, b: Lb.convGeneralDilated(a, b, [1, 1], "SAME"), [ShapedArray(cx, cdt), ShapedArray(cw, cdt)])
            ck = cprog.kernels[0]
            run(f"conv3x3_same_{tag}[32,64,56,56]x[64,64,3,3]", ck,
                [hostrand.normal(1007, cx, 1.0, npdt), hostrand.normal(1007, cw, 0.05, npdt, stream=1)],
                2.0 * 32 * 64 * 56 * 56 * 64 * 9, "TFLOP/s", PEAK_F16_TFLOPS if cdt == DType.Float16 else PEAK_F32_MATRIX_TFLOPS)

        # ResNet-shaped f16 layers (batch 32): 3x3 at 28x28x256 and 14x14x256, and the stride-2 3x3 that halves 56x56.
        for cx, cw, st in (((32, 256, 28, 28), (256, 256, 3, 3), 1), ((32, 256, 14, 14), (256, 256, 3, 3), 1),
                           ((32, 64, 56, 56), (128, 64, 3, 3), 2)):
            cprog = J.jit(lambda a, b: Lb.convGeneralDilated(a, b, [st, st], "SAME"), [ShapedArray(cx, DType.Float16), ShapedArray(cw, DType.Float16)])
            run(f"conv3x3_s{st}_f16[{','.join(map(str, cx))}]x[{','.join(map(str, cw))}]", cprog.kernels[0],
                [hostrand.normal(1007, cx, 1.0, np.float16), hostrand.normal(1007, cw, 0.05, np.float16, stream=1)],
                2.0 * cx[0] * cw[0] * (cx[2] // st) * (cx[3] // st) * cw[1] * 9, "TFLOP/s", PEAK_F16_TFLOPS)

        # The reference's own conv2d bench (website/src/routes/bench/conv2d/strategies.ts:13-19: fp32, one 64 x 256 x 256
        # image, 128 filters of 3 x 3, SAME padding, `lax.convGeneralDilated`), and the same layer in f16.
        for cdt, npdt, tag in ((DType.Float32, np.float32, "f32"), (DType.Float16, np.float16, "f16")):
            cx, cw = (1, 64, 256, 256), (128, 64, 3, 3)
            cprog = J.jit(lambda a, b: Lb.convGeneralDilated(a, b, [1, 1], "SAME"), [ShapedArray(cx, cdt), ShapedArray(cw, cdt)])
            run(f"reference_conv2d_bench_{tag}[1,64,256,256]x[128,64,3,3]", cprog.kernels[0],
                [hostrand.normal(1009, cx, 1.0, npdt), hostrand.normal(1009, cw, 0.05, npdt, stream=1)],
                2.0 * 128 * 64 * 256 * 256 * 9, "TFLOP/s", PEAK_F32_MATRIX_TFLOPS if cdt == DType.Float32 else PEAK_F16_TFLOPS)

        # The two cotangent convolutions of the 56x56x64 layer (what the transpose rule of Conv binds,
        # src/frontend/linearize.ts:783-837): towards the activations and towards the filter (the latter followed by a
        # small transposing map kernel, timed with it).
        from jaxjs_hip.convolution import ConvParams
        cx, cw = (32, 64, 56, 56), (64, 64, 3, 3)
        cp = ConvParams(0, [1, 1], [(1, 1), (1, 1)], [1, 1], [1, 1])
        for cdt, npdt, tag in ((DType.Float16, np.float16, "f16"), (DType.Float32, np.float32, "f32")):
            xs_, ws_, cts_ = (hostrand.normal(1008, cx, 1.0, npdt), hostrand.normal(1008, cw, 0.05, npdt, stream=1),
                              hostrand.normal(1008, (cx[0], cw[0]) + cx[2:], 1.0, npdt, stream=2))
            for what, fn, arrs in (("activations", lambda c, f: J.convTransposeLhs(c, f, list(cx), cp), [cts_, ws_]),
                                   ("filter", lambda a, c: J.convTransposeRhs(a, c, list(cw), cp), [xs_, cts_])):
                cprog = J.jit(fn, [ShapedArray(tuple(a.shape), cdt) for a in arrs])
                ins = []
                for c_ in cprog.consts:  # closed-over constants come first
                    kc = c_.kernel()
                    ins.append(be.malloc(kc.bytes))
                    be.dispatch(be.prepareKernelSync(kc), [], [ins[-1]])
                ins += [upload(be, a) for a in arrs]
                prepared = cprog.prepare(be)

                def once():
                    for o_ in cprog.execute(be, ins, prepared):
                        be.decRef(o_)

                for _ in range(5):
                    once()
                be.dev.sync()
                e0, e1 = be.dev.event(), be.dev.event()
                reps = 50
                be.dev.record(e0)
                for _ in range(reps):
                    once()
                be.dev.record(e1)
                be.dev.sync()
                ms = be.dev.elapsed_ms(e0, e1) / reps
                be.dev.destroy_event(e0)
                be.dev.destroy_event(e1)
                for sl in ins:
                    be.decRef(sl)
                flops = 2.0 * 32 * 64 * 56 * 56 * 64 * 9
                peak = PEAK_F16_TFLOPS if cdt == DType.Float16 else PEAK_F32_MATRIX_TFLOPS
                extra[f"conv3x3_cotangent_{what}_{tag}[32,64,56,56]x[64,64,3,3]"] = {
                    "class": "+".join(be.prepareKernelSync(k_).data.ks.klass for k_ in cprog.kernels), "ms": round(ms, 5),
                    "achieved": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "frac_of_peak": round(flops / (ms * 1e-3) / 1e12 / peak, 4),
                    "timing": f"{reps} executions of the traced program back to back"}

        # Routines: sort / argsort of f32 [8192, 4096] rows (native bitonic network in LDS).
        from jaxjs_hip.routine import Routine, Routines, RoutineType
        rows, L = 8192, 4096
        X = hostrand.normal(1006, (rows, L), 1.0, np.float32)
        xs = upload(be, X)
        for rname, nout in ((Routines.Sort, 1), (Routines.Argsort, 2)):
            rt = Routine(rname, RoutineType([[rows, L]], [DType.Float32], [[rows, L]] * nout, [DType.Float32, DType.Int32][:nout]))
            rexe = be.prepareRoutineSync(rt)
            outs = [be.malloc(rows * L * 4) for _ in range(nout)]
            for _ in range(5):
                be.dispatch(rexe, [xs], outs)
            be.dev.sync()
            e0, e1 = be.dev.event(), be.dev.event()
            be.dev.record(e0)
            for _ in range(10):
                be.dispatch(rexe, [xs], outs)
            be.dev.record(e1)
            be.dev.sync()
            ms = be.dev.elapsed_ms(e0, e1) / 10
            extra[f"routine_{rname.value.lower()}_f32[8192,4096]"] = {"class": "sort", "ms": round(ms, 4),
                                                                        "Gelem/s": round(rows * L / (ms * 1e-3) / 1e9, 2)}
            for o in outs:
                be.decRef(o)
        be.decRef(xs)
        del X
        extra["reference_routine_benches"] = bench_reference_routine_cases(be)
        extra["reference_matmul_matvec_benches"] = bench_reference_matmul_matvec_cases(be, timed)
        result["extra"] = extra

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_matmul(n)
        if not args.no_extra:
            result["extra"]["cpu_secondary"] = cpu_baseline_secondary()
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
