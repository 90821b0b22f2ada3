"""The N-API addon and the JavaScript HipBackend over it (jax-js_amd/napi): loads under the image's Node,
exports one function per C entry point the backend needs, and -- on a GPU -- replays generated kernel plans
with results checked against the CPU oracle."""
import base64
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from jaxjs_hip import AluExp, AluOp, AluVar, DType, Kernel, ShapeTracker
from jaxjs_hip.alu import numpyDtype
from jaxjs_hip.lowering import mapKernel, matmulKernel, matvecKernel, reduceKernel
from jaxjs_hip.plan import exportPlan, exportRoutinePlan
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NAPI = os.path.join(ROOT, "jax-js_amd", "napi")
NODE = shutil.which("node")
needs_node = pytest.mark.skipif(NODE is None or not os.path.exists(os.path.join(NAPI, "jaxhip.node")),
                                reason="node or the built addon is not available")

EXPORTS = ["init", "shutdown", "deviceInfo", "malloc", "free", "h2d", "d2h", "compile", "moduleLoad", "moduleUnload",
           "moduleFunction", "launch", "sync", "eventCreate", "eventRecord", "eventQuery", "eventElapsedMs", "eventDestroy",
           "graphBegin", "graphEnd", "graphLaunch", "graphDestroy", "abiVersion", "d2hAsync", "compilerVersion", "d2d"]


@needs_node
def test_addon_loads_and_exports_every_binding():
    out = subprocess.run([NODE, "-e", "const a=require('./jaxhip.node');console.log(JSON.stringify([Object.keys(a),a.abiVersion()]))"],
                         cwd=NAPI, capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    keys, abi = json.loads(out.stdout)
    assert sorted(keys) == sorted(EXPORTS) and abi == 2


@needs_node
def test_backend_module_loads_and_fails_loudly_without_a_device():
    """No GPU here: constructing the backend must throw (jh_init fails), never fall back to anything."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    out = subprocess.run([NODE, "-e", "const {HipBackend}=require('./hip_backend.js');try{new HipBackend(0);console.log('constructed')}catch(e){console.log('threw:'+e.message)}"],
                         cwd=NAPI, capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and out.stdout.startswith("threw:"), out.stdout + out.stderr


def test_plan_is_plain_data():
    k = reduceKernel([4, 64], [(DType.Float32, ShapeTracker.fromShape([4, 64]))], lambda v: v, AluOp.Add)
    plan = exportPlan(k)
    again = json.loads(json.dumps(plan))
    assert again == plan and plan["outputBytes"] == 16 and plan["steps"][0]["args"][-1] == ["out", 0]


def _cases():
    rng = np.random.default_rng(9)
    f32, f16 = DType.Float32, DType.Float16
    cases = []
    # src/backend.test.ts:37-85: [1,2,3] * flip([4,5,6]) and the sum of the pair
    st3 = ShapeTracker.fromShape([3])
    a, b = np.array([1, 2, 3], np.float32), np.array([4, 5, 6], np.float32)
    cases.append(("mul_flip", mapKernel([3], [(f32, st3), (f32, st3.flip([True]))], lambda x, y: AluExp.mul(x, y)), [a, b]))
    x = rng.standard_normal((300, 1000)).astype(np.float32)
    cases.append(("rowsum_plus1", reduceKernel([300, 1000], [(f32, ShapeTracker.fromShape([300, 1000]))], lambda v: v, AluOp.Add,
                                               epilogue=lambda acc: AluExp.add(acc, AluExp.f32(1))), [x]))
    xi = rng.integers(-100, 100, (64, 4097)).astype(np.int32)
    cases.append(("int_colmax", reduceKernel([4097, 64], [(DType.Int32, ShapeTracker.fromShape([64, 4097]).permute([1, 0]))],
                                             lambda v: v, AluOp.Max), [xi]))
    W = (rng.standard_normal((1024, 512)) * 0.05).astype(np.float16)
    v = rng.standard_normal(512).astype(np.float16)
    cases.append(("matvec_f16", matvecKernel(1024, 512, f16), [W, v]))
    A = rng.integers(-3, 4, (256, 128)).astype(np.float16)
    B = rng.integers(-3, 4, (128, 384)).astype(np.float16)
    cases.append(("gemm_f16_exact", matmulKernel(256, 384, 128, f16), [A, B]))
    return cases


@pytest.mark.gpu
@needs_node
def test_javascript_backend_replays_plans(tmp_path):
    cases = _cases()
    if os.environ.get("JAXHIP_WARM") == "1":
        for _, k, _ in cases:
            exportPlan(k)
        pytest.skip("warm-up run: nothing to execute")
    payload = [dict(name=n, plan=exportPlan(k), inputs=[base64.b64encode(np.ascontiguousarray(x).tobytes()).decode() for x in xs])
               for n, k, xs in cases]
    # the kernel behind the asynchronous-read check: no inputs, 2^26 floats written per launch (tens of microseconds)
    big = Kernel(0, 1 << 26, AluExp.sin(AluExp.cast(DType.Float32, AluVar.gidx)))
    payload.append(dict(name="async_read", plan=exportPlan(big), inputs=[], asyncOnly=True))
    src, dst = tmp_path / "cases.json", tmp_path / "results.json"
    src.write_text(json.dumps(payload))
    out = subprocess.run([NODE, os.path.join(NAPI, "run_plan.js"), str(src), str(dst)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    res = json.loads(dst.read_text())
    assert res["protocol"] is True and "gfx950" in res["device"]["arch"]
    # `read` is asynchronous: pending when it returns, the event loop turns while 400 launches drain, same bytes
    ar = res["asyncRead"]
    assert ar["pendingAtReturn"] and ar["loopTurnsWhilePending"] > 0 and ar["bytesEqual"] and ar["rangedEqual"], ar
    assert ar["emptyLength"] == 0 and ar["unknownSlotRejects"], ar
    classes = set()
    for (name, k, xs), r in zip(cases, res["cases"]):
        assert r["name"] == name
        got = np.frombuffer(base64.b64decode(r["output"]), dtype=numpyDtype(k.dtype))
        want = oracle.run_kernel(k, xs, oracle.MODE_WASM)
        if k.dtype in (DType.Int32,) or name in ("mul_flip", "gemm_f16_exact"):
            np.testing.assert_array_equal(got, want, err_msg=name)
        elif k.dtype == DType.Float16:
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-2, atol=1e-3, err_msg=name)
        else:
            np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=name)
    np.testing.assert_array_equal(np.frombuffer(base64.b64decode(res["cases"][0]["output"]), np.float32), [6, 10, 12])


def _routine_cases():
    import routine_util as R
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 20000)).astype(np.float32)          # sort: LDS tiles + global passes (by-value stride arguments)
    a = rng.standard_normal((2, 24, 24))
    spd = (a @ a.transpose(0, 2, 1) + 24 * np.eye(24)).astype(np.float32)
    re, im = rng.standard_normal((4, 60)).astype(np.float32), rng.standard_normal((4, 60)).astype(np.float32)
    upd, idx = rng.integers(-9, 10, (500, 3)).astype(np.float32), rng.integers(-1, 41, (500,)).astype(np.int32)
    from jaxjs_hip.routine import Routine, Routines, RoutineType
    F, I = DType.Float32, DType.Int32
    return [
        ("sort", Routine(Routines.Sort, RoutineType([[3, 20000]], [F], [[3, 20000]], [F])), [x]),
        ("argsort", Routine(Routines.Argsort, RoutineType([[3, 20000]], [F], [[3, 20000]] * 2, [F, I])), [x]),
        ("cholesky", R.cholesky(spd), [spd]),
        ("lu", R.lu(spd), [spd]),
        ("fft", R.fft(re, im), [re, im]),
        ("scatter_update", R.scatter(upd, [idx], "update", [40, 3], [0], 0), [upd, idx]),
    ]


def test_routine_plan_is_plain_data():
    name, routine, xs = _routine_cases()[0]
    plan = exportRoutinePlan(routine)
    assert json.loads(json.dumps(plan)) == plan and plan["routine"] == "Sort" and plan["outputBytes"] == [240000]
    assert any(kind == "const" for st in plan["steps"] for kind, _ in st["args"])  # the global passes take (k, j) by value


@pytest.mark.gpu
@needs_node
def test_javascript_backend_replays_routine_plans(tmp_path):
    """prepareRoutine/dispatch of the JavaScript backend: several launches per routine, several outputs, by-value
    integer arguments; outputs compared with the CPU checker (bit-exact except Fft, see the routine tests)."""
    import routine_util as R
    cases = _routine_cases()
    if os.environ.get("JAXHIP_WARM") == "1":
        for _, r, _ in cases:
            exportRoutinePlan(r)
        pytest.skip("warm-up run: nothing to execute")
    payload = [dict(name=n, plan=exportRoutinePlan(r), inputs=[base64.b64encode(np.ascontiguousarray(x).tobytes()).decode() for x in xs])
               for n, r, xs in cases]
    src, dst = tmp_path / "cases.json", tmp_path / "results.json"
    src.write_text(json.dumps(payload))
    out = subprocess.run([NODE, os.path.join(NAPI, "run_plan.js"), str(src), str(dst)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    res = json.loads(dst.read_text())
    for (name, routine, xs), r in zip(cases, res["cases"]):
        assert r["name"] == name
        want = R.run_oracle(routine, xs)
        t = routine.type
        for raw, w, dt, shape in zip(r["outputs"], want, t.outputDtypes, t.outputShapes):
            got = np.frombuffer(base64.b64decode(raw), dtype=numpyDtype(dt)).reshape(shape)
            if name == "fft":
                np.testing.assert_allclose(got, w, rtol=0, atol=1e-5 * np.abs(w).max(), err_msg=name)
            else:
                assert R.bits_equal(got, w), name
