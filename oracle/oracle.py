"""ctypes front for `libalu_oracle.so`: evaluate a Kernel on the CPU the way the reference does.

TEST INFRASTRUCTURE ONLY: imported by tests/, `__graft_entry__.smoke()` and the CPU-baseline leg
of bench.py -- never by the package.  `run_kernel` serialises the expression *as the caller
built it* (`Kernel.exp_raw`, `Reduction.epilogue_raw`, GlobalView nodes untouched), so neither
the host-side simplifier nor the view lowering the product uses is on the checking path.  One fold
is applied while serialising, because the reference applies it before any of its backends runs: a
subexpression of constants becomes one constant, evaluated in JavaScript doubles and left unrounded.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, List, Optional, Sequence

import numpy as np

from jaxjs_hip.alu import AluExp, AluOp, DType, Kernel, byteWidth, numpyDtype

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libalu_oracle.so")

MODE_CPU = 0   # interpreter backend: doubles, libm, one rounding on store
MODE_WASM = 1  # Wasm backend: f32 arithmetic, the reference's own polynomials

_DT = {DType.Float32: 0, DType.Int32: 1, DType.Uint32: 2, DType.Bool: 3, DType.Float16: 4, DType.Float64: 5}
_OPS = [
    AluOp.Add, AluOp.Sub, AluOp.Mul, AluOp.Idiv, AluOp.Mod, AluOp.Min, AluOp.Max,
    AluOp.Sin, AluOp.Cos, AluOp.Asin, AluOp.Atan, AluOp.Exp, AluOp.Log, AluOp.Erf, AluOp.Erfc,
    AluOp.Sqrt, AluOp.Floor, AluOp.Ceil, AluOp.Reciprocal, AluOp.Cast, AluOp.Bitcast,
    AluOp.BitCombine, AluOp.BitInvert, AluOp.BitShift,
    AluOp.Cmplt, AluOp.Cmpne, AluOp.Where, AluOp.Threefry2x32,
    AluOp.Const, AluOp.Special, AluOp.Variable, AluOp.GlobalIndex, AluOp.GlobalView,
]
_OP = {op: i for i, op in enumerate(_OPS)}
_VARS = {"gidx": 0, "ridx": 1, "acc": 2}


def build(force: bool = False) -> str:
    """Compile the checker library with the Makefile next to this file."""
    srcs = [os.path.join(_HERE, f) for f in ("alu_oracle.c", "wasm_port.c", "Makefile")]
    stale = (not os.path.exists(_LIB_PATH)) or any(os.path.getmtime(s) > os.path.getmtime(_LIB_PATH) for s in srcs)
    if force or stale:
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libalu_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("exp", "log", "sin", "cos", "atan", "asin", "erf", "erfc"):
            f = getattr(_lib, f"jo_wasm_{name}")
            f.restype, f.argtypes = ctypes.c_float, [ctypes.c_float]
        for name in ("jo_js_erf", "jo_js_erfc"):
            f = getattr(_lib, name)
            f.restype, f.argtypes = ctypes.c_double, [ctypes.c_double]
        _lib.jo_double_to_half.restype, _lib.jo_double_to_half.argtypes = ctypes.c_uint16, [ctypes.c_double]
        _lib.jo_half_to_double.restype, _lib.jo_half_to_double.argtypes = ctypes.c_double, [ctypes.c_uint16]
        _lib.jo_run_kernel.restype = ctypes.c_int
    return _lib


_LEAVES = (AluOp.Const, AluOp.Special, AluOp.Variable, AluOp.GlobalIndex, AluOp.GlobalView)
_FLOATS = (DType.Float32, DType.Float16, DType.Float64)


def _fold_constant(e: AluExp) -> Optional[AluExp]:
    """`e` with all-constant operands as one constant holding the unrounded JavaScript number (None: leave `e`)."""
    if e.op in _LEAVES or not e.src or any(x.op != AluOp.Const for x in e.src):
        return None
    probe = AluExp.cast(DType.Float64, e) if e.dtype in _FLOATS else e
    (value,) = run_kernel(Kernel(0, 1, probe), [], MODE_CPU, fold_constants=False)
    if e.dtype in _FLOATS:
        return AluExp.const(e.dtype, float(value))
    return AluExp.const(e.dtype, bool(value) if e.dtype == DType.Bool else int(value))


class _Program:
    """Topologically ordered flat encoding of an expression DAG."""

    def __init__(self, exp: Optional[AluExp], views: List[int], fold_constants: bool = True):
        self.op: List[int] = []
        self.dt: List[int] = []
        self.soff: List[int] = [0]
        self.src: List[int] = []
        self.ia: List[int] = []
        self.fa: List[float] = []
        if exp is None:
            return
        index: Dict[int, int] = {}

        def emit(node: AluExp, srcs: list) -> int:
            i = len(self.op)
            index[id(node)] = i
            self.op.append(_OP[node.op])
            self.dt.append(_DT[node.dtype])
            self.src.extend(srcs)
            self.soff.append(len(self.src))
            a0 = a1 = 0
            f = 0.0
            op = node.op
            if op == AluOp.Const:
                if node.dtype in (DType.Float32, DType.Float16, DType.Float64):
                    f = float(node.arg)
                else:
                    a0 = int(node.arg)
            elif op == AluOp.BitCombine:
                a0 = {"and": 0, "or": 1, "xor": 2}[node.arg]
            elif op == AluOp.BitShift:
                a0 = {"shl": 0, "shr": 1}[node.arg]
            elif op == AluOp.Threefry2x32:
                a0 = 2 if node.arg == "xor" else int(node.arg)
            elif op == AluOp.Special:
                a0 = _VARS[node.arg[0]]
            elif op == AluOp.Variable:
                a0 = _VARS[node.arg]
            elif op == AluOp.GlobalIndex:
                a0 = node.arg[0]
            elif op == AluOp.GlobalView:
                a0 = node.arg[0]
                a1 = len(views)
                st = node.arg[1]
                views.append(len(st.views))
                for v in st.views:
                    views.extend([v.ndim, v.offset, 1 if v.mask is not None else 0])
                    views.extend(v.shape)
                    views.extend(v.strides)
                    if v.mask is not None:
                        for lo, hi in v.mask:
                            views.extend([lo, hi])
            elif op == AluOp.BitInvert:
                raise NotImplementedError("BitInvert has no evaluation rule in the reference")
            self.ia.extend([a0, a1])
            self.fa.append(f)
            return i

        # The reference folds constant subexpressions before any backend sees the kernel: a node whose operands are all
        # constants becomes `const(dtype, evaluate())` (src/alu.ts:670-675), evaluated in JavaScript doubles with the
        # CPU backend's arithmetic and *not* rounded to the node's type (`evaluate` hands a Const's number on as it is,
        # :1128-1137) -- so `x_f64 + 3.141592653589793` adds the double although the literal was typed float32, and
        # `cos(1.0) * x` multiplies by the rounded double cosine, not by the Wasm polynomial's value.  The same fold,
        # bottom-up, with the checker's own CPU-mode evaluator:
        if fold_constants:
            exp = exp.rewrite(_fold_constant)
        exp.fold(emit)
        # `fold` visits the root last, so the result is the last node.
        assert index[id(exp)] == len(self.op) - 1

    def arrays(self):
        return (
            np.asarray(self.op, dtype=np.int32),
            np.asarray(self.dt, dtype=np.int32),
            np.asarray(self.soff, dtype=np.int32),
            np.asarray(self.src if self.src else [0], dtype=np.int32),
            np.asarray(self.ia if self.ia else [0, 0], dtype=np.int64),
            np.asarray(self.fa if self.fa else [0.0], dtype=np.float64),
        )


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def run_kernel(kernel: Kernel, inputs: Sequence, mode: int = MODE_WASM, gidx: Optional[Sequence[int]] = None,
               return_oob: bool = False, fold_constants: bool = True):
    """Evaluate `kernel` over host arrays.  Returns the typed output (length `kernel.size`, or
    `len(gidx)` when only selected output positions are requested)."""
    L = lib()
    exp = kernel.exp_raw
    re = kernel.reduction
    epi = None
    if re is not None:
        if exp.dtype != re.dtype:  # src/tuner.ts:225-226
            exp = AluExp.cast(re.dtype, exp)
        epi = re.epilogue_raw
    views: List[int] = [0]
    pe, pp = _Program(exp, views, fold_constants), _Program(epi, views, fold_constants)
    ea, pa = pe.arrays(), pp.arrays()
    va = np.asarray(views, dtype=np.int64)

    bufs = []
    for x in inputs:
        if x is None:
            bufs.append(np.zeros(0, dtype=np.uint8))
        else:
            bufs.append(np.ascontiguousarray(np.frombuffer(x, dtype=np.uint8) if isinstance(x, (bytes, bytearray, memoryview))
                                             else np.asarray(x)).view(np.uint8).reshape(-1))
    n = len(bufs)
    ptrs = (ctypes.c_void_p * max(n, 1))(*[b.ctypes.data for b in bufs])
    nbytes = np.asarray([b.nbytes for b in bufs] or [0], dtype=np.int64)

    out_dt = kernel.dtype
    glist = None if gidx is None else np.asarray(list(gidx), dtype=np.int64)
    count = kernel.size if glist is None else len(glist)
    out = np.zeros(max(count, 1), dtype=numpyDtype(out_dt))
    oob = ctypes.c_int64(0)
    err = ctypes.create_string_buffer(256)
    rc = L.jo_run_kernel(
        ctypes.c_int(mode), ctypes.c_int64(kernel.size), ctypes.c_int64(re.size if re else -1),
        ctypes.c_int(_OP[re.op] if re else 0), ctypes.c_int(_DT[re.dtype] if re else 0),
        ctypes.c_int(len(pe.op)), *[_ptr(a) for a in ea],
        ctypes.c_int(len(pp.op)), *[_ptr(a) for a in pa],
        _ptr(va), ctypes.c_int(n), ptrs, _ptr(nbytes),
        _ptr(out), ctypes.c_int(_DT[out_dt]),
        _ptr(glist) if glist is not None else ctypes.c_void_p(0), ctypes.c_int64(count),
        ctypes.byref(oob), err, ctypes.c_int(256),
    )
    if rc != 0:
        raise RuntimeError(f"oracle: {err.value.decode()}")
    out = out[:count]
    return (out, oob.value) if return_oob else out


def wasm_builtin(name: str, x: float) -> float:
    """One of the Wasm backend's software transcendentals, evaluated on a single f32."""
    return float(getattr(lib(), f"jo_wasm_{name}")(ctypes.c_float(x)))
