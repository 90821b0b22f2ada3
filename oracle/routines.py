"""CPU restatement of the reference's routines (src/routine.ts:130-640).  TEST INFRASTRUCTURE ONLY: tests,
the smoke check and the benchmark's CPU leg may call it; the product (`jaxjs_hip`) never does -- its routines
run as GPU kernels or raise.

  Sort / Argsort      numpy (TypedArray.prototype.sort order: NaNs last; Argsort stable)   src/routine.ts:185-213
  Scatter             numpy, sequential semantics (later updates win, adds in order)        src/routine.ts:226-296
  TriangularSolve, Cholesky, LU, JacobiEigh, Fft   C (`routines_oracle.c` + `routines_body.h`), float32 / float64 /
                      float16 elements, every scalar a double as in the reference                 src/routine.ts:298-640
  Attention           numpy float64 (the fused-attention extension)                        src/library/nn.ts:478-583

Parity pinning: the linear-algebra and FFT functions are checked in `tests/test_routines_oracle.py` against what
the mathematics fixes (reconstruction identities, numpy.linalg / numpy.fft / scipy on well-conditioned inputs)
and against the tables the reference's own tests hold; Scatter against brute-force Python loops.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libroutines_oracle.so")
_lib = None

_NP = {"float32": np.float32, "int32": np.int32, "uint32": np.uint32, "bool": np.int32, "float16": np.float16, "float64": np.float64}


def build(force: bool = False) -> str:
    srcs = [os.path.join(_HERE, f) for f in ("routines_oracle.c", "routines_body.h", "half.h", "Makefile")]
    stale = (not os.path.exists(_LIB_PATH)) or any(os.path.getmtime(s) > os.path.getmtime(_LIB_PATH) for s in srcs)
    if force or stale:
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libroutines_oracle.so"], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        P, I64 = ctypes.c_void_p, ctypes.c_int64
        for sfx in ("", "_f64", "_f16"):
            getattr(_lib, "ro_triangular_solve" + sfx).argtypes = [P, P, P, I64, I64, I64, ctypes.c_int]
            getattr(_lib, "ro_cholesky" + sfx).argtypes = [P, P, I64, I64]
            getattr(_lib, "ro_lu" + sfx).argtypes = [P, P, P, P, I64, I64, I64]
            getattr(_lib, "ro_jacobi_eigh" + sfx).argtypes = [P, P, P, I64, I64, I64, ctypes.c_double]
            getattr(_lib, "ro_fft" + sfx).argtypes = [P, P, P, P, I64, I64, P, ctypes.c_int32, ctypes.c_int]
            getattr(_lib, "ro_fft" + sfx).restype = ctypes.c_int
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _typed(bufs: Sequence, dtypes, shapes, writable: bool, views=None) -> List[np.ndarray]:
    """Host buffers as arrays of the routine's operand types.  `views[i]`, when given, says operand i is a strided
    window (element strides, offset) onto a larger buffer instead of the whole of a contiguous one."""
    out = []
    for i, (buf, dt, shape) in enumerate(zip(bufs, dtypes, shapes)):
        a = np.frombuffer(buf, dtype=_NP[str(dt)])
        if writable and not a.flags.writeable:
            raise ValueError("routine outputs must be writable buffers")
        v = views[i] if views else None
        if v is None:
            out.append(a.reshape(shape))
        else:
            if v["elements"] > a.size:
                raise ValueError(f"operand {i}: the view addresses {v['elements']} elements of a buffer of {a.size}")
            out.append(np.lib.stride_tricks.as_strided(a[v["offset"]:], shape=tuple(shape), strides=tuple(sd * a.itemsize for sd in v["strides"]), writeable=False))
    return out


_DENSE = {"float32": ("", np.float32), "float64": ("_f64", np.float64), "float16": ("_f16", np.float16)}


def _dense(name, fn, dtypes):
    """The C function of `fn` for the operands' common floating-point type, and that type in numpy."""
    kinds = {str(d) for d in dtypes}
    if len(kinds) != 1 or next(iter(kinds)) not in _DENSE:
        raise NotImplementedError(f"{name}: the checker covers operands of one floating-point type, got {sorted(kinds)}")
    sfx, npt = _DENSE[next(iter(kinds))]
    return getattr(lib(), fn + sfx), npt


def runCpuRoutine(routine, inputs: Sequence, outputs: Sequence) -> None:
    """Run `routine` (an object with .name, .type, .params like the reference's Routine) on host buffers,
    fully initialising every output (src/routine.ts:130-160)."""
    t = routine.type
    name = str(routine.name)
    params = routine.params or {}
    ins = _typed(inputs, t.inputDtypes, t.inputShapes, False, params.get("views"))
    outs = _typed(outputs, t.outputDtypes, t.outputShapes, True)
    if name == "Sort":
        if ins[0].ndim == 0:
            raise ValueError("sort: cannot sort a scalar")
        outs[0][...] = np.sort(ins[0], axis=-1)
    elif name == "Argsort":
        if ins[0].ndim == 0:
            raise ValueError("argsort: cannot sort a scalar")
        order = np.argsort(ins[0], axis=-1, kind="stable")
        outs[1][...] = order.astype(outs[1].dtype)
        outs[0][...] = np.take_along_axis(ins[0], order, axis=-1)
    elif name == "Scatter":
        scatter(t, ins, outs[0], params)
    elif name == "TriangularSolve":
        fn, npt = _dense(name, "ro_triangular_solve", t.inputDtypes)
        a, b = np.ascontiguousarray(ins[0]), np.ascontiguousarray(ins[1])
        if a.ndim < 2 or b.ndim < 2:
            raise ValueError("triangular_solve: operands must be at least 2D")
        n = a.shape[-2]
        if n != a.shape[-1] or n != b.shape[-1]:
            raise ValueError(f"triangular_solve: incompatible shapes a={a.shape}, b={b.shape}")
        mats = a.size // (n * n) if n else 0
        x = np.zeros(b.shape, npt)
        fn(_ptr(a), _ptr(b), _ptr(x), mats, b.shape[-2], n, int(bool(params.get("unitDiagonal", False))))
        outs[0][...] = x
    elif name == "Cholesky":
        fn, npt = _dense(name, "ro_cholesky", t.inputDtypes)
        a = np.ascontiguousarray(ins[0])
        if a.ndim < 2:
            raise ValueError("cholesky: input must be at least 2D")
        n = a.shape[-2]
        if n != a.shape[-1]:
            raise ValueError(f"cholesky: input must be square, got [{n}, {a.shape[-1]}]")
        y = np.zeros(a.shape, npt)
        with np.errstate(all="ignore"):
            fn(_ptr(a), _ptr(y), a.size // (n * n) if n else 0, n)
        outs[0][...] = y
    elif name == "LU":
        fn, npt = _dense(name, "ro_lu", t.inputDtypes)
        a = np.ascontiguousarray(ins[0])
        if a.ndim < 2:
            raise ValueError("lu: input must be at least 2D")
        m, n = a.shape[-2:]
        mats = int(np.prod(a.shape[:-2], dtype=np.int64))
        lu = np.zeros(a.shape, npt)
        piv = np.zeros(a.shape[:-2] + (min(m, n),), np.int32)
        perm = np.zeros(a.shape[:-2] + (m,), np.int32)
        fn(_ptr(a), _ptr(lu), _ptr(piv), _ptr(perm), mats, m, n)
        outs[0][...], outs[1][...], outs[2][...] = lu, piv, perm
    elif name == "JacobiEigh":
        fn, npt = _dense(name, "ro_jacobi_eigh", t.inputDtypes)
        a = np.ascontiguousarray(ins[0])
        if a.ndim < 2:
            raise ValueError("jacobi_eigh: input must be at least 2D")
        n = a.shape[-1]
        if n != a.shape[-2]:
            raise ValueError(f"jacobi_eigh: input must be square, got {a.shape}")
        d, v = np.zeros(a.shape, npt), np.zeros(a.shape, npt)
        fn(_ptr(a), _ptr(d), _ptr(v), a.size // (n * n) if n else 0, n, int(params["maxSweeps"]), float(params["tolerance"]))
        outs[0][...], outs[1][...] = d, v
    elif name == "Fft":
        fn, npt = _dense(name, "ro_fft", t.inputDtypes)
        re, im = np.ascontiguousarray(ins[0]), np.ascontiguousarray(ins[1])
        if re.ndim < 1:
            raise ValueError("fft: input must be at least 1D")
        n = re.shape[-1]
        if n < 1:
            raise ValueError(f"fft: final axis must be non-empty, got {n}")
        factors = np.asarray(list(params["factors"]), np.int32)
        o_re, o_im = np.zeros(re.shape, npt), np.zeros(re.shape, npt)
        if fn(_ptr(re), _ptr(im), _ptr(o_re), _ptr(o_im), re.size // n, n, _ptr(factors), len(factors), int(bool(params["inverse"]))):
            raise MemoryError("fft oracle: allocation failed")
        outs[0][...], outs[1][...] = o_re, o_im
    elif name == "Attention":
        outs[0][...] = attention(ins[0], ins[1], ins[2], float(params["scale"]), bool(params.get("isCausal", False))).astype(outs[0].dtype)
    else:
        raise NotImplementedError(name)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, causal: bool) -> np.ndarray:
    """softmax_s(scale * q.k (+ mask s <= l)) @ v over [B,L,N,H] / [B,S,N,H] operands, in float64: the function the
    reference's dotProductAttention composes from einsum, where(tri) and softmax (src/library/nn.ts:478-583).  Not a
    reference routine; it checks the fused GPU kernel, and is itself checked against the unfused composition replayed
    kernel by kernel on the CPU checker."""
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    scores = np.einsum("blnh,bsnh->bnls", q64, k64) * scale
    if causal:
        L, S = scores.shape[-2:]
        scores = np.where(np.arange(S)[None, :] <= np.arange(L)[:, None], scores, -np.inf)
    scores = scores - scores.max(axis=-1, keepdims=True)
    p = np.exp(scores)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bnls,bsnh->blnh", p, v64)


def scatter(t, ins: List[np.ndarray], out: np.ndarray, params: dict) -> None:
    """Zero-fill, then write/add each update at the coordinate its index arrays select; updates whose coordinate
    falls outside the output are dropped (src/routine.ts:226-296)."""
    out[...] = 0
    updates, indices = ins[0], ins[1:]
    if updates.size == 0:
        return
    op = str(params["op"])
    op = getattr(params["op"], "value", op)
    out_shape, axes, out_dim = list(params["shape"]), list(params["axis"]), int(params["outDim"])
    accumulate = op != "update" and not params.get("uniqueIndices", False)
    ushape = list(updates.shape)
    index_rank = max(len(i.shape) for i in indices) if indices else 0
    coords = np.indices(ushape).reshape(len(ushape), -1)  # coordinate of every update element, in update order
    free_dims = [d for d in range(len(ushape)) if d < out_dim or d >= out_dim + index_rank]
    flat = np.zeros(coords.shape[1], dtype=np.int64)
    valid = np.ones(coords.shape[1], dtype=bool)
    strides = [int(np.prod(out_shape[d + 1:])) for d in range(len(out_shape))]
    free_iter = iter(free_dims)
    for axis, extent in enumerate(out_shape):
        if axis in axes:
            ia = indices[axes.index(axis)]
            first = out_dim + index_rank - ia.ndim
            sel = tuple(coords[first + j] if ia.shape[j] != 1 else np.zeros_like(coords[0]) for j in range(ia.ndim))
            c = ia[sel].astype(np.int64) if ia.ndim else np.full(coords.shape[1], int(ia), dtype=np.int64)
        else:
            c = coords[next(free_iter)].astype(np.int64)
        valid &= (c >= 0) & (c < extent)
        flat += np.where(valid, c, 0) * strides[axis]
    flat, vals = flat[valid], updates.reshape(-1)[valid]
    target = out.reshape(-1)
    if accumulate and str(t.inputDtypes[0]) == "bool":
        np.bitwise_or.at(target, flat, vals)
    elif accumulate:
        np.add.at(target, flat, vals)  # in update order, rounding to the element type at every step
    else:
        target[flat] = vals  # later updates win, as in the sequential reference loop
