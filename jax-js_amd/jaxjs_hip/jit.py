"""The caller side of the backend: tracing to a Jaxpr and splitting it into Kernels.

This restates the slice of the reference's front-end that decides WHICH Kernels reach a backend,
so that whole programs (the fused softmax/argmax rows, the transformer block) present the same
Kernel sequence to the `hip` backend that `jit()` would:

  Jaxpr, JaxprEqn, Var, Lit, simplify     src/frontend/jaxpr.ts:40-255, 259-360
  promoteAvals / weak types               src/frontend/core.ts:721-736, 1288-1300
  jitRules (expression per primitive)     src/frontend/jit.ts:486-770
  splitGraphDataflow (kernel boundaries)  src/frontend/jit.ts:792-1096
  jitCompile (Kernel construction)        src/frontend/jit.ts:263-469
  JitProgram.execute                      src/frontend/jit.ts:111-162

Only the primitives whose lowering is a fused Kernel are covered (elementwise, Compare, Where,
Reduce, Dot, Conv, Pool, Transpose/Reshape/Broadcast/Flip/Shrink/Pad); routines, Gather, RandomBits,
Concatenate/Split are not traced here; PoolTranspose, which only transforms emit, can be bound by hand.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Set, Tuple, Union

from .alu import AluExp, AluOp, AluVar, DType, Kernel, Reduction, byteWidth, isFloatDtype
from .convolution import ConvParams, checkConvShape, checkPoolShape, pool, poolTranspose, prepareConv
from .shape import ShapeTracker, prod, unravelAlu

# ---- abstract values ------------------------------------------------------------------------------

_RANK = {DType.Bool: 0, DType.Uint32: 1, DType.Int32: 2, DType.Float16: 3, DType.Float32: 4, DType.Float64: 5}


def promoteTypes(a: DType, b: DType) -> DType:
    """src/alu.ts:68-83: the later dtype in bool < u32 < i32 < f16 < f32 < f64."""
    return a if _RANK[a] >= _RANK[b] else b


def generalBroadcast(a: Sequence[int], b: Sequence[int]) -> Tuple[int, ...]:
    out = []
    for i in range(max(len(a), len(b))):
        x = a[len(a) - 1 - i] if i < len(a) else 1
        y = b[len(b) - 1 - i] if i < len(b) else 1
        if x != y and x != 1 and y != 1:
            raise ValueError(f"incompatible shapes for broadcasting: {list(a)} and {list(b)}")
        out.append(max(x, y) if min(x, y) != 0 else 0)
    return tuple(reversed(out))


@dataclass(frozen=True)
class ShapedArray:
    shape: Tuple[int, ...]
    dtype: DType
    weak: bool = False

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return prod(self.shape)


def promoteAvals(a: ShapedArray, b: ShapedArray) -> ShapedArray:
    """src/frontend/core.ts:721-736: a weak (Python-scalar) operand takes the strong one's dtype."""
    shape = generalBroadcast(a.shape, b.shape)
    if a.weak == b.weak:
        dtype = promoteTypes(a.dtype, b.dtype)
    elif a.weak:
        dtype = promoteTypes(b.dtype, DType.Uint32)
    else:
        dtype = promoteTypes(a.dtype, DType.Uint32)
    return ShapedArray(shape, dtype, a.weak and b.weak)


class Var:
    _next = 0

    def __init__(self, aval: ShapedArray):
        self.aval = aval
        Var._next += 1
        self.id = Var._next

    def __repr__(self):
        return f"v{self.id}:{self.aval.dtype.value}{list(self.aval.shape)}"


class Lit:
    def __init__(self, value, aval: ShapedArray):
        self.value = value
        self.aval = aval

    @property
    def dtype(self):
        return self.aval.dtype

    def __repr__(self):
        return f"{self.value}:{self.aval.dtype.value}"


Atom = Union[Var, Lit]


def _is_lit(a: Atom, value=None) -> bool:
    return isinstance(a, Lit) and (value is None or a.value == value)


@dataclass
class JaxprEqn:
    primitive: str
    inputs: List[Atom]
    params: Dict[str, Any]
    outBinders: List[Var]


VIEW_PRIMITIVES = ("Transpose", "Broadcast", "Reshape", "Flip", "Shrink", "Pad")  # src/frontend/jit.ts:905-912
REDUCE_PRIMITIVES = ("Reduce", "Dot", "Conv", "PoolTranspose")
UNARY_FUSABLE = ("Neg", "Reciprocal", "Floor", "Ceil", "StopGradient", "Cast", "Bitcast", "Sin", "Cos", "Asin", "Atan",
                 "Exp", "Log", "Erf", "Erfc", "Sqrt")
BINARY_FUSABLE = ("Add", "Mul", "Idiv", "Mod", "Min", "Max", "BitCombine", "BitShift")
# Primitives handed to the backend as a unit (src/frontend/core.ts:154-163): primitive name == routine name.
# Their outputs index their inputs in several different ways: always dispatched (src/frontend/jit.ts:972-977).
HETEROGENEOUS_VIEW_PRIMITIVES = ("RandomBits", "Gather")
# Routines that take an operand as base buffer + strides + offset, with the views each one accepts (fused attention:
# 128-bit loads along the head dimension, so unit stride there and everything else a multiple of 8 elements).
STRIDED_OPERAND_ROUTINES = {"Attention": lambda strides, offset: strides[-1] == 1 and offset % 8 == 0 and all(s % 8 == 0 for s in strides[:-1])}
ROUTINE_PRIMITIVES = ("Sort", "Argsort", "Scatter", "TriangularSolve", "Cholesky", "LU", "JacobiEigh", "Fft",
                      "Attention")  # the last one is this backend's extension (fused attention), see routine.py


@dataclass
class Jaxpr:
    inBinders: List[Var]
    eqns: List[JaxprEqn]
    outs: List[Atom]

    def simplify(self) -> "Jaxpr":
        """Fold +0 / *1 / literal arithmetic and drop no-op movement ops and dead equations
        (src/frontend/jaxpr.ts:259-360)."""
        ctx: Dict[Var, Atom] = {}
        new: List[JaxprEqn] = []
        for e in self.eqns:
            inputs = [ctx.get(x, x) if isinstance(x, Var) else x for x in e.inputs]
            eqn = JaxprEqn(e.primitive, inputs, e.params, e.outBinders)
            c = eqn.outBinders[0]
            p = eqn.primitive
            if p == "Add":
                a, b = inputs
                if _is_lit(a, 0):
                    ctx[c] = b
                elif _is_lit(b, 0):
                    ctx[c] = a
                elif _is_lit(a) and _is_lit(b):
                    v = min(a.value + b.value, 1) if a.dtype == DType.Bool else a.value + b.value
                    ctx[c] = Lit(v, promoteAvals(a.aval, b.aval))
                else:
                    new.append(eqn)
            elif p == "Neg":
                (a,) = inputs
                if _is_lit(a):
                    ctx[c] = Lit(-a.value, a.aval)
                else:
                    new.append(eqn)
            elif p == "Mul":
                a, b = inputs
                if _is_lit(a, 1):
                    ctx[c] = b
                elif _is_lit(b, 1):
                    ctx[c] = a
                elif _is_lit(a) and _is_lit(b):
                    ctx[c] = Lit(a.value * b.value, promoteAvals(a.aval, b.aval))
                else:
                    new.append(eqn)
            elif p == "Idiv":
                a, b = inputs
                if _is_lit(b, 1) and not isFloatDtype(a.aval.dtype):
                    ctx[c] = a
                else:
                    new.append(eqn)
            elif ((p in ("Broadcast", "Reshape") and tuple(eqn.params["shape"]) == tuple(inputs[0].aval.shape))
                  or (p == "Transpose" and all(q == i for i, q in enumerate(eqn.params["perm"])))
                  or (p == "Flip" and len(eqn.params["axis"]) == 0)
                  or (p == "Shrink" and all(s == 0 and e_ == inputs[0].aval.shape[i]
                                            for i, (s, e_) in enumerate(eqn.params["slice"])))
                  or (p == "Pad" and all(w0 == 0 and w1 == 0 for w0, w1 in eqn.params["width"]))):
                ctx[c] = inputs[0]
            else:
                new.append(eqn)
        outs = [ctx.get(x, x) if isinstance(x, Var) else x for x in self.outs]
        used: Set[Var] = {x for x in outs if isinstance(x, Var)}
        live: List[JaxprEqn] = []
        for eqn in reversed(new):
            if any(v in used for v in eqn.outBinders):
                live.append(eqn)
                used.update(v for v in eqn.inputs if isinstance(v, Var))
        return Jaxpr(self.inBinders, list(reversed(live)), outs)

    def __str__(self):
        lines = ["{ lambda " + ", ".join(map(repr, self.inBinders)) + " ."]
        for e in self.eqns:
            ps = " ".join(f"{k}={v}" for k, v in e.params.items())
            lines.append(f"  {', '.join(map(repr, e.outBinders))} = {e.primitive}[{ps}] " + " ".join(map(repr, e.inputs)))
        lines.append("  in " + ", ".join(map(repr, self.outs)) + " }")
        return "\n".join(lines)


# ---- tracing ---------------------------------------------------------------------------------------

class _Builder:
    def __init__(self):
        self.eqns: List[JaxprEqn] = []
        self.consts: List[Tuple[Var, "ConstArray"]] = []
        self._const_vars: Dict[int, Var] = {}

    def const_var(self, c: "ConstArray") -> Var:
        v = self._const_vars.get(id(c))
        if v is None:
            v = Var(ShapedArray(tuple(c.shape), c.dtype, False))
            self._const_vars[id(c)] = v
            self.consts.append((v, c))
        return v


_builders: List[_Builder] = []


@dataclass
class ConstArray:
    """An array that exists before the traced function runs (the reference realises such closed-over
    arrays and passes them as leading jit inputs, src/frontend/jaxpr.ts:1166-1169).  `exp` is its lazy
    definition over `AluVar.idx`-free `gidx` (as arange/tri build them, src/frontend/array.ts:1570-1627);
    `kernel()` is the nullary Kernel that realises it."""
    shape: Tuple[int, ...]
    dtype: DType
    exp: AluExp

    def kernel(self) -> Kernel:
        return Kernel(0, prod(self.shape), self.exp)


TracerValue = Union["Tracer", int, float, bool, ConstArray]


class Tracer:
    def __init__(self, atom: Atom):
        self.atom = atom

    @property
    def aval(self) -> ShapedArray:
        return self.atom.aval

    @property
    def shape(self):
        return self.aval.shape

    @property
    def dtype(self):
        return self.aval.dtype

    @property
    def ndim(self):
        return len(self.shape)

    # -- primitives as methods (src/frontend/core.ts:800-960) --
    def add(self, o):
        return add(self, o)

    def mul(self, o):
        return mul(self, o)

    def sub(self, o):
        return add(self, neg(o))  # core.ts:945-947

    def div(self, o):
        return mul(self, reciprocal(o)) if isFloatDtype(self.dtype) else bind1("Idiv", [self, o])  # :950-955

    def astype(self, dtype: DType):
        return self if self.dtype == dtype else bind1("Cast", [self], dict(dtype=dtype))

    def view(self, dtype: Optional[DType] = None):
        """Reinterpret the bits as another type of the same width (core.ts:937-940)."""
        return self if dtype is None or dtype == self.dtype else bitcast(self, dtype)

    def greater(self, o): return greater(self, o)
    def greaterEqual(self, o): return greaterEqual(self, o)
    def less(self, o): return less(self, o)
    def lessEqual(self, o): return lessEqual(self, o)
    def equal(self, o): return equal(self, o)
    def notEqual(self, o): return notEqual(self, o)

    def flatten(self):
        return reshape(self, [-1])

    def ravel(self):
        return reshape(self, [-1])

    def slice(self, *index):
        """Indexing as the reference's `Tracer.slice` spells it (core.ts:1110-1231): an int picks one entry of an axis and
        drops the axis (negative counts from the end), `[]` keeps the axis, `[i]` is `i:`, `[i, j]` is `i:j`, `None` adds
        an axis, an integer array gathers along its axis.  Several arrays broadcast together; their dimensions stay in
        place when the arrays and ints sit next to each other in the index and move to the front otherwise (numpy's
        rule).  Strided slices are not part of it."""
        def bound(n: int, i: int) -> int:
            if i > n or i < -n:
                raise IndexError(f"Index {i} out of bounds for axis of size {n}")
            return n + i if i < 0 else i

        is_array = lambda v: isinstance(v, (Tracer, ConstArray))  # noqa: E731
        arrays = [v for v in index if is_array(v)]
        gather_axes: List[int] = []
        out_dim = -1
        if arrays:
            advanced, at = [], 0
            for pos, v in enumerate(index):
                if is_array(v):
                    advanced.append(pos)
                    gather_axes.append(at)
                    at += 1
                elif isinstance(v, int) and not isinstance(v, bool):
                    advanced.append(pos)  # squeezed out: takes no axis of the sliced array
                else:
                    at += 1
            out_dim = gather_axes[0] if advanced[-1] - advanced[0] == len(advanced) - 1 else 0
        window, shape, reshaped, axis = [], [], False, 0
        for v in index:
            if v is None:
                shape.append(1)
                reshaped = True
                continue
            if axis >= self.ndim:
                raise IndexError("Too many indices")
            n = self.shape[axis]
            axis += 1
            if is_array(v):
                shape.append(n)
                window.append((0, n))
            elif isinstance(v, int) and not isinstance(v, bool):
                i = bound(n, v)
                window.append((i, i + 1))
                reshaped = True
            elif isinstance(v, (list, tuple)) and len(v) <= 2:
                lo = bound(n, v[0]) if len(v) >= 1 else 0
                hi = bound(n, v[1]) if len(v) == 2 else n
                if lo > hi:
                    raise IndexError(f"Slice start at {lo} > end at {hi}")
                shape.append(hi - lo)
                window.append((lo, hi))
            else:
                raise TypeError(f"Invalid slice argument: {v!r}")
        for n in self.shape[axis:]:
            window.append((0, n))
            shape.append(n)
        out = shrink(self, window)
        if reshaped:
            out = reshape(out, shape)
        return gather(out, arrays, gather_axes, out_dim) if arrays else out

    def reshape(self, shape):
        return reshape(self, shape)

    def transpose(self, perm=None):
        return transpose(self, perm)

    def sum(self, axis=None, keepdims=False):
        return reduce(self, AluOp.Add, axis, keepdims)

    def max(self, axis=None, keepdims=False):
        return reduce(self, AluOp.Max, axis, keepdims)

    def min(self, axis=None, keepdims=False):
        return reduce(self, AluOp.Min, axis, keepdims)

    def mean(self, axis=None, keepdims=False):
        """f32 sum times 1/n, cast back for float inputs (core.ts:878-893)."""
        ax = _normalize_axis(axis, self.ndim)
        n = prod([self.shape[a] for a in ax])
        if n == 0:
            raise ValueError("mean: cannot compute mean over zero-length axis")
        orig = self.dtype
        out = reduce(self.astype(promoteTypes(orig, DType.Float32)), AluOp.Add, ax, keepdims).mul(1 / n)
        return out.astype(orig) if isFloatDtype(orig) else out


def _raise(x: TracerValue) -> Tracer:
    if isinstance(x, Tracer):
        return x
    if isinstance(x, ConstArray):
        return Tracer(_builders[-1].const_var(x))
    if isinstance(x, bool):
        return Tracer(Lit(int(x), ShapedArray((), DType.Bool, False)))  # core.ts:1291-1296
    if isinstance(x, (int, float)):
        return Tracer(Lit(float(x), ShapedArray((), DType.Float32, True)))
    raise TypeError(f"Unknown value: {x!r}")


def scalar(value, dtype: DType) -> Tracer:
    """A strongly typed scalar literal (`array(5, {dtype})`, inlined by jaxpr.ts `_inlineLiterals`)."""
    return Tracer(Lit(value, ShapedArray((), dtype, False)))


def _normalize_axis(axis, ndim) -> List[int]:
    if axis is None:
        return list(range(ndim))
    if isinstance(axis, int):
        axis = [axis]
    return sorted({a + ndim if a < 0 else a for a in axis})


def _out_aval(prim: str, avals: List[ShapedArray], params: Dict[str, Any]) -> ShapedArray:
    if prim in BINARY_FUSABLE:
        return promoteAvals(avals[0], avals[1])
    if prim == "Compare":
        return ShapedArray(generalBroadcast(avals[0].shape, avals[1].shape), DType.Bool, False)
    if prim == "Where":
        xy = promoteAvals(avals[1], avals[2])
        return ShapedArray(generalBroadcast(avals[0].shape, xy.shape), xy.dtype, xy.weak)
    if prim == "Bitcast":  # src/frontend/jaxpr.ts:838-848
        src_dt, dtype = avals[0].dtype, params["dtype"]
        if src_dt != dtype and DType.Bool in (src_dt, dtype):
            raise TypeError("Bitcast to/from bool is not allowed")
        if byteWidth(src_dt) != byteWidth(dtype):
            raise TypeError(f"Bitcast from {src_dt.value} to {dtype.value} with different byte width")
        return ShapedArray(avals[0].shape, dtype, False)
    if prim == "Cast":
        return ShapedArray(avals[0].shape, params["dtype"], False)
    if prim in UNARY_FUSABLE:
        return avals[0]
    if prim == "Reduce":
        ax = params["axis"]
        return ShapedArray(tuple(d for i, d in enumerate(avals[0].shape) if i not in ax), avals[0].dtype, avals[0].weak)
    if prim == "Dot":
        c = promoteAvals(avals[0], avals[1])
        return ShapedArray(c.shape[:-1], c.dtype, c.weak)
    if prim == "Conv":
        c = promoteAvals(ShapedArray((), avals[0].dtype, avals[0].weak), ShapedArray((), avals[1].dtype, avals[1].weak))
        return ShapedArray(tuple(checkConvShape(avals[0].shape, avals[1].shape, params["conv"])), c.dtype, c.weak)
    if prim == "Pool":
        return ShapedArray(tuple(checkPoolShape(avals[0].shape, params["window"], params["strides"])), avals[0].dtype, avals[0].weak)
    if prim == "PoolTranspose":  # src/frontend/jaxpr.ts:867-882
        want = checkPoolShape(params["inShape"], params["window"], params["strides"])
        if list(avals[0].shape) != list(want):
            raise ValueError(f"poolTranspose() of shape {list(avals[0].shape)}: a pool of {list(params['inShape'])} has shape {want}")
        return ShapedArray(tuple(params["inShape"]), avals[0].dtype, avals[0].weak)
    if prim == "Transpose":
        return ShapedArray(tuple(avals[0].shape[p] for p in params["perm"]), avals[0].dtype, avals[0].weak)
    if prim in ("Reshape", "Broadcast"):
        return ShapedArray(tuple(params["shape"]), avals[0].dtype, avals[0].weak)
    if prim == "Flip":
        return avals[0]
    if prim == "Shrink":
        return ShapedArray(tuple(e - s for s, e in params["slice"]), avals[0].dtype, avals[0].weak)
    if prim == "Pad":
        return ShapedArray(tuple(d + a + b for d, (a, b) in zip(avals[0].shape, params["width"])), avals[0].dtype, avals[0].weak)
    if prim == "Concatenate":
        ax = params["axis"]
        first = avals[0]
        for x in avals:
            if x.ndim != first.ndim or any(i != ax and a != b for i, (a, b) in enumerate(zip(x.shape, first.shape))):
                raise TypeError(f"Concatenate: inputs {first.shape} and {x.shape} must match shapes except on axis {ax}")
        shape = list(first.shape)
        shape[ax] = sum(x.shape[ax] for x in avals)
        d = ShapedArray((), first.dtype, first.weak)
        for x in avals[1:]:
            d = promoteAvals(d, ShapedArray((), x.dtype, x.weak))
        return ShapedArray(tuple(shape), d.dtype, d.weak)
    if prim == "RandomBits":
        k0, k1 = avals
        shape = tuple(params["shape"])
        if k0.dtype != DType.Uint32 or k1.dtype != DType.Uint32:
            raise TypeError(f"RandomBits requires uint32 keys, got {k0.dtype} and {k1.dtype}")
        if tuple(k0.shape) != tuple(k1.shape) or shape[:k0.ndim] != tuple(k0.shape):
            raise TypeError(f"RandomBits: generated shape {shape} must match key shape {k0.shape}")
        return ShapedArray(shape, DType.Uint32, False)
    if prim == "Gather":
        x, indices = avals[0], avals[1:]
        return ShapedArray(tuple(gatherShape(x.shape, indices, params["axis"], params["outDim"])), x.dtype, x.weak)
    raise NotImplementedError(f"jit: primitive {prim}")


def gatherShape(operandShape, indices: Sequence[ShapedArray], axis: Sequence[int], outDim: int) -> List[int]:
    """Result shape of `x[:, ...indices, :]` with the index dimensions placed at `outDim` (src/frontend/jaxpr.ts:774-800)."""
    for a in indices:
        if a.dtype not in (DType.Int32, DType.Uint32):
            raise TypeError(f"indices must be Int32 or Uint32, got {a.dtype}")
    if len(axis) != len(indices):
        raise TypeError(f"got {list(axis)} axes but {len(indices)} indices")
    if not indices:
        raise TypeError("must have at least one index")
    if any(a < 0 or a >= len(operandShape) for a in axis):
        raise TypeError("axis out of bounds")
    if outDim < 0 or outDim > len(operandShape) - len(axis):
        raise TypeError("outDim out of bounds")
    if len(set(axis)) != len(axis):
        raise TypeError("axes are not unique")
    indexShape: Tuple[int, ...] = ()
    for a in indices:
        indexShape = generalBroadcast(indexShape, a.shape)
    result = [d for i, d in enumerate(operandShape) if i not in set(axis)]
    result[outDim:outDim] = list(indexShape)
    return result


def _routine_out_avals(prim: str, avals: List[ShapedArray], params: Dict[str, Any]) -> List[ShapedArray]:
    """Output types of the routine primitives (src/frontend/jaxpr.ts:976-1062)."""
    a = avals[0]
    same = ShapedArray(tuple(a.shape), a.dtype, a.weak)
    if prim == "Split":  # a fusable multi-output primitive, not a routine (src/frontend/jaxpr.ts:913-927)
        ax, sizes = params["axis"], list(params["sizes"])
        if a.shape[ax] != sum(sizes):
            raise TypeError(f"Split: sizes {sizes} do not sum to dimension {a.shape[ax]} on axis {ax}")
        return [ShapedArray(tuple(a.shape[:ax]) + (sz,) + tuple(a.shape[ax + 1:]), a.dtype, a.weak) for sz in sizes]
    if prim in ("Sort", "Argsort"):
        if a.ndim == 0:
            raise TypeError(f"{prim.lower()}: requires at least 1D input")
        return [same] if prim == "Sort" else [same, ShapedArray(tuple(a.shape), DType.Int32, False)]
    if prim == "Scatter":
        return [ShapedArray(tuple(params["shape"]), a.dtype, a.weak)]
    if prim == "TriangularSolve":
        b = avals[1]
        if a.ndim < 2 or b.ndim < 2:
            raise TypeError("triangular_solve: operands must be at least 2D")
        if (tuple(a.shape[:-2]) != tuple(b.shape[:-2]) or a.dtype != b.dtype or a.shape[-2] != a.shape[-1]
                or a.shape[-1] != b.shape[-1]):
            raise TypeError(f"triangular_solve: mismatch {a.shape} vs {b.shape}")
        return [ShapedArray(tuple(b.shape), b.dtype, a.weak and b.weak)]
    if prim in ("Cholesky", "JacobiEigh"):
        if a.ndim < 2 or a.shape[-2] != a.shape[-1]:
            raise TypeError(f"{prim.lower()}: requires a batch of square matrices, got {a.shape}")
        if prim == "Cholesky":
            return [same]
        if a.dtype not in (DType.Float16, DType.Float32, DType.Float64):
            raise TypeError("jacobi_eigh: requires floating-point input")
        return [same, same]
    if prim == "LU":
        if a.ndim < 2:
            raise TypeError("lu: requires at least 2D input")
        batch, (m, n) = tuple(a.shape[:-2]), a.shape[-2:]
        return [same, ShapedArray(batch + (min(m, n),), DType.Int32, False), ShapedArray(batch + (m,), DType.Int32, False)]
    if prim == "Attention":
        k, v = avals[1], avals[2]
        if a.ndim != 4 or tuple(k.shape) != tuple(v.shape) or k.ndim != 4 or (k.shape[0], k.shape[2], k.shape[3]) != (a.shape[0], a.shape[2], a.shape[3]):
            raise TypeError(f"attention: shape mismatch q={a.shape} k={k.shape} v={v.shape}")
        return [same]
    if prim == "Fft":
        b = avals[1]
        if tuple(a.shape) != tuple(b.shape) or a.dtype != b.dtype:
            raise TypeError("fft: real and imag arrays must match")
        if a.ndim < 1 or a.dtype not in (DType.Float16, DType.Float32, DType.Float64):
            raise TypeError("fft: requires floating-point input of at least 1D")
        if prod(list(params["factors"])) != a.shape[-1]:
            raise TypeError(f"fft: factorization {params['factors']} does not match size {a.shape[-1]}")
        return [same, same]
    raise NotImplementedError(prim)


def bind(prim: str, args: Sequence[TracerValue], params: Optional[Dict[str, Any]] = None) -> List[Tracer]:
    """Multi-output primitive application; the routine primitives go through here."""
    if not _builders:
        raise RuntimeError("bind outside of a trace")
    ts = [_raise(a) for a in args]
    params = dict(params or {})
    outs = [Var(av) for av in _routine_out_avals(prim, [t.aval for t in ts], params)]
    _builders[-1].eqns.append(JaxprEqn(prim, [t.atom for t in ts], params, outs))
    return [Tracer(o) for o in outs]


def bind1(prim: str, args: Sequence[TracerValue], params: Optional[Dict[str, Any]] = None) -> Tracer:
    if not _builders:
        raise RuntimeError("bind1 outside of a trace")
    ts = [_raise(a) for a in args]
    params = dict(params or {})
    out = Var(_out_aval(prim, [t.aval for t in ts], params))
    _builders[-1].eqns.append(JaxprEqn(prim, [t.atom for t in ts], params, [out]))
    return Tracer(out)


def add(x, y): return bind1("Add", [x, y])
def mul(x, y): return bind1("Mul", [x, y])
def neg(x): return bind1("Neg", [x])
def reciprocal(x): return bind1("Reciprocal", [x])
def exp(x): return bind1("Exp", [x])
def log(x): return bind1("Log", [x])
def sqrt(x): return bind1("Sqrt", [x])
def erfc(x): return bind1("Erfc", [x])
def erf(x): return bind1("Erf", [x])
def sin(x): return bind1("Sin", [x])
def cos(x): return bind1("Cos", [x])
def asin(x): return bind1("Asin", [x])
def atan(x): return bind1("Atan", [x])
def floor(x): return bind1("Floor", [x])
def ceil(x): return bind1("Ceil", [x])
def idiv(x, y): return bind1("Idiv", [x, y])
def mod(x, y): return bind1("Mod", [x, y])  # sign of the numerator (core.ts:43)
def bitCombine(x, y, op: str): return bind1("BitCombine", [x, y], dict(op=op))  # core.ts:189-195
def bitShift(x, y, op: str): return bind1("BitShift", [x, y], dict(op=op))  # core.ts:197-199
def bitcast(x, dtype: DType): return bind1("Bitcast", [x], dict(dtype=dtype))
def stopGradient(x): return bind1("StopGradient", [x])
def maximum(x, y): return bind1("Max", [x, y])
def minimum(x, y): return bind1("Min", [x, y])
def where(c, x, y): return bind1("Where", [c, x, y])
def less(x, y): return bind1("Compare", [x, y], dict(op="Less"))
def greater(x, y): return bind1("Compare", [y, x], dict(op="Less"))
def equal(x, y): return bind1("Compare", [x, y], dict(op="Equal"))
def notEqual(x, y): return bind1("Compare", [x, y], dict(op="NotEqual"))
def lessEqual(x, y): return bind1("Compare", [x, y], dict(op="LessEqual"))
def greaterEqual(x, y): return bind1("Compare", [y, x], dict(op="LessEqual"))  # core.ts:329-331


def dot(x, y):
    return bind1("Dot", [x, y])


def conv(x, y, params: ConvParams):
    """The Conv primitive (src/frontend/core.ts:295-312): shapes are checked when the output aval is formed."""
    return bind1("Conv", [x, y], dict(conv=params))


def poolWindows(x, window, strides):
    """The Pool primitive: `[..., *spatial] -> [..., *out, *window]` (a view; reduce the trailing axes)."""
    return bind1("Pool", [x], dict(window=tuple(window), strides=tuple(strides)))


def transpose(x, perm=None):
    x = _raise(x)
    perm = list(reversed(range(x.ndim))) if perm is None else [p + x.ndim if p < 0 else p for p in perm]
    return bind1("Transpose", [x], dict(perm=perm))


def reshape(x, shape):
    x = _raise(x)
    shape = [shape] if isinstance(shape, int) else list(shape)
    if -1 in shape:
        known = prod([d for d in shape if d != -1])
        shape[shape.index(-1)] = x.aval.size // max(known, 1)
    if prod(shape) != x.aval.size:
        raise ValueError(f"reshape: cannot reshape {list(x.shape)} into {shape}")
    return bind1("Reshape", [x], dict(shape=tuple(shape)))


def broadcast(x, shape, axis):
    return bind1("Broadcast", [x], dict(shape=tuple(shape), axis=list(axis)))


def shrink(x, slices):
    """`x.slice(...)`: keep `[start, end)` per axis."""
    return bind1("Shrink", [x], dict(slice=[tuple(s) for s in slices]))


def pad(x, width):
    """Zero padding `[(before, after), ...]` per axis (the Pad primitive, src/frontend/core.ts:253-262)."""
    return bind1("Pad", [x], dict(width=[tuple(w) for w in width]))


def flip(x, axis):
    x = _raise(x)
    return bind1("Flip", [x], dict(axis=_normalize_axis(axis, x.ndim)))


def concatenate(xs, axis: int):
    xs = [_raise(x) for x in xs]
    if not xs:
        raise ValueError("concatenate requires at least one input")
    (axis,) = _normalize_axis(axis, xs[0].ndim)
    return bind1("Concatenate", xs, dict(axis=axis))


def split(x, axis: int, sizes):
    x = _raise(x)
    (axis,) = _normalize_axis(axis, x.ndim)
    sizes = [int(sz) for sz in sizes]
    if any(sz < 0 for sz in sizes) or sum(sizes) != x.shape[axis]:
        raise ValueError(f"split: sizes must be nonnegative and sum to the size of axis {axis}, got {sizes}")
    return bind("Split", [x], dict(axis=axis, sizes=sizes))


def randomBits(k0, k1, shape, mode="xor"):
    return bind1("RandomBits", [k0, k1], dict(shape=tuple(shape), mode=mode))


def gather(x, indices, axis, outDim: int):
    """`x[:, ...indices, :]` with the broadcast index dimensions starting at `outDim` (src/frontend/core.ts:414-434)."""
    x = _raise(x)
    axis = [a + x.ndim if a < 0 else a for a in axis]
    return bind1("Gather", [x] + list(indices), dict(axis=axis, outDim=int(outDim)))


def sort(x):
    return bind("Sort", [x])[0]


def argsort(x):
    """Returns (sorted values, int32 indices) along the last axis (src/frontend/core.ts:600-605)."""
    return tuple(bind("Argsort", [x]))


def scatter(updates, indices, params):
    return bind("Scatter", [updates] + list(indices), params)[0]


def triangularSolve(a, b, lower: bool = False, unitDiagonal: bool = False):
    """Solves `a @ x.T = b.T`; a lower-triangular system is flipped into the upper-triangular form the routine
    takes (src/frontend/core.ts:530-555)."""
    if lower:
        a, b = flip(a, [-2, -1]), flip(b, [-1])
    x = bind("TriangularSolve", [a, b], dict(unitDiagonal=bool(unitDiagonal)))[0]
    return flip(x, [-1]) if lower else x


def cholesky(x):
    return bind("Cholesky", [x])[0]


def lu(x):
    return tuple(bind("LU", [x]))


def jacobiEigh(x, maxSweeps: int, tolerance: float):
    return tuple(bind("JacobiEigh", [x], dict(maxSweeps=int(maxSweeps), tolerance=float(tolerance))))


def attention(q, k, v, scale: float, isCausal: bool):
    """Fused scaled-dot-product attention as one backend routine (an extension; the reference composes it)."""
    return bind("Attention", [q, k, v], dict(scale=float(scale), isCausal=bool(isCausal)))[0]


def fft(real, imag, factors, inverse: bool):
    return tuple(bind("Fft", [real, imag], dict(factors=[int(f) for f in factors], inverse=bool(inverse))))


def reduce(x, op: AluOp, axis=None, keepdims=False):
    """src/frontend/core.ts:271-289."""
    x = _raise(x)
    ax = _normalize_axis(axis, x.ndim)
    original = x.shape
    out = bind1("Reduce", [x], dict(op=op, axis=ax))
    if keepdims:
        out = out.reshape([1 if i in ax else d for i, d in enumerate(original)])
    return out


def trace(fn: Callable[..., Any], avals: Sequence[ShapedArray]) -> Tuple[Jaxpr, List[ConstArray]]:
    """Run `fn` on tracers and return the simplified Jaxpr; closed-over ConstArrays come first in
    `inBinders` (src/frontend/jaxpr.ts:707-720)."""
    b = _Builder()
    _builders.append(b)
    try:
        ins = [Var(a) for a in avals]
        outs = fn(*[Tracer(v) for v in ins])
        if isinstance(outs, (Tracer, ConstArray, int, float, bool)):
            outs = [outs]
        out_atoms = [_raise(o).atom for o in outs]
    finally:
        _builders.pop()
    jaxpr = Jaxpr([v for v, _ in b.consts] + ins, b.eqns, out_atoms).simplify()
    return jaxpr, [c for _, c in b.consts]


# ---- jit rules: one expression per primitive (src/frontend/jit.ts:486-770) -----------------------

def reshapeViews(exp: AluExp, mapping: Callable[[ShapeTracker], Optional[ShapeTracker]], reduceAxis: bool = False) -> AluExp:
    def visit(e: AluExp):
        if e.op == AluOp.GlobalView:
            gid, st = e.arg
            new = mapping(st)
            if new is not None:
                if reduceAxis:
                    indices = unravelAlu(new.shape[:-1], AluVar.gidx) + [AluVar.ridx]
                else:
                    indices = unravelAlu(new.shape, AluVar.gidx)
                return AluExp.globalView(e.dtype, gid, new, indices)
        elif e.op == AluOp.GlobalIndex:
            raise RuntimeError("internal: reshapeViews() called with GlobalIndex op")
        return None
    return exp.rewrite(visit)


def aluCompare(a: AluExp, b: AluExp, op: str) -> AluExp:
    """src/frontend/array.ts:1786-1800."""
    if op == "Less":
        return AluExp.cmplt(a, b)
    if op == "Equal":
        return AluExp.cmpne(a, b).not_()
    if op == "NotEqual":
        return AluExp.cmpne(a, b)
    if op == "LessEqual":
        return AluExp.add(AluExp.cmplt(a, b), AluExp.cmpne(a, b).not_())
    raise ValueError(op)


def _broadcasted(fn, skipCastIdx=()):
    def rule(exps, avals, params):
        new = avals[0]
        for a in avals[1:]:
            new = promoteAvals(new, a)
        newShape, newDtype = new.shape, new.dtype
        if skipCastIdx:
            rest = [a for i, a in enumerate(avals) if i not in skipCastIdx]
            d = rest[0]
            for a in rest[1:]:
                d = promoteAvals(d, a)
            newDtype = d.dtype
        out = []
        for i, e in enumerate(exps):
            def mapping(st, _shape=newShape):
                if tuple(st.shape) != tuple(_shape):
                    return st.broadcast(list(_shape), list(range(len(_shape) - len(st.shape))))
                return None
            e = reshapeViews(e, mapping)
            if e.dtype != newDtype and i not in skipCastIdx:
                e = AluExp.cast(newDtype, e)
            out.append(e)
        return [fn(out, params)], None
    return rule


def _unop(fn):
    return lambda exps, avals, params: ([fn(exps[0], params)], None)


def _reshape_rule(fn):
    return lambda exps, avals, params: ([reshapeViews(exps[0], lambda st: fn(st, params))], None)


def _reduce_rule(exps, avals, params):
    a, aval = exps[0], avals[0]
    axis = params["axis"]
    kept = [i for i in range(aval.ndim) if i not in axis]
    shifted = [i for i in range(aval.ndim) if i in axis]
    newShape = [aval.shape[i] for i in kept]
    rsize = prod([aval.shape[i] for i in shifted])
    newShape.append(rsize)
    perm = kept + shifted
    a = reshapeViews(a, lambda st: st.permute(perm).reshape(newShape), True)
    return [a], Reduction(a.dtype, params["op"], rsize)


def _dot_rule(exps, avals, params):
    (c,), _ = JIT_RULES["Mul"](exps, avals, {})
    cs = promoteAvals(avals[0], avals[1])
    return _reduce_rule([c], [cs], dict(op=AluOp.Add, axis=[cs.ndim - 1]))


def _conv_rule(exps, avals, params):
    """src/frontend/jit.ts:622-635: re-view both operands, then it is a Dot."""
    stX, stY = prepareConv(ShapeTracker.fromShape(list(avals[0].shape)), ShapeTracker.fromShape(list(avals[1].shape)), params["conv"])
    a = reshapeViews(exps[0], lambda st: st.compose(stX))
    b = reshapeViews(exps[1], lambda st: st.compose(stY))
    as_ = ShapedArray(tuple(stX.shape), avals[0].dtype, avals[0].weak)
    bs_ = ShapedArray(tuple(stY.shape), avals[1].dtype, avals[1].weak)
    return _dot_rule([a, b], [as_, bs_], {})


def _pool_transpose_rule(exps, avals, params):
    """src/frontend/jit.ts:623-638: the adjoint pool view with its repeat axes merged, summed over them."""
    inShape = list(params["inShape"])
    stX = poolTranspose(ShapeTracker.fromShape(list(avals[0].shape)), inShape, list(params["window"]), list(params["strides"]))
    stX = stX.reshape(inShape + [prod(list(stX.shape[len(inShape):]))])
    a = reshapeViews(exps[0], lambda st: st.compose(stX), True)
    return [a], Reduction(a.dtype, AluOp.Add, stX.shape[-1])


def poolTransposeWindows(ct, inShape, window, strides):
    """The PoolTranspose primitive (src/frontend/core.ts:112-116): `[..., *out, *window] -> inShape`, every pooled element
    added back onto the input position it was read from.  Only transforms bind it in the reference (the transpose rule
    of Pool, src/frontend/linearize.ts:755-762); it is here so that those Kernels can be presented to the backend."""
    return bind1("PoolTranspose", [ct], dict(inShape=tuple(inShape), window=tuple(window), strides=tuple(strides)))


def convTransposeLhs(ct, rhs, lhsShape, p):
    """What the transpose rule of Conv binds for the cotangent of the activations (src/frontend/linearize.ts:783-812):
    a convolution of the cotangent with the flipped filter whose channel axes are exchanged.  Only transforms bind it in
    the reference; it is here, like `poolTransposeWindows`, so that those Kernels can be presented to the backend."""
    v = p.vmapDims
    rev01 = list(range(v)) + [v + 1, v] + list(range(v + 2, ct.ndim))
    kernel = flip(transpose(rhs, rev01), list(range(v + 2, rhs.ndim)))
    padding = []
    for i, (pl, _pr) in enumerate(p.padding):
        dil_k = (kernel.shape[i + v + 2] - 1) * p.rhsDilation[i] + 1
        dil_ct = (ct.shape[i + v + 2] - 1) * p.strides[i] + 1
        before = dil_k - 1 - pl
        dil_lhs = (lhsShape[i + v + 2] - 1) * p.lhsDilation[i] + 1
        padding.append((before, dil_lhs + dil_k - 1 - dil_ct - before))
    return conv(ct, kernel, ConvParams(v, list(p.lhsDilation), padding, list(p.strides), list(p.rhsDilation)))


def convTransposeRhs(lhs, ct, rhsShape, p):
    """The cotangent of the filter (src/frontend/linearize.ts:813-837): the activations convolved with the cotangent, batch
    and channel axes exchanged on both, window strides and filter dilations exchanged."""
    v = p.vmapDims
    rev01 = list(range(v)) + [v + 1, v] + list(range(v + 2, ct.ndim))
    padding = []
    for i, (pl, _pr) in enumerate(p.padding):
        dil_lhs = (lhs.shape[i + v + 2] - 1) * p.lhsDilation[i] + 1
        dil_k = (rhsShape[i + v + 2] - 1) * p.rhsDilation[i] + 1
        dil_ct = (ct.shape[i + v + 2] - 1) * p.strides[i] + 1
        padding.append((pl, dil_ct - dil_lhs + dil_k - pl - 1))
    out = conv(transpose(lhs, rev01), transpose(ct, rev01), ConvParams(v, list(p.rhsDilation), padding, list(p.lhsDilation), list(p.strides)))
    return transpose(out, rev01)


def _flip_rule(st, params):
    arg = [False] * len(st.shape)
    for ax in params["axis"]:
        arg[ax] = True
    return st.flip(arg)


def _concatenate_rule(exps, avals, params):
    """Every input cast to the common type, padded with zeros to the final extent, then summed (jit.ts:666-685)."""
    axis = params["axis"]
    ndim = avals[0].ndim
    sizes = [a.shape[axis] for a in avals]
    final = sum(sizes)
    d = ShapedArray((), avals[0].dtype, avals[0].weak)
    for a in avals[1:]:
        d = promoteAvals(d, ShapedArray((), a.dtype, a.weak))
    cum, src = 0, []
    for e, size in zip(exps, sizes):
        padding = [(cum, final - cum - size) if i == axis else (0, 0) for i in range(ndim)]
        src.append(reshapeViews(AluExp.cast(d.dtype, e), lambda st, padding=padding: st.pad(padding)))
        cum += size
    out = src[0]
    for x in src[1:]:
        out = AluExp.add(out, x)
    return [out], None


def _split_rule(exps, avals, params):
    a, aval = exps[0], avals[0]
    out, start = [], 0
    for size in params["sizes"]:
        sl = [(start, start + size) if d == params["axis"] else (0, aval.shape[d]) for d in range(aval.ndim)]
        out.append(reshapeViews(a, lambda st, sl=sl: st.shrink(sl)))
        start += size
    return out, None


def _random_bits_rule(keys, avals, params):
    """threefry2x32(k0, k1, 0, position within the key's block) (jit.ts:698-714)."""
    shape, keyShape = list(params["shape"]), list(avals[0].shape)

    def mapping(st):
        if list(st.shape) != shape:
            return st.broadcast(shape, list(range(len(st.shape), len(shape))))
        return None
    k0, k1 = reshapeViews(keys[0], mapping), reshapeViews(keys[1], mapping)
    c1 = AluExp.mod(AluExp.cast(DType.Uint32, AluVar.gidx), AluExp.u32(max(prod(shape[len(keyShape):]), 1)))
    return [AluExp.threefry2x32(k0, k1, AluExp.u32(0), c1, params.get("mode", "xor"))], None


def _gather_rule(exps, avals, params):
    """The operand's flat index is rebuilt from the output coordinates, with the gathered axes read from the
    (broadcast) index arrays (jit.ts:715-763)."""
    x, indices = exps[0], exps[1:]
    xs, ishapes = avals[0], avals[1:]
    axis, outDim = list(params["axis"]), params["outDim"]
    axisSet = set(axis)
    indexShape: Tuple[int, ...] = ()
    for a in ishapes:
        indexShape = generalBroadcast(indexShape, a.shape)
    finalShape = [d for i, d in enumerate(xs.shape) if i not in axisSet]
    finalShape[outDim:outDim] = list(indexShape)
    idxAll = unravelAlu(finalShape, AluVar.gidx)
    idxNonaxis = list(idxAll)
    del idxNonaxis[outDim:outDim + len(indexShape)]
    src: List[Optional[AluExp]] = list(idxNonaxis)
    for i in range(len(xs.shape)):
        if i in axisSet:
            src.insert(i, None)
    for i, iexp in enumerate(indices):
        def mapping(st):
            lead = list(range(outDim + len(indexShape) - len(st.shape)))
            return st.broadcast(finalShape, lead + list(range(outDim + len(indexShape), len(finalShape))))
        src[axis[i]] = AluExp.cast(DType.Int32, reshapeViews(iexp, mapping))
    index, valid = ShapeTracker.fromShape(list(xs.shape)).toAluExp(src)
    if not valid.resolve():
        raise RuntimeError("internal: expected full validity mask in Gather")
    return [x.substitute({"gidx": index})], None


JIT_RULES: Dict[str, Callable] = {
    "Concatenate": _concatenate_rule,
    "Split": _split_rule,
    "RandomBits": _random_bits_rule,
    "Gather": _gather_rule,
    "Add": _broadcasted(lambda e, p: AluExp.add(e[0], e[1])),
    "Mul": _broadcasted(lambda e, p: AluExp.mul(e[0], e[1])),
    "Idiv": _broadcasted(lambda e, p: AluExp.idiv(e[0], e[1])),
    "Mod": _broadcasted(lambda e, p: AluExp.mod(e[0], e[1])),
    "Min": _broadcasted(lambda e, p: AluExp.min(e[0], e[1])),
    "Max": _broadcasted(lambda e, p: AluExp.max(e[0], e[1])),
    "BitCombine": _broadcasted(lambda e, p: AluExp.bitCombine(e[0], e[1], p["op"])),
    "BitShift": _broadcasted(lambda e, p: AluExp.bitShift(e[0], e[1], p["op"])),
    "Neg": _unop(lambda a, p: AluExp.sub(AluExp.const(a.dtype, 0), a)),
    "Reciprocal": _unop(lambda a, p: AluExp.reciprocal(a)),
    "Floor": _unop(lambda a, p: AluExp.floor(a)),
    "Ceil": _unop(lambda a, p: AluExp.ceil(a)),
    "StopGradient": _unop(lambda a, p: a),
    "Cast": _unop(lambda a, p: AluExp.cast(p["dtype"], a)),
    "Bitcast": _unop(lambda a, p: AluExp.bitcast(p["dtype"], a)),
    "Sin": _unop(lambda a, p: AluExp.sin(a)),
    "Cos": _unop(lambda a, p: AluExp.cos(a)),
    "Asin": _unop(lambda a, p: AluExp.asin(a)),
    "Atan": _unop(lambda a, p: AluExp.atan(a)),
    "Exp": _unop(lambda a, p: AluExp.exp(a)),
    "Log": _unop(lambda a, p: AluExp.log(a)),
    "Erf": _unop(lambda a, p: AluExp.erf(a)),
    "Erfc": _unop(lambda a, p: AluExp.erfc(a)),
    "Sqrt": _unop(lambda a, p: AluExp.sqrt(a)),
    "Reduce": _reduce_rule,
    "Dot": _dot_rule,
    "Conv": _conv_rule,
    "Pool": _reshape_rule(lambda st, p: pool(st, list(p["window"]), list(p["strides"]))),
    "PoolTranspose": _pool_transpose_rule,
    "Compare": _broadcasted(lambda e, p: aluCompare(e[0], e[1], p["op"])),
    "Where": _broadcasted(lambda e, p: AluExp.where(e[0], e[1], e[2]), skipCastIdx=(0,)),
    "Transpose": _reshape_rule(lambda st, p: st.permute(p["perm"])),
    "Broadcast": _reshape_rule(lambda st, p: st.broadcast(list(p["shape"]), list(p["axis"]))),
    "Reshape": _reshape_rule(lambda st, p: st.reshape(list(p["shape"]))),
    "Flip": _reshape_rule(_flip_rule),
    "Shrink": _reshape_rule(lambda st, p: st.shrink([tuple(s) for s in p["slice"]])),
    "Pad": _reshape_rule(lambda st, p: st.pad([tuple(w) for w in p["width"]])),
}


# ---- kernel boundaries (src/frontend/jit.ts:792-1096) ----------------------------------------------

def splitGraphDataflow(jaxpr: Jaxpr, maxArgs: int) -> Set[Var]:
    varToDefn: Dict[Var, int] = {}
    varToUsages: Dict[Var, List[int]] = {}
    for i, eqn in enumerate(jaxpr.eqns):
        for v in eqn.outBinders:
            varToDefn[v] = i
        for x in eqn.inputs:
            if isinstance(x, Var):
                varToUsages.setdefault(x, []).append(i)

    # Reduction epilogues: unary ops, and binary ops against a literal or an array that does not
    # broadcast the reduction's output.
    epilogueEqns: Set[int] = set()
    endpointEqns: Set[int] = set()
    for i, eqn in enumerate(jaxpr.eqns):
        if eqn.primitive not in REDUCE_PRIMITIVES:
            continue
        head = i
        while True:
            epilogueEqns.add(head)
            outVar = jaxpr.eqns[head].outBinders[0]
            usages = varToUsages.get(outVar, [])
            if outVar in jaxpr.outs or len(usages) != 1:
                break
            if usages[0] in epilogueEqns:
                break
            nxt = jaxpr.eqns[usages[0]]
            if nxt.primitive in UNARY_FUSABLE:
                head = usages[0]
                continue
            if nxt.primitive in BINARY_FUSABLE:
                other = next(v for v in nxt.inputs if v is not outVar)
                if isinstance(other, Lit) or generalBroadcast(other.aval.shape, outVar.aval.shape) == tuple(outVar.aval.shape):
                    head = usages[0]
                    continue
            break
        endpointEqns.add(head)

    # A computed value that a Dot would broadcast (and so recompute per output) is materialised first.
    materialized: Set[Var] = set()

    def hasReuse(shape, promoted) -> bool:
        offset = len(promoted) - len(shape)
        for axis in range(len(promoted) - 1):
            dim = 1 if axis < offset else shape[axis - offset]
            if dim == 1 and promoted[axis] > 1:
                return True
        return False

    def markNonViewProducer(v: Var) -> None:
        cur = v
        while True:
            d = varToDefn.get(cur)
            if d is None:
                return
            eqn = jaxpr.eqns[d]
            if eqn.primitive not in VIEW_PRIMITIVES:
                break
            inp = next((x for x in eqn.inputs if isinstance(x, Var)), None)
            if inp is None:
                return
            cur = inp
        materialized.add(cur)

    for eqn in jaxpr.eqns:
        if eqn.primitive == "Dot":
            shapes = [eqn.inputs[0].aval.shape, eqn.inputs[1].aval.shape]
        elif eqn.primitive == "Conv":
            lhs, rhs = prepareConv(ShapeTracker.fromShape(list(eqn.inputs[0].aval.shape)),
                                   ShapeTracker.fromShape(list(eqn.inputs[1].aval.shape)), eqn.params["conv"])
            shapes = [tuple(lhs.shape), tuple(rhs.shape)]
        else:
            continue
        promoted = generalBroadcast(shapes[0], shapes[1])
        for i, x in enumerate(eqn.inputs):
            if isinstance(x, Var) and hasReuse(shapes[i], promoted):
                markNonViewProducer(x)
    for eqn in jaxpr.eqns:
        if eqn.primitive in ("Pad", "Concatenate"):  # padding an expression would pad its inner views: needs clean inputs
            for x in eqn.inputs:
                if isinstance(x, Var):
                    markNonViewProducer(x)

    # A routine reads whole buffers: each operand must be dispatched before it.  The reference marks the operand's
    # non-view producer (src/frontend/jit.ts:990-999) and then refuses an operand that is still a view of it
    # ("routine primitive input is not imm", jit.ts:307-311, e.g. the flips of a lower-triangular solve); here the
    # operand itself is materialised, so such a view is realised by a copy kernel instead of failing.
    # The fused-attention routine addresses its operands through strides, so a plain strided view of a buffer (the
    # q/k/v slices of one QKV projection) is passed as it is: only the view's producer is materialised.
    for eqn in jaxpr.eqns:
        if eqn.primitive in ROUTINE_PRIMITIVES:
            for x in eqn.inputs:
                if isinstance(x, Var) and x in varToDefn:
                    if eqn.primitive in STRIDED_OPERAND_ROUTINES:
                        markNonViewProducer(x)
                    else:
                        materialized.add(x)

    # Backwards: a node is black when it is an output, a reduction endpoint, materialised, or when two
    # different black nodes are reachable from it through non-black nodes.
    black: Set[Var] = set()
    nextBlack: Dict[Var, Var] = {}
    for v in jaxpr.outs:
        if isinstance(v, Var):
            black.add(v)
            nextBlack[v] = v
    for i in range(len(jaxpr.eqns) - 1, -1, -1):
        eqn = jaxpr.eqns[i]
        if (i in endpointEqns or eqn.primitive in ROUTINE_PRIMITIVES or eqn.primitive in HETEROGENEOUS_VIEW_PRIMITIVES
                or any(v in materialized for v in eqn.outBinders)
                or any(v in black for v in eqn.outBinders)):
            for v in eqn.outBinders:
                black.add(v)
                nextBlack[v] = v
            continue
        reach: List[Var] = []
        for v in eqn.outBinders:
            for j in varToUsages.get(v, []):
                for o in jaxpr.eqns[j].outBinders:
                    u = nextBlack.get(o)
                    if u is not None and u not in reach:
                        reach.append(u)
        if len(reach) > 1:
            for v in eqn.outBinders:
                black.add(v)
                nextBlack[v] = v
        elif len(reach) == 1:
            for v in eqn.outBinders:
                nextBlack[v] = reach[0]

    # Forwards: split further wherever a fused expression would read more than maxArgs buffers.
    deps: Dict[Var, Set[Var]] = {v: {v} for v in jaxpr.inBinders}
    idx = 0
    while idx < len(jaxpr.eqns):
        eqn = jaxpr.eqns[idx]
        idx += 1
        per_input: List[Set[Var]] = []
        for x in eqn.inputs:
            if isinstance(x, Var):
                per_input.append({x} if x in black else deps[x])
            else:
                per_input.append(set())
        counter: Dict[Var, int] = {}
        for s in per_input:
            for d in s:
                counter[d] = counter.get(d, 0) + 1
        if len(counter) > maxArgs:
            best, which = 0, -1
            for i, x in enumerate(eqn.inputs):
                if isinstance(x, Var) and x in varToDefn:
                    unique = sum(1 for d in per_input[i] if counter[d] == 1)
                    if unique > best:
                        best, which = unique, i
            if which == -1:
                raise RuntimeError(f"internal: maxArgs, no input found to mark as black in {eqn.primitive}")
            idx = varToDefn[eqn.inputs[which]]
            for out in jaxpr.eqns[idx].outBinders:
                black.add(out)
            idx += 1
        else:
            s = set(counter.keys())
            for out in eqn.outBinders:
                deps[out] = s
    return black


# ---- jitCompile / JitProgram (src/frontend/jit.ts:111-162, 263-469) ----------------------------------

@dataclass
class JitStep:
    kind: str                      # "malloc" | "execute" | "free" | "incref"
    kernel: Optional[Kernel] = None    # an "execute" step runs either a Kernel (one output) ...
    inputs: List[int] = field(default_factory=list)
    output: int = -1
    size: int = 0
    routine: Any = None                # ... or a Routine with `outputs`
    outputs: List[int] = field(default_factory=list)


@dataclass
class JitProgram:
    steps: List[JitStep]
    nargs: int
    outputs: List[int]
    consts: List[ConstArray]

    @property
    def kernels(self) -> List[Kernel]:
        return [s.kernel for s in self.steps if s.kind == "execute" and s.kernel is not None]

    @property
    def routines(self) -> List[Any]:
        return [s.routine for s in self.steps if s.kind == "execute" and s.routine is not None]

    def execute(self, backend, inputs: Sequence[int], prepared: Optional[Dict[int, Any]] = None) -> List[int]:
        """Run on `backend` with input slots (closed-over constants first).  Returns output slots owned
        by the caller; inputs stay owned by the caller."""
        if len(inputs) != self.nargs:
            raise ValueError(f"jit program takes {self.nargs} inputs, got {len(inputs)}")
        scope: Dict[int, int] = {i: s for i, s in enumerate(inputs)}
        for k, step in enumerate(self.steps):
            if step.kind == "malloc":
                scope[step.output] = backend.malloc(step.size)
            elif step.kind == "execute" and step.routine is not None:
                exe = prepared[k] if prepared is not None else backend.prepareRoutineSync(step.routine)
                backend.dispatch(exe, [scope[i] for i in step.inputs], [scope[o] for o in step.outputs])
            elif step.kind == "execute":
                exe = prepared[k] if prepared is not None else backend.prepareKernelSync(step.kernel)
                backend.dispatch(exe, [scope[i] for i in step.inputs], [scope[step.output]])
            elif step.kind == "free":
                backend.decRef(scope.pop(step.output))
            elif step.kind == "incref":
                backend.incRef(scope[step.output])
        return [scope[o] for o in self.outputs]

    def prepare(self, backend) -> Dict[int, Any]:
        return {k: (backend.prepareRoutineSync(s.routine) if s.routine is not None else backend.prepareKernelSync(s.kernel))
                for k, s in enumerate(self.steps) if s.kind == "execute"}


def _plain_strided_view(jv: tuple, aval: ShapedArray):
    """(buffer id, strides, offset, elements addressed) when the pending value `jv` is nothing but one unmasked strided
    view of one buffer, read at the identity index; else None."""
    if jv[0] != "exp" or len(jv[2]) != 1:
        return None
    e = jv[1]
    if e.op != AluOp.GlobalView or e.dtype != aval.dtype:
        return None
    gid, st = e.arg
    if len(st.views) != 1 or list(st.shape) != list(aval.shape):
        return None
    v = st.views[0]
    if v.mask is not None or any(s < 0 for s in v.strides):
        return None
    want = unravelAlu(list(st.shape), AluVar.gidx)
    if len(want) != len(e.src) or any(a.simplify().getHash() != b.simplify().getHash() for a, b in zip(want, e.src)):
        return None
    strides = [0 if d == 1 else int(sd) for d, sd in zip(st.shape, v.strides)]
    elements = int(v.offset) + sum((d - 1) * sd for d, sd in zip(st.shape, strides)) + 1
    return jv[2][gid], strides, int(v.offset), elements


def jitCompile(jaxpr: Jaxpr, consts: Sequence[ConstArray] = (), maxArgs: int = 64) -> JitProgram:
    nargs = len(jaxpr.inBinders)
    black = splitGraphDataflow(jaxpr, maxArgs)
    steps: List[JitStep] = []
    next_id = [nargs]

    # ctx values: ("imm", id) | ("exp", exp, args) | ("red", exp, reduction, args)
    ctx: Dict[Var, tuple] = {v: ("imm", i) for i, v in enumerate(jaxpr.inBinders)}
    for eqn in jaxpr.eqns:
        if eqn.primitive in ROUTINE_PRIMITIVES:  # src/frontend/jit.ts:290-327
            from .alu import byteWidth
            from .routine import Routine, Routines, RoutineType

            rtype = RoutineType([list(x.aval.shape) for x in eqn.inputs], [x.aval.dtype for x in eqn.inputs],
                                [list(v.aval.shape) for v in eqn.outBinders], [v.aval.dtype for v in eqn.outBinders])
            r_inputs: List[int] = []
            r_views: List[Any] = []
            for x in eqn.inputs:
                if not isinstance(x, Var):
                    raise NotImplementedError(f"jit: literal operand of routine {eqn.primitive}")
                jv = ctx[x]
                view = None
                if jv[0] != "imm" and eqn.primitive in STRIDED_OPERAND_ROUTINES:
                    view = _plain_strided_view(jv, x.aval)
                    if view is not None and not STRIDED_OPERAND_ROUTINES[eqn.primitive](view[1], view[2]):
                        view = None
                    if view is None:  # anything else (masked, computed, a reduction): realised by a copy kernel first
                        kernel = Kernel(len(jv[-1]), x.aval.size, jv[1], jv[2] if jv[0] == "red" else None)
                        out_id = next_id[0]
                        next_id[0] += 1
                        steps.append(JitStep("malloc", output=out_id, size=kernel.bytes))
                        steps.append(JitStep("execute", kernel=kernel, inputs=list(jv[-1]), output=out_id))
                        jv = ctx[x] = ("imm", out_id)
                if view is not None:
                    r_inputs.append(view[0])
                    r_views.append(dict(strides=view[1], offset=view[2], elements=view[3]))
                    continue
                if jv[0] != "imm":
                    raise RuntimeError(f"jit: routine primitive {eqn.primitive} input is not imm")
                r_inputs.append(jv[1])
                r_views.append(None)
            r_outputs: List[int] = []
            for v in eqn.outBinders:
                out_id = next_id[0]
                next_id[0] += 1
                steps.append(JitStep("malloc", output=out_id, size=v.aval.size * byteWidth(v.aval.dtype)))
                r_outputs.append(out_id)
                ctx[v] = ("imm", out_id)
            r_params = dict(eqn.params)
            if any(v is not None for v in r_views):
                r_params["views"] = r_views
            steps.append(JitStep("execute", routine=Routine(Routines(eqn.primitive), rtype, r_params or None),
                                 inputs=r_inputs, outputs=r_outputs))
            continue
        rule = JIT_RULES.get(eqn.primitive)
        if rule is None:
            raise NotImplementedError(f"JIT not implemented for primitive {eqn.primitive}")
        inputExps: List[AluExp] = []
        inputAvals: List[ShapedArray] = []
        inputArgs: List[int] = []
        inputReduction = None

        def addArgs(args):
            out = []
            for a in args:
                if a not in inputArgs:
                    inputArgs.append(a)
                out.append(inputArgs.index(a))
            return out

        for x in eqn.inputs:
            if isinstance(x, Var):
                jv = ctx[x]
                if jv[0] == "exp":
                    inputExps.append(jv[1].reindexGids(addArgs(jv[2])))
                elif jv[0] == "imm":
                    (gid,) = addArgs([jv[1]])
                    st = ShapeTracker.fromShape(list(x.aval.shape))
                    inputExps.append(AluExp.globalView(x.aval.dtype, gid, st, unravelAlu(st.shape, AluVar.gidx)))
                else:
                    if inputReduction is not None:
                        raise RuntimeError("jit: unexpected, multiple red inputs")
                    inputExps.append(jv[2].epilogue.reindexGids(addArgs(jv[3])))
                    inputReduction = jv
            else:
                inputExps.append(AluExp.const(x.dtype, x.value))
            inputAvals.append(x.aval)

        if inputReduction is not None:
            (newEpilogue,), _ = rule(inputExps, inputAvals, eqn.params)
            jv = inputReduction
            exps = [jv[1].reindexGids(addArgs(jv[3]))]
            red = jv[2]
            reduction = Reduction(red.dtype, red.op, red.size, newEpilogue)
        else:
            exps, reduction = rule(inputExps, inputAvals, eqn.params)

        for i, outVar in enumerate(eqn.outBinders):
            if outVar in black:
                kernel = Kernel(len(inputArgs), outVar.aval.size, exps[i], reduction)
                out_id = next_id[0]
                next_id[0] += 1
                steps.append(JitStep("malloc", output=out_id, size=kernel.bytes))
                steps.append(JitStep("execute", kernel=kernel, inputs=list(inputArgs), output=out_id))
                ctx[outVar] = ("imm", out_id)
            elif reduction is not None:
                ctx[outVar] = ("red", exps[i], reduction, list(inputArgs))
            else:
                ctx[outVar] = ("exp", exps[i], list(inputArgs))

    outputs: List[int] = []
    for out in jaxpr.outs:
        if isinstance(out, Lit):  # a literal output is realised by a nullary kernel (pushLit, src/frontend/jit.ts:176-183)
            kernel = Kernel(0, out.aval.size, AluExp.const(out.aval.dtype, out.value))
            out_id = next_id[0]
            next_id[0] += 1
            steps.append(JitStep("malloc", output=out_id, size=kernel.bytes))
            steps.append(JitStep("execute", kernel=kernel, inputs=[], output=out_id))
            outputs.append(out_id)
            continue
        jv = ctx[out]
        if jv[0] != "imm":
            raise RuntimeError("internal: Expected imm, since outs are black nodes")
        outputs.append(jv[1])

    # Every returned slot carries a reference of its own: an input returned directly, or an id returned a second
    # time, gets an "incref" step (src/frontend/jit.ts:449-458).
    needs_ref = set(range(nargs))
    for o in outputs:
        if o in needs_ref:
            steps.append(JitStep("incref", output=o))
        else:
            needs_ref.add(o)

    # Free every intermediate after its last use (JitProgramBuilder.insertFreeSteps).
    last_use: Dict[int, int] = {}
    written = lambda s: s.outputs if s.routine is not None else [s.output]  # noqa: E731
    for k, s in enumerate(steps):
        if s.kind == "execute":
            for i in s.inputs:
                last_use[i] = k
            for o in written(s):
                last_use.setdefault(o, k)
    final: List[JitStep] = []
    for k, s in enumerate(steps):
        final.append(s)
        if s.kind == "execute":
            for i in dict.fromkeys(s.inputs + written(s)):
                if i >= nargs and i not in outputs and last_use.get(i) == k:
                    final.append(JitStep("free", output=i))
    return JitProgram(final, nargs, outputs, list(consts))


def jit(fn: Callable[..., Any], avals: Sequence[ShapedArray], maxArgs: int = 64) -> JitProgram:
    """Trace `fn` at the given input avals and compile it to a Kernel program."""
    jaxpr, consts = trace(fn, avals)
    return jitCompile(jaxpr, consts, maxArgs)
