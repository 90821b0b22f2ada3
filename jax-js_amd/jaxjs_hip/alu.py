"""Scalar IR consumed by the `hip` backend: DType, AluOp, AluExp, Kernel, Reduction.

Host-side mirror of the reference's IR module (reference: src/alu.ts).  The
front-end lowers every eager op and every jit-fused group to one `Kernel`:
"evaluate `exp` at gidx in [0,size) and, when `reduction` is present, fold it
over ridx in [0,reduction.size) and apply `reduction.epilogue(acc, gidx)`"
(src/alu.ts:1479-1527, 1544-1661).  The backend only ever sees these objects.

Differences from the reference that are deliberate:

* Nodes are hash-consed: two structurally equal expressions are the same
  Python object, so identity comparison doubles as structural comparison and
  the code generator's common-subexpression elimination is a dict lookup.
* `Kernel.exp_raw` / `Reduction.epilogue_raw` keep the expression exactly as
  the caller built it (before `simplify()`), so that a checker can evaluate the
  un-simplified form independently of the simplifier below.
* Integer constant folding wraps exactly modulo 2**32 (the Wasm backend's
  behaviour, src/backend/wasm/translation.ts:38-70) instead of going through
  IEEE doubles.
"""

from __future__ import annotations

import math
import struct
import weakref
from enum import Enum
from typing import Any, Callable, Dict, Iterable, Iterator, List, Optional, Sequence, Tuple

import numpy as np

INF = math.inf


class DType(str, Enum):
    """Element types (src/alu.ts:6-13).  Bool is stored as int32 0/1."""

    Float32 = "float32"
    Int32 = "int32"
    Uint32 = "uint32"
    Bool = "bool"
    Float16 = "float16"
    Float64 = "float64"

    def __str__(self) -> str:  # matches the reference's string enum
        return self.value


def byteWidth(dtype: DType) -> int:
    """Bytes per stored element (src/alu.ts:23-37); Bool occupies 4 bytes."""
    if dtype in (DType.Float32, DType.Int32, DType.Uint32, DType.Bool):
        return 4
    if dtype == DType.Float16:
        return 2
    if dtype == DType.Float64:
        return 8
    raise TypeError(f"Unknown dtype: {dtype}")


def isFloatDtype(dtype: DType) -> bool:
    return dtype in (DType.Float32, DType.Float16, DType.Float64)


_PROMOTE_RANK = {
    DType.Bool: 0,
    DType.Uint32: 1,
    DType.Int32: 2,
    DType.Float16: 3,
    DType.Float32: 4,
    DType.Float64: 5,
}


def promoteTypes(a: DType, b: DType) -> DType:
    """Join in the lattice bool < uint32 < int32 < f16 < f32 < f64 (src/alu.ts:68-83)."""
    return a if _PROMOTE_RANK[a] >= _PROMOTE_RANK[b] else b


_NUMPY_DTYPE = {
    DType.Float32: np.float32,
    DType.Int32: np.int32,
    DType.Uint32: np.uint32,
    DType.Bool: np.int32,
    DType.Float16: np.float16,
    DType.Float64: np.float64,
}


def numpyDtype(dtype: DType):
    """numpy storage type of a DType (Bool lives in int32, src/alu.ts:95)."""
    return _NUMPY_DTYPE[dtype]


def dtypedArray(dtype: DType, data: bytes | bytearray | memoryview | np.ndarray) -> np.ndarray:
    """View raw bytes as a typed array (src/alu.ts:85-106)."""
    return np.frombuffer(data, dtype=_NUMPY_DTYPE[dtype])


class AluOp(str, Enum):
    """Scalar operations (src/alu.ts:1365-1407)."""

    Add = "Add"
    Sub = "Sub"
    Mul = "Mul"
    Idiv = "Idiv"
    Mod = "Mod"
    Min = "Min"
    Max = "Max"

    Sin = "Sin"
    Cos = "Cos"
    Asin = "Asin"
    Atan = "Atan"
    Exp = "Exp"
    Log = "Log"
    Erf = "Erf"
    Erfc = "Erfc"
    Sqrt = "Sqrt"
    Floor = "Floor"
    Ceil = "Ceil"
    Reciprocal = "Reciprocal"
    Cast = "Cast"
    Bitcast = "Bitcast"

    BitCombine = "BitCombine"  # arg = 'or' | 'and' | 'xor'
    BitInvert = "BitInvert"
    BitShift = "BitShift"  # arg = 'shl' | 'shr'

    Cmplt = "Cmplt"
    Cmpne = "Cmpne"
    Where = "Where"

    Threefry2x32 = "Threefry2x32"  # arg = 'xor' | 0 | 1

    Const = "Const"  # arg = value
    Special = "Special"  # arg = (name, n)
    Variable = "Variable"  # arg = name
    GlobalIndex = "GlobalIndex"  # arg = (gid, len); src = [bufidx]
    GlobalView = "GlobalView"  # arg = (gid, ShapeTracker); src = indices

    def __str__(self) -> str:
        return self.value


class AluGroup:
    """Operation families (src/alu.ts:1409-1459)."""

    Binary = frozenset(
        [AluOp.Add, AluOp.Sub, AluOp.Mul, AluOp.Idiv, AluOp.Mod, AluOp.Min, AluOp.Max, AluOp.BitCombine, AluOp.BitShift]
    )
    Unary = frozenset(
        [
            AluOp.Sin, AluOp.Cos, AluOp.Asin, AluOp.Atan, AluOp.Exp, AluOp.Log, AluOp.Erf, AluOp.Erfc,
            AluOp.Sqrt, AluOp.Floor, AluOp.Ceil, AluOp.Reciprocal, AluOp.Cast, AluOp.Bitcast,
        ]
    )
    Compare = frozenset([AluOp.Cmplt, AluOp.Cmpne])
    Variable = frozenset([AluOp.Special, AluOp.Variable, AluOp.GlobalIndex, AluOp.GlobalView])
    Reduce = frozenset([AluOp.Add, AluOp.Mul, AluOp.Min, AluOp.Max])
    RequiredFloat = frozenset(
        [
            AluOp.Sin, AluOp.Cos, AluOp.Asin, AluOp.Atan, AluOp.Exp, AluOp.Log, AluOp.Erf, AluOp.Erfc,
            AluOp.Sqrt, AluOp.Reciprocal, AluOp.Floor, AluOp.Ceil,
        ]
    )


def _wrap_i32(v: int) -> int:
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v & 0x80000000 else v


def _wrap_u32(v: int) -> int:
    return v & 0xFFFFFFFF


def _trunc_to_int(value: Any) -> int:
    """JS `Math.trunc(x) | 0`-style conversion of a Python number to an integer (NaN/Inf -> 0)."""
    if isinstance(value, (bool, np.bool_)):
        return int(value)
    if isinstance(value, (int, np.integer)):
        return int(value)
    value = float(value)
    if math.isnan(value) or math.isinf(value):
        return 0
    return int(math.trunc(value))


def _clamp(x, lo, hi):
    return max(lo, min(x, hi))


def _gcd(*values: int) -> int:
    a = 0
    for b in values:
        a = math.gcd(a, int(b))
    return abs(a)


def _safe_exp(x: float) -> float:
    try:
        return math.exp(x)
    except OverflowError:
        return INF


def _safe_log(x: float) -> float:
    if math.isnan(x) or x < 0:
        return math.nan
    if x == 0:
        return -INF
    return math.log(x)


def _safe_sqrt(x: float) -> float:
    if math.isnan(x) or x < 0:
        return math.nan
    return math.sqrt(x)


def _erfapprox(x: float) -> float:
    """P(t)*exp(-x^2) of the Abramowitz-Stegun 7.1.26 approximation (src/alu.ts:1766-1777)."""
    p = 0.3275911
    a1, a2, a3, a4, a5 = 0.254829592, -0.284496736, 1.421413741, -1.453152027, 1.061405429
    t = 1.0 / (1.0 + p * x)
    poly = ((((a5 * t + a4) * t + a3) * t + a2) * t + a1) * t
    return poly * _safe_exp(-x * x)


def erf(x: float) -> float:
    """The IR's erf: A&S 7.1.26 with fixed coefficients, not libm (src/alu.ts:1779-1785)."""
    return 1 - _erfapprox(x) if x >= 0 else _erfapprox(-x) - 1


def erfc(x: float) -> float:
    """The IR's erfc (src/alu.ts:1787-1793)."""
    return _erfapprox(x) if x >= 0 else 2 - _erfapprox(-x)


def threefry2x32(k0: int, k1: int, c0: int, c1: int) -> Tuple[int, int]:
    """Threefry-2x32, 20 rounds, as used by the IR's PRNG op (src/alu.ts:1699-1745)."""
    M = 0xFFFFFFFF

    def rotl(x: int, r: int) -> int:
        return ((x << r) | (x >> (32 - r))) & M

    ks = (k0 & M, k1 & M, (k0 ^ k1 ^ 0x1BD11BDA) & M)
    x0 = (c0 + ks[0]) & M
    x1 = (c1 + ks[1]) & M
    rots = ((13, 15, 26, 6), (17, 29, 16, 24))
    for block in range(5):
        for r in rots[block % 2]:
            x0 = (x0 + x1) & M
            x1 = rotl(x1, r) ^ x0
        x0 = (x0 + ks[(block + 1) % 3]) & M
        x1 = (x1 + ks[(block + 2) % 3] + block + 1) & M
    return x0, x1


def _js_min(x, y):
    if isinstance(x, float) or isinstance(y, float):
        if math.isnan(x) or math.isnan(y):
            return math.nan
        if x == y == 0:
            return x if math.copysign(1.0, x) < 0 else y
    return x if x < y else y


def _js_max(x, y):
    if isinstance(x, float) or isinstance(y, float):
        if math.isnan(x) or math.isnan(y):
            return math.nan
        if x == y == 0:
            return x if math.copysign(1.0, x) > 0 else y
    return x if x > y else y


def _arg_key(op: AluOp, arg: Any):
    if op == AluOp.Const:
        if isinstance(arg, float):
            return ("f", struct.pack("<d", arg))
        return ("i", int(arg))
    if op == AluOp.GlobalView:
        return (arg[0], arg[1].key())
    if isinstance(arg, list):
        return tuple(arg)
    return arg


class _BuilderOrBound:
    """Descriptor: on the class a binary node builder, on an instance a range bound."""

    def __init__(self, op: "AluOp", which: int):
        self.op, self.which = op, which

    def __get__(self, obj, cls):
        if obj is None:
            op = self.op
            return lambda a, b: cls(op, a.dtype, (a, b))
        return obj._compute_range()[self.which]


class AluExp:
    """Immutable scalar expression node (src/alu.ts:133-187).  Build through the static helpers."""

    __slots__ = ("op", "dtype", "src", "arg", "_range", "_simplified", "_key", "__weakref__")

    _interned: "weakref.WeakValueDictionary[tuple, AluExp]" = weakref.WeakValueDictionary()

    def __new__(cls, op: AluOp, dtype: DType, src: Sequence["AluExp"] = (), arg: Any = None):
        src = tuple(src)
        if op in AluGroup.RequiredFloat and not isFloatDtype(dtype):
            raise TypeError(f"Unsupported dtype for {op}: {dtype}")
        # Type guards (src/alu.ts:148-186).
        if op == AluOp.Bitcast:
            if dtype == DType.Bool or src[0].dtype == DType.Bool or byteWidth(dtype) != byteWidth(src[0].dtype):
                raise TypeError(f"Bitcast from {src[0].dtype} -> {dtype}")
        elif op == AluOp.Threefry2x32:
            if dtype != DType.Uint32 or any(s.dtype != DType.Uint32 for s in src):
                raise TypeError("Threefry2x32 requires uint32 types")
        elif op == AluOp.BitCombine:
            if src[0].dtype != src[1].dtype or isFloatDtype(src[0].dtype):
                raise TypeError(
                    f"BitCombine[{arg}] requires matching integral dtype, got {src[0].dtype} and {src[1].dtype}"
                )
        elif op == AluOp.BitShift:
            if (
                src[0].dtype == DType.Bool
                or src[1].dtype == DType.Bool
                or isFloatDtype(src[0].dtype)
                or isFloatDtype(src[1].dtype)
            ):
                raise TypeError(
                    f"BitShift[{arg}] requires two integral, non-bool dtypes, got {src[0].dtype} and {src[1].dtype}"
                )
        elif op == AluOp.BitInvert:
            if isFloatDtype(src[0].dtype):
                raise TypeError(f"BitInvert requires an integral dtype, got {src[0].dtype}")
        if isinstance(arg, list):
            arg = tuple(arg)
        key = (op, dtype, tuple(id(s) for s in src), _arg_key(op, arg))
        hit = cls._interned.get(key)
        if hit is not None:
            return hit
        self = object.__new__(cls)
        self.op = op
        self.dtype = dtype
        self.src = src
        self.arg = arg
        self._range = None
        self._simplified = None
        self._key = key
        cls._interned[key] = self
        return self

    # -- builders (src/alu.ts:189-335) -------------------------------------------------------
    @staticmethod
    def add(a: "AluExp", b: "AluExp") -> "AluExp":
        return AluExp(AluOp.Add, a.dtype, (a, b))

    @staticmethod
    def sub(a, b):
        return AluExp(AluOp.Sub, a.dtype, (a, b))

    @staticmethod
    def mul(a, b):
        return AluExp(AluOp.Mul, a.dtype, (a, b))

    @staticmethod
    def idiv(a, b):
        return AluExp(AluOp.Idiv, a.dtype, (a, b))

    @staticmethod
    def mod(a, b):
        return AluExp(AluOp.Mod, a.dtype, (a, b))

    @staticmethod
    def sin(a):
        return AluExp(AluOp.Sin, a.dtype, (a,))

    @staticmethod
    def cos(a):
        return AluExp(AluOp.Cos, a.dtype, (a,))

    @staticmethod
    def asin(a):
        return AluExp(AluOp.Asin, a.dtype, (a,))

    @staticmethod
    def atan(a):
        return AluExp(AluOp.Atan, a.dtype, (a,))

    @staticmethod
    def exp(a):
        return AluExp(AluOp.Exp, a.dtype, (a,))

    @staticmethod
    def log(a):
        return AluExp(AluOp.Log, a.dtype, (a,))

    @staticmethod
    def erf(a):
        return AluExp(AluOp.Erf, a.dtype, (a,))

    @staticmethod
    def erfc(a):
        return AluExp(AluOp.Erfc, a.dtype, (a,))

    @staticmethod
    def sqrt(a):
        return AluExp(AluOp.Sqrt, a.dtype, (a,))

    @staticmethod
    def floor(a):
        return AluExp(AluOp.Floor, a.dtype, (a,)) if isFloatDtype(a.dtype) else a

    @staticmethod
    def ceil(a):
        return AluExp(AluOp.Ceil, a.dtype, (a,)) if isFloatDtype(a.dtype) else a

    @staticmethod
    def reciprocal(a):
        return AluExp(AluOp.Reciprocal, a.dtype, (a,))

    @staticmethod
    def cast(dtype: DType, a: "AluExp") -> "AluExp":
        return a if a.dtype == dtype else AluExp(AluOp.Cast, dtype, (a,))

    @staticmethod
    def bitcast(dtype: DType, a: "AluExp") -> "AluExp":
        return a if a.dtype == dtype else AluExp(AluOp.Bitcast, dtype, (a,))

    @staticmethod
    def threefry2x32(k0, k1, c0, c1, mode: Any = "xor"):
        return AluExp(AluOp.Threefry2x32, DType.Uint32, (k0, k1, c0, c1), mode)

    @staticmethod
    def bitCombine(a, b, mode: str):
        return AluExp(AluOp.BitCombine, a.dtype, (a, b), mode)

    @staticmethod
    def bitShift(a, b, mode: str):
        return AluExp(AluOp.BitShift, a.dtype, (a, b), mode)

    @staticmethod
    def cmplt(a, b):
        return AluExp(AluOp.Cmplt, DType.Bool, (a, b))

    @staticmethod
    def cmpne(a, b):
        return AluExp(AluOp.Cmpne, DType.Bool, (a, b))

    @staticmethod
    def where(cond, a, b):
        return AluExp(AluOp.Where, a.dtype, (cond, a, b))

    @staticmethod
    def const(dtype: DType, value: Any) -> "AluExp":
        """Literal; integers are normalised the way the reference does (src/alu.ts:280-294)."""
        if dtype == DType.Bool:
            value = int(bool(value))
        elif dtype == DType.Int32:
            value = _wrap_i32(_trunc_to_int(value))
        elif dtype == DType.Uint32:
            value = _wrap_u32(_trunc_to_int(value))
        else:
            if not isinstance(value, (int, float, np.floating, np.integer)) or isinstance(value, bool):
                raise TypeError(f"Expected a number for constant, got {type(value).__name__}: {value}")
            value = float(value)
        return AluExp(AluOp.Const, dtype, (), value)

    @staticmethod
    def special(dtype: DType, name: str, n: int) -> "AluExp":
        return AluExp(AluOp.Special, dtype, (), (name, int(n)))

    @staticmethod
    def variable(dtype: DType, name: str) -> "AluExp":
        return AluExp(AluOp.Variable, dtype, (), name)

    @staticmethod
    def globalIndex(dtype: DType, gid: int, length: int, bufidx: "AluExp") -> "AluExp":
        return AluExp(AluOp.GlobalIndex, dtype, (bufidx,), (int(gid), int(length)))

    @staticmethod
    def globalView(dtype: DType, gid: int, st, indices: Sequence["AluExp"]) -> "AluExp":
        return AluExp(AluOp.GlobalView, dtype, tuple(indices), (int(gid), st))

    @staticmethod
    def f32(v):
        return AluExp.const(DType.Float32, v)

    @staticmethod
    def i32(v):
        return AluExp.const(DType.Int32, v)

    @staticmethod
    def u32(v):
        return AluExp.const(DType.Uint32, v)

    @staticmethod
    def bool(v):
        return AluExp.const(DType.Bool, int(bool(v)))

    @staticmethod
    def f16(v):
        return AluExp.const(DType.Float16, v)

    @staticmethod
    def f64(v):
        return AluExp.const(DType.Float64, v)

    def not_(self) -> "AluExp":
        """Logical negation of a bool expression (`not()` in src/alu.ts:337-342)."""
        if self.dtype != DType.Bool:
            raise TypeError("not() can only be called on boolean expressions")
        return AluExp.cmpne(self, AluExp.const(DType.Bool, True))

    # -- identity ---------------------------------------------------------------------------
    def getHash(self) -> int:
        """Structural identity; equal structure <=> same object because nodes are interned."""
        return id(self)

    def __repr__(self) -> str:
        return self.toString()

    # -- traversal helpers (src/alu.ts:1291-1361) ---------------------------------------------
    def fold(self, reducer: Callable[["AluExp", list], Any]) -> Any:
        """Bottom-up fold over the DAG, visiting each distinct node once."""
        visited: Dict[int, Any] = {}
        stack: List[Tuple[AluExp, bool]] = [(self, False)]
        while stack:
            node, expanded = stack.pop()
            if id(node) in visited:
                continue
            if expanded:
                visited[id(node)] = reducer(node, [visited[id(s)] for s in node.src])
            else:
                stack.append((node, True))
                for s in node.src:
                    if id(s) not in visited:
                        stack.append((s, False))
        return visited[id(self)]

    def some(self, predicate: Callable[["AluExp"], bool]) -> bool:
        seen = set()
        stack = [self]
        while stack:
            node = stack.pop()
            if id(node) in seen:
                continue
            if predicate(node):
                return True
            seen.add(id(node))
            stack.extend(node.src)
        return False

    def rewrite(self, visitor: Callable[["AluExp"], Optional["AluExp"]]) -> "AluExp":
        def step(node: AluExp, new_src: list) -> AluExp:
            if all(a is b for a, b in zip(new_src, node.src)):
                cand = node
            else:
                cand = AluExp(node.op, node.dtype, new_src, node.arg)
            out = visitor(cand)
            return cand if out is None else out

        return self.fold(step)

    def collect(self, predicate: Callable[["AluExp"], bool]) -> List["AluExp"]:
        out: List[AluExp] = []

        def step(node, _):
            if predicate(node):
                out.append(node)

        self.fold(step)
        return out

    def distinctOps(self) -> Dict[AluOp, set]:
        ops: Dict[AluOp, set] = {}

        def step(node, _):
            ops.setdefault(node.op, set()).add(node.dtype)

        self.fold(step)
        return ops

    def substitute(self, variables: Dict[str, "AluExp"]) -> "AluExp":
        """Replace `Variable` nodes by name (src/alu.ts:369-380)."""

        def visit(node: AluExp):
            if node.op == AluOp.Variable and node.arg in variables:
                repl = variables[node.arg]
                if repl.dtype != node.dtype:
                    raise TypeError(f"Type mismatch: {node.dtype} vs {repl.dtype}")
                return repl
            return None

        return self.rewrite(visit)

    def reindexGids(self, newGids: Sequence[int]) -> "AluExp":
        """Renumber buffer arguments (src/alu.ts:383-399)."""

        def visit(node: AluExp):
            if node.op == AluOp.GlobalIndex:
                gid, length = node.arg
                if newGids[gid] != gid:
                    return AluExp.globalIndex(node.dtype, newGids[gid], length, node.src[0])
            elif node.op == AluOp.GlobalView:
                gid = node.arg[0]
                if newGids[gid] != gid:
                    return AluExp.globalView(node.dtype, newGids[gid], node.arg[1], node.src)
            return None

        return self.rewrite(visit)

    def rewriteGlobalViews(self) -> "AluExp":
        """Lower every GlobalView to index arithmetic + GlobalIndex (src/alu.ts:1354-1361)."""

        def visit(node: AluExp):
            if node.op == AluOp.GlobalView:
                gid, st = node.arg
                return accessorGlobal(node.dtype, gid, st, node.src)
            return None

        return self.rewrite(visit)

    def _pureNonNegativeIndex(self) -> bool:
        """Index arithmetic only (symbols, non-negative constants, +, *, % and / by positive constants): non-negative in
        exact arithmetic by structure.  Nothing that reads a buffer qualifies."""
        if self.dtype != DType.Int32:
            return False
        if self.op in (AluOp.Special, AluOp.Variable):
            return True
        if self.op == AluOp.Const:
            return int(self.arg) >= 0
        if self.op in (AluOp.Add, AluOp.Mul):
            return self.src[0]._pureNonNegativeIndex() and self.src[1]._pureNonNegativeIndex()
        if self.op in (AluOp.Mod, AluOp.Idiv):
            return self.src[1].op == AluOp.Const and int(self.src[1].arg) > 0 and self.src[0]._pureNonNegativeIndex()
        return False

    def reduceExactIndex(self) -> "AluExp":
        """`(sum of index terms) % D` and `/ D` with every term's constant multiplier reduced modulo D, in exact arithmetic.

        The index expression of a chain of views unravels a flat index into conceptual arrays whose extents can pass
        2^31 (output channels x batch x padded image: `(o * 349748352 + ... + x * 59) % 58` for the operands of a
        layer-sized filter cotangent).  The reference's simplifier removes such terms because its range analysis never
        wraps (src/alu.ts:425-571 with the rule "(x + A*y) % B => x % B when B | A"), so the kernels its backends compile
        never evaluate them; the range analysis here gives up where a bound leaves 32 bits, so the same reduction is
        done explicitly, and only on pure index arithmetic (symbols and constants: values read from buffers keep their
        wrap-around semantics)."""

        def visit(n: AluExp):
            if n.op not in (AluOp.Mod, AluOp.Idiv) or n.dtype != DType.Int32 or n.src[1].op != AluOp.Const:
                return None
            D = int(n.src[1].arg)
            if D <= 1 or not n.src[0]._pureNonNegativeIndex():
                return None
            terms = list(n.src[0].splitOp(AluOp.Add))
            if len(terms) < 2:
                return None
            rest, quot, changed = [], [], False
            for t in terms:
                f = t.constFactor()
                q = t.divides(f) if f > 1 else None
                if q is None or f < D:
                    rest.append(t)
                    continue
                changed = True
                if f // D:
                    quot.append(q if f // D == 1 else AluExp.mul(q, AluExp.i32(f // D)))
                if f % D:
                    rest.append(q if f % D == 1 else AluExp.mul(q, AluExp.i32(f % D)))
            if not changed:
                return None

            def total(parts):
                acc = parts[0]
                for x in parts[1:]:
                    acc = AluExp.add(acc, x)
                return acc

            low = total(rest) if rest else AluExp.i32(0)
            if n.op == AluOp.Mod:
                return AluExp.mod(low, n.src[1])
            return total(quot + [AluExp.idiv(low, n.src[1])]) if quot else AluExp.idiv(low, n.src[1])

        return self.rewrite(visit)

    def splitOp(self, sep: AluOp) -> Iterator["AluExp"]:
        """Flatten nested applications of an associative op (src/alu.ts:630-636)."""
        if self.op == sep:
            for s in self.src:
                yield from s.splitOp(sep)
        else:
            yield self

    # -- range analysis (src/alu.ts:401-581) --------------------------------------------------
    def _compute_range(self) -> Tuple[float, float]:
        if self._range is not None:
            return self._range
        src = self.src
        op = self.op
        unbounded = (-INF, INF)

        def corners(f):
            a, b = src[0]._compute_range(), src[1]._compute_range()
            vals = []
            for x in a:
                for y in b:
                    try:
                        vals.append(f(x, y))
                    except (ZeroDivisionError, OverflowError, ValueError):
                        vals.append(math.nan)
            if any(isinstance(v, float) and math.isnan(v) for v in vals):
                return (math.nan, math.nan)
            return (min(vals), max(vals))

        def js_div_trunc(a, b):
            if b == 0:
                if a == 0 or (isinstance(a, float) and math.isnan(a)):
                    return math.nan
                return INF if (a > 0) == (math.copysign(1.0, b) > 0) else -INF
            q = a / b
            if math.isinf(q) or math.isnan(q):
                return q
            return math.trunc(q)

        def js_mul(a, b):
            if (a == 0 and math.isinf(b)) or (b == 0 and math.isinf(a)):
                return math.nan
            return a * b

        try:
            if op == AluOp.Add:
                ret = (src[0].min + src[1].min, src[0].max + src[1].max)
            elif op == AluOp.Sub:
                ret = (src[0].min - src[1].max, src[0].max - src[1].min)
            elif op == AluOp.Mul:
                ret = corners(js_mul)
            elif op == AluOp.Idiv:
                ret = corners(js_div_trunc)
            elif op == AluOp.Mod:
                # C-style remainder: sign follows the dividend (src/alu.ts:432-458).
                lo, hi = src[1]._compute_range()
                if lo <= 0 <= hi:
                    lo, hi = 0, max(-lo, hi)
                if hi < 0:
                    lo, hi = -hi, -lo
                max_div = hi if isFloatDtype(self.dtype) else hi - 1
                ret = (_clamp(src[0].min, -max_div, 0), _clamp(src[0].max, 0, max_div))
            elif op == AluOp.Min:
                ret = (min(src[0].min, src[1].min), min(src[0].max, src[1].max))
            elif op == AluOp.Max:
                ret = (max(src[0].min, src[1].min), max(src[0].max, src[1].max))
            elif op in (AluOp.Sin, AluOp.Cos):
                ret = (-1, 1)
            elif op in (AluOp.Asin, AluOp.Atan):
                ret = (-math.pi / 2, math.pi / 2)
            elif op == AluOp.Exp:
                ret = (_safe_exp(src[0].min), _safe_exp(src[0].max))
            elif op == AluOp.Log:
                ret = (_safe_log(src[0].min), _safe_log(src[0].max))
            elif op == AluOp.Erf:
                ret = (erf(src[0].min), erf(src[0].max))
            elif op == AluOp.Erfc:
                ret = (erfc(src[0].max), erfc(src[0].min))
            elif op == AluOp.Sqrt:
                ret = (_safe_sqrt(src[0].min), _safe_sqrt(src[0].max))
            elif op == AluOp.Floor:
                ret = tuple(v if math.isinf(v) else math.floor(v) for v in (src[0].min, src[0].max))
            elif op == AluOp.Ceil:
                ret = tuple(v if math.isinf(v) else math.ceil(v) for v in (src[0].min, src[0].max))
            elif op == AluOp.Reciprocal:
                if src[0].min <= 0 <= src[0].max:
                    ret = unbounded
                else:
                    ret = (1 / src[0].max, 1 / src[0].min)
            elif op == AluOp.Cast:
                lo, hi = src[0].min, src[0].max
                was_float = isFloatDtype(src[0].dtype)
                bounded = math.isfinite(lo) and math.isfinite(hi)
                if self.dtype == DType.Bool:
                    can_zero = lo <= 0 <= hi
                    must_zero = lo == 0 and hi == 0
                    ret = (0, 0) if must_zero else ((0, 1) if can_zero else (1, 1))
                elif self.dtype == DType.Int32:
                    if not bounded:
                        ret = unbounded
                    else:
                        a = _wrap_i32(_trunc_to_int(_clamp(lo, -2147483648, 2147483647) if was_float else lo))
                        b = _wrap_i32(_trunc_to_int(_clamp(hi, -2147483648, 2147483647) if was_float else hi))
                        ret = (a, b) if a <= b else unbounded
                elif self.dtype == DType.Uint32:
                    if not bounded:
                        ret = (0, INF)
                    else:
                        a = _wrap_u32(_trunc_to_int(_clamp(lo, 0, 4294967295) if was_float else lo))
                        b = _wrap_u32(_trunc_to_int(_clamp(hi, 0, 4294967295) if was_float else hi))
                        ret = (a, b) if a <= b else (0, INF)
                else:
                    ret = (lo, hi)
            elif op in (AluOp.Cmplt, AluOp.Cmpne):
                ret = (0, 1)
            elif op == AluOp.Where:
                ret = (min(src[1].min, src[2].min), max(src[1].max, src[2].max))
            elif op == AluOp.Const:
                ret = (self.arg, self.arg)
            elif op == AluOp.Special:
                ret = (0, self.arg[1] - 1)
            else:
                ret = unbounded
        except (OverflowError, ValueError, ZeroDivisionError):
            ret = unbounded
        lo, hi = ret
        if (isinstance(lo, float) and math.isnan(lo)) or (isinstance(hi, float) and math.isnan(hi)):
            lo, hi = unbounded
        if self.dtype == DType.Bool:
            lo, hi = _clamp(lo, 0, 1), _clamp(hi, 0, 1)
        # Integer arithmetic is exact modulo 2^32: a bound outside the type's range means the value may have
        # wrapped, so nothing is known.  (The reference only clamps the lower bound of uint32 to 0,
        # src/alu.ts:570-572, which folds `0 - x` on uint32 to the constant 0; that is not followed here.)
        if self.dtype == DType.Uint32:
            if op in (AluOp.Add, AluOp.Sub, AluOp.Mul, AluOp.Idiv, AluOp.Mod) and (lo < 0 or hi > 4294967295):
                lo, hi = 0, INF
            lo = max(0, lo)
        if self.dtype == DType.Int32 and op in (AluOp.Add, AluOp.Sub, AluOp.Mul):
            if lo < -2147483648 or hi > 2147483647:
                lo, hi = -INF, INF
        self._range = (lo, hi)
        return self._range

    # `AluExp.min(a, b)` builds a Min node while `exp.min` is the lower bound of exp's range, as
    # in the reference where the static builder and the accessor share a name.
    min = _BuilderOrBound(AluOp.Min, 0)  # noqa: A003
    max = _BuilderOrBound(AluOp.Max, 1)  # noqa: A003

    # -- divisibility helpers (src/alu.ts:583-623) -------------------------------------------
    def constFactor(self) -> int:
        """Largest known integer dividing this expression."""
        if self.op == AluOp.Const:
            return abs(int(self.arg)) if float(self.arg).is_integer() else 1
        if self.op == AluOp.Add:
            return _gcd(self.src[0].constFactor(), self.src[1].constFactor())
        if self.op == AluOp.Mul:
            for s in self.src:
                if s._isConstInt():
                    return abs(int(s.arg))
        return 1

    def divides(self, v: int) -> Optional["AluExp"]:
        """Quotient by an integer if provably exact, else None."""
        if v == 1:
            return self
        if self.op == AluOp.Const and self._isConstInt() and self.arg % v == 0:
            return AluExp.const(self.dtype, self.arg // v)
        if self.op == AluOp.Add:
            a = self.src[0].divides(v)
            if a is not None:
                b = self.src[1].divides(v)
                if b is not None:
                    return AluExp.add(a, b)
        if self.op == AluOp.Mul:
            a = self.src[0].divides(v)
            if a is not None:
                return AluExp.mul(a, self.src[1])
            b = self.src[1].divides(v)
            if b is not None:
                return AluExp.mul(self.src[0], b)
        return None

    def _isConstInt(self) -> bool:
        return self.op == AluOp.Const and self.dtype in (DType.Int32, DType.Uint32)

    # -- simplification ------------------------------------------------------------------------
    def simplify(self, cache: Optional[dict] = None) -> "AluExp":
        """Algebraic clean-up of index arithmetic; see `_simplify_node` for the rule list."""
        if self._simplified is not None:
            return self._simplified
        # Iterative post-order to stay clear of Python's recursion limit on deep chains.
        stack: List[AluExp] = [self]
        while stack:
            node = stack[-1]
            if node._simplified is not None:
                stack.pop()
                continue
            pending = [s for s in node.src if s._simplified is None]
            if pending:
                stack.extend(pending)
                continue
            stack.pop()
            out = _simplify_node(node)
            if out._simplified is None:
                out._simplified = out
            node._simplified = out._simplified
        return self._simplified

    def resolve(self) -> Any:
        """Constant value if the expression folds to one, else None (src/alu.ts:1045-1049)."""
        x = self.simplify()
        return x.arg if x.op == AluOp.Const else None

    # -- evaluation ---------------------------------------------------------------------------
    def evaluate(self, context: Dict[str, Any], globals_: Optional[Callable[[int, int], Any]] = None):
        """Scalar interpreter used for constant folding and tiny host-side checks.

        Follows `AluExp.evaluate` (src/alu.ts:1059-1213): floats are Python doubles, Bool is
        0/1.  Integer arithmetic wraps modulo 2**32.
        """
        memo: Dict[int, Any] = {}

        def ev(node: AluExp):
            k = id(node)
            if k in memo:
                return memo[k]
            r = _eval_node(node, ev, context, globals_)
            memo[k] = r
            return r

        return ev(self)

    # -- printing (src/alu.ts:1216-1288) --------------------------------------------------------
    def toString(self) -> str:
        BIN = {AluOp.Add: "+", AluOp.Sub: "-", AluOp.Mul: "*", AluOp.Idiv: "/", AluOp.Mod: "%"}
        CMP = {AluOp.Cmplt: "<", AluOp.Cmpne: "!="}

        def strip1(s: str) -> str:
            return s[1:-1] if s.startswith("(") and s.endswith(")") and _balanced(s[1:-1]) else s

        def step(node: AluExp, parts: list) -> str:
            op = node.op
            if op == AluOp.Const:
                return str(bool(node.arg)).lower() if node.dtype == DType.Bool else repr(node.arg)
            if op == AluOp.Variable:
                return f"${node.arg}:{node.dtype}"
            if op == AluOp.Special:
                return f"#{node.arg[0]}{{{node.arg[1]}}}"
            if op == AluOp.GlobalIndex:
                return f"G_{node.arg[0]}<{node.dtype}>[{strip1(parts[0])}]"
            if op == AluOp.GlobalView:
                gid, st = node.arg
                shape = ",".join(map(str, st.shape))
                strides = ",".join(map(str, st.lastStrides))
                cont = "c" if st.contiguous else "nc"
                return f"GV_{gid}<{node.dtype}>{{{shape}:{strides}:{cont}}}[{', '.join(map(strip1, parts))}]"
            if op in BIN:
                return f"({parts[0]} {BIN[op]} {parts[1]})"
            if op in CMP:
                return f"({parts[0]} {CMP[op]} {parts[1]})"
            if op == AluOp.BitCombine:
                sym = {"and": "&", "or": "|", "xor": "^"}[node.arg]
                return f"({parts[0]} {sym} {parts[1]})"
            if op == AluOp.BitShift:
                return f"({parts[0]} {'<<' if node.arg == 'shl' else '>>'} {parts[1]})"
            if op == AluOp.Reciprocal:
                return f"1/{parts[0]}"
            if op == AluOp.Cast:
                return f"Cast<{node.dtype}>({strip1(parts[0])})"
            if op == AluOp.Bitcast:
                return f"Bitcast<{node.dtype}>({strip1(parts[0])})"
            return f"{op}({', '.join(map(strip1, parts))})"

        return self.fold(step)


def _balanced(s: str) -> bool:
    depth = 0
    for ch in s:
        if ch == "(":
            depth += 1
        elif ch == ")":
            depth -= 1
            if depth < 0:
                return False
    return depth == 0


# ---------------------------------------------------------------------------------------------
# Scalar evaluation of one node
# ---------------------------------------------------------------------------------------------


def _bits_of(value, dtype: DType) -> bytes:
    return np.array([value], dtype=_NUMPY_DTYPE[dtype]).tobytes()


def _eval_node(node: AluExp, ev, context, globals_):
    op, dtype, src = node.op, node.dtype, node.src
    is_int = dtype in (DType.Int32, DType.Uint32)
    wrap = _wrap_i32 if dtype == DType.Int32 else _wrap_u32

    if op in AluGroup.Binary or op in AluGroup.Compare:
        x, y = ev(src[0]), ev(src[1])
        if op == AluOp.Add:
            if dtype == DType.Bool:
                return int(bool(x) or bool(y))
            return wrap(x + y) if is_int else _fadd(x, y)
        if op == AluOp.Sub:
            return wrap(x - y) if is_int else _fadd(x, -y)
        if op == AluOp.Mul:
            if dtype == DType.Bool:
                return int(bool(x) and bool(y))
            return wrap(x * y) if is_int else _fmul(x, y)
        if op == AluOp.Idiv:
            if is_int or dtype == DType.Bool:
                if y == 0:
                    return 0
                q = abs(x) // abs(y)
                return wrap(q if (x < 0) == (y < 0) else -q)
            q = _fdiv(x, y)
            return q if (math.isnan(q) or math.isinf(q)) else float(math.trunc(q))
        if op == AluOp.Mod:
            if is_int or dtype == DType.Bool:
                if y == 0:
                    return 0
                r = abs(x) % abs(y)
                return wrap(-r if x < 0 else r)
            if math.isnan(x) or math.isnan(y) or math.isinf(x) or y == 0:
                return math.nan
            if math.isinf(y):
                return x
            return math.fmod(x, y)
        if op == AluOp.Min:
            return _js_min(x, y)
        if op == AluOp.Max:
            return _js_max(x, y)
        if op == AluOp.BitCombine:
            xi, yi = int(x) & 0xFFFFFFFF, int(y) & 0xFFFFFFFF
            r = xi & yi if node.arg == "and" else (xi | yi if node.arg == "or" else xi ^ yi)
            if dtype == DType.Bool:
                return r & 1
            return _wrap_i32(r) if dtype == DType.Int32 else r
        if op == AluOp.BitShift:
            xi, sh = int(x) & 0xFFFFFFFF, int(y) & 31
            r = (xi << sh) & 0xFFFFFFFF if node.arg == "shl" else xi >> sh
            # Right shifts are logical for int32 as well (src/alu.ts:1088-1091): the JS `>>>`
            # result is non-negative and only wraps when stored.
            return _wrap_i32(r) if dtype == DType.Int32 else r
        if op == AluOp.Cmplt:
            return int(x < y)
        if op == AluOp.Cmpne:
            return int(x != y)
        raise NotImplementedError(op)

    if op in AluGroup.Unary:
        x = ev(src[0])
        if op == AluOp.Sin:
            return math.sin(x) if math.isfinite(x) else math.nan
        if op == AluOp.Cos:
            return math.cos(x) if math.isfinite(x) else math.nan
        if op == AluOp.Asin:
            return math.asin(x) if -1 <= x <= 1 else math.nan
        if op == AluOp.Atan:
            return math.atan(x)
        if op == AluOp.Exp:
            return x if math.isnan(x) else _safe_exp(x)
        if op == AluOp.Log:
            return _safe_log(x)
        if op == AluOp.Erf:
            return erf(x)
        if op == AluOp.Erfc:
            return erfc(x)
        if op == AluOp.Sqrt:
            return _safe_sqrt(x)
        if op == AluOp.Floor:
            return x if not math.isfinite(x) else float(math.floor(x))
        if op == AluOp.Ceil:
            return x if not math.isfinite(x) else float(math.ceil(x))
        if op == AluOp.Reciprocal:
            return _fdiv(1.0, x)
        if op == AluOp.Cast:
            was_float = isFloatDtype(src[0].dtype)
            if dtype == DType.Int32:
                if was_float:
                    return 0 if math.isnan(x) else int(_clamp(math.trunc(x) if math.isfinite(x) else x, -2147483648, 2147483647))
                return _wrap_i32(int(x))
            if dtype == DType.Uint32:
                if was_float:
                    return 0 if math.isnan(x) else int(_clamp(math.trunc(x) if math.isfinite(x) else x, 0, 4294967295))
                return _wrap_u32(int(x))
            if isFloatDtype(dtype):
                return float(x)
            if dtype == DType.Bool:
                return int(x != 0)
            raise NotImplementedError(f"Unsupported cast to {dtype}")
        if op == AluOp.Bitcast:
            raw = _bits_of(x, src[0].dtype)
            v = np.frombuffer(raw, dtype=_NUMPY_DTYPE[dtype])[0]
            return float(v) if isFloatDtype(dtype) else int(v)
        raise NotImplementedError(op)

    if op == AluOp.Where:
        return ev(src[1]) if ev(src[0]) else ev(src[2])
    if op == AluOp.Threefry2x32:
        k0, k1, c0, c1 = (int(ev(s)) for s in src)
        x0, x1 = threefry2x32(k0, k1, c0, c1)
        if node.arg == "xor":
            return x0 ^ x1
        if node.arg == 0:
            return x0
        if node.arg == 1:
            return x1
        raise ValueError(f"Invalid Threefry2x32 mode: {node.arg}")
    if op == AluOp.Const:
        return node.arg
    if op == AluOp.Special:
        if node.arg[0] not in context:
            raise KeyError(f"Missing special: {node.arg[0]}")
        return context[node.arg[0]]
    if op == AluOp.Variable:
        if node.arg not in context:
            raise KeyError(f"Missing variable: {node.arg}")
        return context[node.arg]
    if op == AluOp.GlobalIndex:
        if globals_ is None:
            raise ValueError("Missing globals function")
        return globals_(node.arg[0], ev(src[0]))
    if op == AluOp.GlobalView:
        if globals_ is None:
            raise ValueError("Missing globals function")
        gid, st = node.arg
        iexpr, vexpr = st.toAluExp(list(src))
        if vexpr.evaluate(context, globals_):
            return globals_(gid, iexpr.evaluate(context, globals_))
        return 0
    raise NotImplementedError(op)


def _fadd(x, y):
    try:
        return x + y
    except OverflowError:
        return math.nan


def _fmul(x, y):
    try:
        return x * y
    except OverflowError:
        return math.nan


def _fdiv(x, y):
    x, y = float(x), float(y)
    if y == 0:
        if x == 0 or math.isnan(x):
            return math.nan
        return INF if (x > 0) == (math.copysign(1.0, y) > 0) else -INF
    try:
        return x / y
    except OverflowError:
        return INF if (x > 0) == (y > 0) else -INF


# ---------------------------------------------------------------------------------------------
# Simplifier
# ---------------------------------------------------------------------------------------------

_COMMUTATIVE = (AluOp.Add, AluOp.Mul, AluOp.Max, AluOp.Min)


def _S(e: AluExp) -> AluExp:
    return e.simplify()


def _is_const(e: AluExp, value=None) -> bool:
    return e.op == AluOp.Const and (value is None or e.arg == value)


def _simplify_node(node: AluExp) -> AluExp:
    """One simplification step on a node whose sources are already simplified.

    Rule set (same algebra the reference applies in src/alu.ts:667-1042, which in turn follows
    tinygrad's symbolic rewrites): constant folding, empty-range folding, neutral elements,
    `x + (-1*y)`, `where(c,1,0)`, provably-true/false compares, selects on a known condition,
    mod/div collapses driven by value ranges (`x % C`, nested mods, `(x/A)*A + x%A`,
    `(x*A + y)/B`, `(x + A*y) % B`), const-to-the-right canonicalisation, division of a sum by
    the gcd of its terms, and the split of `sum % C` / `sum / C` into quotient and remainder
    parts.  Sources are simplified before this is called.
    """
    op, dtype = node.op, node.dtype
    src = tuple(s._simplified if s._simplified is not None else s.simplify() for s in node.src)
    C = lambda v: AluExp.const(dtype, v)  # noqa: E731

    # Constant folding.
    if src and all(s.op == AluOp.Const for s in src) and op not in AluGroup.Variable and op != AluOp.BitInvert:
        try:
            return AluExp.const(dtype, AluExp(op, dtype, src, node.arg).evaluate({}))
        except (NotImplementedError, OverflowError, ValueError):
            pass

    cur = node if all(a is b for a, b in zip(src, node.src)) else AluExp(op, dtype, src, node.arg)

    # A non-constant whose range is a single point is that constant.
    if op != AluOp.Const:
        lo, hi = cur.min, cur.max
        if lo == hi and not (isinstance(lo, float) and math.isinf(lo)):
            return AluExp.const(dtype, lo)

    if op in AluGroup.Binary or op in AluGroup.Compare:
        for i in (0, 1):
            if src[i].op != AluOp.Const:
                continue
            x, other = src[i].arg, src[1 - i]
            if op == AluOp.Add and x == 0:
                return other
            if op == AluOp.Sub and i == 1 and x == 0:
                return other
            if op == AluOp.Mul and x == 1:
                return other
            if op == AluOp.Mul and x == 0 and not isFloatDtype(dtype):
                return C(0)
            if op == AluOp.Mul and x == 0 and isFloatDtype(dtype) and math.isfinite(other.min) and math.isfinite(other.max):
                return C(0)
            if op == AluOp.Idiv and i == 1 and x == 1 and not isFloatDtype(dtype):
                return other
            if op == AluOp.Cmpne and src[i].dtype == DType.Bool and x == 0:
                return other

    # x + (-1*y) => x - y ;  x - (-1*y) => x + y
    if op in (AluOp.Add, AluOp.Sub) and src[1].op == AluOp.Mul:
        a, b = src[1].src
        neg = AluOp.Sub if op == AluOp.Add else AluOp.Add
        if _is_const(a, -1):
            return _S(AluExp(neg, dtype, (src[0], b)))
        if _is_const(b, -1):
            return _S(AluExp(neg, dtype, (src[0], a)))

    if op == AluOp.Where:
        if _is_const(src[1], 1) and _is_const(src[2], 0):
            return _S(AluExp.cast(dtype, src[0]))
        if src[0].max == 0:
            return src[2]
        if src[0].min == 1:
            return src[1]

    if op == AluOp.Cmplt:
        if src[0].min >= src[1].max:
            return AluExp.const(DType.Bool, False)
        if src[0].max < src[1].min:
            return AluExp.const(DType.Bool, True)
    if op == AluOp.Cmpne:
        if src[0].max < src[1].min or src[0].min > src[1].max:
            return AluExp.const(DType.Bool, True)

    if op == AluOp.Mod and src[1]._isConstInt():
        x, B = src[0], src[1].arg
        # x % C => x when 0 <= x < C
        if x.min >= 0 and x.max < B:
            return x
        # (x % A) % B => x % min(A,B) when one divides the other
        if x.op == AluOp.Mod and x.src[1]._isConstInt():
            A = x.src[1].arg
            if A > 0 and B > 0 and (A % B == 0 or B % A == 0):
                return _S(AluExp.mod(x.src[0], C(min(A, B))))

    # (x/A)*A + x%A => x ;  ((x/A)%B)*A + x%A => x % (A*B)
    if (
        op == AluOp.Add
        and src[0].op == AluOp.Mul
        and src[0].src[1]._isConstInt()
        and src[1].op == AluOp.Mod
        and src[1].src[1]._isConstInt()
        and src[0].src[1].arg == src[1].src[1].arg
    ):
        mul, mod = src
        A = mod.src[1].arg

        def is_quot(e: AluExp) -> bool:
            return e.op == AluOp.Idiv and e.src[1]._isConstInt() and e.src[1].arg == A and e.src[0] is mod.src[0]

        if is_quot(mul.src[0]):
            return mod.src[0]
        if mul.src[0].op == AluOp.Mod and is_quot(mul.src[0].src[0]):
            return _S(AluExp.mod(mod.src[0], AluExp.mul(mod.src[1], mul.src[0].src[1])))

    if op == AluOp.Idiv and src[1]._isConstInt() and src[1].arg != 0:
        numer, B = src[0], src[1].arg
        for i in (0, 1):
            # (x*A)/B => x*(A/B)
            if numer.op == AluOp.Mul and numer.src[i]._isConstInt():
                A = numer.src[i].arg
                if A % B == 0:
                    ret = numer.src[1 - i]
                    if A // B != 1:
                        ret = AluExp.mul(ret, AluExp.const(ret.dtype, A // B))
                    return _S(ret)
            # (x*A + y)/B => x*(A/B) + y/B
            if numer.op == AluOp.Add:
                for j in (0, 1):
                    t = numer.src[j]
                    if t.op == AluOp.Mul and t.src[i]._isConstInt():
                        A = t.src[i].arg
                        if A % B != 0:
                            continue
                        ret = t.src[1 - i]
                        if A // B != 1:
                            ret = AluExp.mul(ret, AluExp.const(ret.dtype, A // B))
                        y = numer.src[1 - j]
                        y_over = y.divides(B)
                        if y_over is not None:
                            return _S(AluExp.add(ret, y_over))
                        ret_s = _S(ret)
                        # trunc(q + y/B) == q + trunc(y/B) only when both point the same way.
                        if B > 0 and ((ret_s.min >= 0 and y.min >= 0) or (ret_s.max <= 0 and y.max <= 0)):
                            return _S(AluExp.add(ret, AluExp.idiv(y, AluExp.const(ret.dtype, B))))

    if op == AluOp.Mod and src[1]._isConstInt() and src[1].arg > 0 and src[0].min >= 0:
        numer, denom = src
        B = denom.arg
        for i in (0, 1):
            if numer.op == AluOp.Add:
                t, x = numer.src[i], numer.src[1 - i]
                # (x + A) % B => x % B when B | A and x >= 0
                if t._isConstInt() and t.arg % B == 0 and x.min >= 0:
                    return _S(AluExp.mod(x, denom))
                # (x + A*y) % B => x % B when B | A and x >= 0
                if t.op == AluOp.Mul:
                    for j in (0, 1):
                        if t.src[j]._isConstInt() and t.src[j].arg % B == 0 and x.min >= 0:
                            return _S(AluExp.mod(x, denom))
            elif numer.op == AluOp.Mul and numer.src[i]._isConstInt():
                A = numer.src[i].arg
                if A % B == 0:
                    return C(0)
                if A % B == 1:
                    return _S(AluExp.mod(numer.src[1 - i], denom))

    # Move constants outward and to the right so later rules see a canonical form.
    if op in _COMMUTATIVE and dtype != DType.Bool:
        P = lambda a, b: AluExp(op, dtype, (a, b))  # noqa: E731
        if src[0].op == AluOp.Const and src[1].op != AluOp.Const:
            return _S(P(src[1], src[0]))
        # Reassociation of floating-point sums/products changes rounding, so only integers
        # (where the arithmetic is exact modulo 2**32) and min/max are regrouped.
        if not isFloatDtype(dtype) or op in (AluOp.Max, AluOp.Min):
            if src[0].op == op and src[0].src[1].op == AluOp.Const:
                if src[1].op == AluOp.Const:
                    return _S(P(src[0].src[0], P(src[0].src[1], src[1])))
                return _S(P(P(src[0].src[0], src[1]), src[0].src[1]))
            if src[1].op == op and src[1].src[1].op == AluOp.Const:
                return _S(P(P(src[0], src[1].src[0]), src[1].src[1]))

    if op in (AluOp.Mod, AluOp.Idiv) and src[1]._isConstInt() and src[1].arg != 0 and not isFloatDtype(dtype):
        x, y = src
        # Divide numerator terms and denominator by their common gcd.
        factors, terms = [], []
        for u in x.splitOp(AluOp.Add):
            f = u.constFactor()
            q = u.divides(f) if f != 0 else None
            if q is None:
                f, q = 1, u
            factors.append(f)
            terms.append(q)
        g = _gcd(y.arg, *factors)
        if g > 1:
            parts = [AluExp.mul(AluExp.const(t.dtype, f // g), t) for f, t in zip(factors, terms)]
            total = parts[-1]
            for p in reversed(parts[:-1]):
                total = AluExp.add(p, total)
            ret = AluExp(op, dtype, (total, AluExp.const(y.dtype, y.arg // g)))
            if op == AluOp.Mod:
                ret = AluExp.mul(ret, C(g))
            return _S(ret)

        # Split a non-negative sum into the part that is a multiple of y and the rest.
        if y.arg > 0 and x.min >= 0:
            x_nc, cval = x, 0
            if x.op == AluOp.Add and x.src[1]._isConstInt():
                x_nc, cval = x.src[0], x.src[1].arg
            terms, factors = [], []
            for u in x_nc.splitOp(AluOp.Add):
                f = u.constFactor()
                d = u.divides(f) if f != 0 else None
                terms.append(d if d is not None else u)
                factors.append(f if d is not None else 1)
            Y = y.arg
            quot = [f // Y for f in factors]
            rems = [f % Y for f in factors]
            gv = Y
            for r in rems:
                gv = _gcd(gv, r)
            if (
                (cval % Y != cval)
                or gv != 1
                or any(r == 0 or (r != f and op == AluOp.Mod) for r, f in zip(rems, factors))
            ):
                quo = AluExp.const(x.dtype, cval // Y)
                rem = AluExp.const(x.dtype, (cval % Y) // gv)
                for t, f, q, r in zip(terms, factors, quot, rems):
                    if op == AluOp.Idiv and r != 0:
                        rem = AluExp.add(rem, AluExp.mul(AluExp.const(x.dtype, f // gv), t))
                    else:
                        rem = AluExp.add(rem, AluExp.mul(AluExp.const(x.dtype, r // gv), t))
                        quo = AluExp.add(quo, AluExp.mul(AluExp.const(x.dtype, q), t))
                if rem.min >= 0:
                    if op == AluOp.Mod:
                        return _S(
                            AluExp.add(
                                AluExp.mul(AluExp.const(x.dtype, gv), AluExp.mod(rem, AluExp.const(x.dtype, Y // gv))),
                                AluExp.const(x.dtype, cval % gv),
                            )
                        )
                    return _S(AluExp.add(AluExp.idiv(rem, AluExp.const(x.dtype, Y // gv)), quo))

    return cur


# ---------------------------------------------------------------------------------------------
# Variables, Kernel, Reduction
# ---------------------------------------------------------------------------------------------


class _AluVar:
    """Well-known variables (src/alu.ts:1462-1470)."""

    gidx = AluExp.variable(DType.Int32, "gidx")
    ridx = AluExp.variable(DType.Int32, "ridx")
    idx = AluExp.variable(DType.Int32, "idx")
    unroll = AluExp.variable(DType.Int32, "unroll")
    upcast = AluExp.variable(DType.Int32, "upcast")

    @staticmethod
    def acc(dtype: DType) -> AluExp:
        return AluExp.variable(dtype, "acc")


AluVar = _AluVar


class Reduction:
    """Fold over one axis with an optional fused epilogue (src/alu.ts:1544-1661)."""

    def __init__(self, dtype: DType, op: AluOp, size: int, epilogue: Optional[AluExp] = None):
        if op not in AluGroup.Reduce:
            raise TypeError(f"Unsupported reduction: {op}")
        if epilogue is None:
            epilogue = AluVar.acc(dtype)
        self.op = op
        self.size = int(size)
        raw = epilogue
        epilogue = epilogue.simplify()
        # Low-precision float sums accumulate in float32 (src/alu.ts:1560-1568).
        if dtype == DType.Float16 and op == AluOp.Add:
            sub = {"acc": AluExp.cast(dtype, AluVar.acc(DType.Float32))}
            epilogue = epilogue.substitute(sub)
            raw = raw.substitute(sub)
            dtype = DType.Float32
        self.dtype = dtype
        self.epilogue = epilogue
        self.epilogue_raw = raw

    def key(self):
        return (self.dtype, self.op, self.size, id(self.epilogue))

    def __repr__(self) -> str:
        return f"{self.op}{{{self.size}}} -> {self.epilogue}"

    @property
    def identity(self):
        """Neutral element per dtype/op (src/alu.ts:1584-1604)."""
        d, op = self.dtype, self.op
        if d == DType.Bool:
            return 0 if op in (AluOp.Add, AluOp.Max) else 1
        if d == DType.Int32:
            return {AluOp.Add: 0, AluOp.Mul: 1, AluOp.Min: 0x7FFFFFFF, AluOp.Max: -(1 << 31)}[op]
        if d == DType.Uint32:
            return {AluOp.Add: 0, AluOp.Mul: 1, AluOp.Min: 0xFFFFFFFF, AluOp.Max: 0}[op]
        if isFloatDtype(d):
            return {AluOp.Add: 0.0, AluOp.Mul: 1.0, AluOp.Min: INF, AluOp.Max: -INF}[op]
        raise TypeError(f"Unsupported reduction: {op} {d}")

    def evaluate(self, *values):
        """Fold values on the host (src/alu.ts:1607-1660)."""
        d, op = self.dtype, self.op
        acc = self.identity
        for v in values:
            if d == DType.Bool:
                acc = int(bool(acc) or bool(v)) if op in (AluOp.Add, AluOp.Max) else int(bool(acc) and bool(v))
            elif op == AluOp.Add:
                acc = acc + v
            elif op == AluOp.Mul:
                acc = acc * v
            elif op == AluOp.Min:
                acc = _js_min(acc, v)
            else:
                acc = _js_max(acc, v)
            if d == DType.Int32:
                acc = _wrap_i32(acc)
            elif d == DType.Uint32:
                acc = _wrap_u32(acc)
        return acc


class Kernel:
    """One fused elementwise map with an optional reduce axis (src/alu.ts:1479-1527)."""

    def __init__(self, nargs: int, size: int, exp: AluExp, reduction: Optional[Reduction] = None):
        self.nargs = int(nargs)
        self.size = int(size)
        self.exp_raw = exp
        self.exp = exp.simplify()
        self.reduction = reduction

    @property
    def dtype(self) -> DType:
        return self.reduction.epilogue.dtype if self.reduction else self.exp.dtype

    @property
    def bytes(self) -> int:
        return self.size * byteWidth(self.dtype)

    def key(self):
        """Cache key: structural identity of the kernel (plays the role of FpHash.hash(kernel))."""
        return (self.nargs, self.size, id(self.exp), self.reduction.key() if self.reduction else None)

    def __repr__(self) -> str:
        s = f"{{ exp = {self.exp}\n  size = {self.size}"
        if self.reduction:
            s += f"\n  reduction = {self.reduction}"
        return s + " }"


def accessorGlobal(dtype: DType, gid: int, st, indices: Sequence[AluExp]) -> AluExp:
    """`where(valid, load(buffer gid at st[indices]), 0)` (src/alu.ts:1664-1679)."""
    index, valid = st.toAluExp(list(indices))
    _, length = st.views[0].dataRange()
    if valid.resolve():
        return AluExp.globalIndex(dtype, gid, length, index)
    return AluExp.where(valid, AluExp.globalIndex(dtype, gid, length, index), AluExp.const(dtype, 0))


def accessorAluExp(exp: AluExp, st, indices: Sequence[AluExp]) -> AluExp:
    """Index a virtual array given by an expression in `idx` (src/alu.ts:1682-1695)."""
    index, valid = st.toAluExp(list(indices))
    if valid.resolve():
        return exp.substitute({"idx": index})
    return AluExp.where(valid, exp.substitute({"idx": index}), AluExp.const(exp.dtype, 0))
