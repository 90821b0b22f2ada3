"""AluExp -> HIP C++ expression text for gfx950 kernels.

Plays the role the WGSL expression generator plays for the reference's WebGPU backend
(src/backend/webgpu/codegen.ts:148-319): linearise a fused scalar DAG into statements, giving every
node referenced more than once a temporary.  The emitted text only uses the helpers of
`csrc/templates/prelude.hip.inc`; op semantics are listed there.
"""

from __future__ import annotations

import math
import struct
from typing import Callable, Dict, List, Optional

import numpy as np

from .alu import AluExp, AluGroup, AluOp, DType, isFloatDtype
from .errors import UnsupportedOpError

# A generated source may open with lines of this form; `runtime.compile_source` adds the named option (from a fixed
# list) to the compiler's command line for that source alone.
SOURCE_OPTION = "// hiprtc-option: "
SOURCE_OPTIONS_ALLOWED = ("-fno-slp-vectorize",)

CTYPE = {
    DType.Float32: "float",
    DType.Int32: "int",
    DType.Uint32: "jh_u32",
    DType.Bool: "bool",
    DType.Float16: "jh_f16",
    DType.Float64: "double",
}
# Element type of a buffer holding the dtype (Bool is stored as int32 0/1, src/alu.ts:95).
STORAGE_CTYPE = dict(CTYPE)
STORAGE_CTYPE[DType.Bool] = "int"

_INT32_MIN, _INT32_MAX = -(1 << 31), (1 << 31) - 1


def const_literal(dtype: DType, value) -> str:
    """C++ literal with exactly the value the reference's backends materialise for a Const."""
    if dtype == DType.Bool:
        return "true" if value else "false"
    if dtype == DType.Int32:
        v = int(value)
        return "(-2147483647 - 1)" if v == _INT32_MIN else str(v)
    if dtype == DType.Uint32:
        return f"{int(value)}u"
    v = float(value)
    if dtype == DType.Float64:
        if math.isnan(v):
            return "__builtin_nan(\"\")"
        if math.isinf(v):
            return "__builtin_inf()" if v > 0 else "(-__builtin_inf())"
        return v.hex()
    # f32 / f16: round once to the storage precision, then print exactly.
    with np.errstate(over="ignore"):
        r = float(np.float32(v)) if dtype == DType.Float32 else float(np.float16(v))
    if math.isnan(r):
        lit = "jh_nan_f32()"
    elif math.isinf(r):
        lit = "jh_inf_f32()" if r > 0 else "(-jh_inf_f32())"
    else:
        lit = r.hex() + "f"
    return lit if dtype == DType.Float32 else f"(jh_f16)({lit})"


def _fits_i32(e: AluExp) -> bool:
    lo, hi = e.min, e.max
    return lo >= _INT32_MIN and hi <= _INT32_MAX


class HipExpCodegen:
    """Emit statements for expressions into `lines`; `run(exp)` returns the text of its value.

    `names` maps Special/Variable names to C identifiers.  `loads` optionally overrides how a
    particular GlobalIndex node is read (used for lanes of a vector load).  `args[gid]` is the
    pointer variable of buffer gid.  With `numerics == "wasm"` f64 transcendentals go through the
    f32 routines as the reference's Wasm backend does (src/backend/wasm/translation.ts:113-122).
    """

    def __init__(self, args: List[str], names: Dict[str, str], indent: str = "  ", prefix: str = "alu",
                 numerics: str = "wasm"):
        self.args = args
        self.names = dict(names)
        self.indent = indent
        self.prefix = prefix
        self.numerics = numerics
        self.lines: List[str] = []
        self.loads: Dict[int, str] = {}
        self._refs: Dict[int, int] = {}
        self._seen: set = set()
        self._ctx: Dict[int, str] = {}
        self._n = 0

    # -- bookkeeping ------------------------------------------------------------------------------
    def countReferences(self, exp: AluExp) -> None:
        stack = [exp]
        while stack:
            node = stack.pop()
            self._refs[id(node)] = self._refs.get(id(node), 0) + 1
            if id(node) not in self._seen:
                self._seen.add(id(node))
                stack.extend(node.src)

    def reset(self) -> None:
        self._refs.clear()
        self._seen.clear()
        self._ctx.clear()

    def gensym(self) -> str:
        self._n += 1
        return f"{self.prefix}{self._n - 1}"

    def emit(self, line: str) -> None:
        self.lines.append(self.indent + line)

    def take_lines(self) -> List[str]:
        out, self.lines = self.lines, []
        return out

    # -- expression generation --------------------------------------------------------------------
    def run(self, exp: AluExp) -> str:
        order: List[AluExp] = []
        seen = set()
        stack = [(exp, False)]
        while stack:
            node, done = stack.pop()
            if id(node) in self._ctx or (id(node) in seen and not done):
                continue
            if done:
                order.append(node)
                continue
            seen.add(id(node))
            stack.append((node, True))
            if node.op == AluOp.GlobalIndex and id(node) in self.loads:
                continue  # index arithmetic of an overridden load is not needed
            for s in node.src:
                if id(s) not in self._ctx and id(s) not in seen:
                    stack.append((s, False))
        for node in order:
            if id(node) not in self._ctx:
                self._gen(node)
        return self._ctx[id(exp)]

    def _gen(self, node: AluExp) -> None:
        text, inline = self._render(node)
        if not inline and self._refs.get(id(node), 0) > 1:
            name = self.gensym()
            self.emit(f"const {CTYPE[node.dtype]} {name} = {text};")
            text = name
        self._ctx[id(node)] = text

    def _unsupported(self, node: AluExp, arg=None):
        return UnsupportedOpError(node.op, node.dtype, "hip", arg)

    def _render(self, node: AluExp):
        op, dtype, src, arg = node.op, node.dtype, node.src, node.arg
        S = [self._ctx[id(s)] for s in src] if not (op == AluOp.GlobalIndex and id(node) in self.loads) else []
        ct = CTYPE[dtype]
        isf = isFloatDtype(dtype)

        if op in AluGroup.Binary or op in AluGroup.Compare:
            a, b = S
            if op in (AluOp.Add, AluOp.Sub, AluOp.Mul):
                if dtype == DType.Bool:
                    if op == AluOp.Add:
                        return f"({a} || {b})", False
                    if op == AluOp.Mul:
                        return f"({a} && {b})", False
                    return f"({a} != {b})", False
                sym = {AluOp.Add: "+", AluOp.Sub: "-", AluOp.Mul: "*"}[op]
                if dtype == DType.Int32 and not _fits_i32(node):
                    fn = {AluOp.Add: "jh_add_i32", AluOp.Sub: "jh_sub_i32", AluOp.Mul: "jh_mul_i32"}[op]
                    return f"{fn}({a}, {b})", False
                if dtype == DType.Float16:
                    return f"(jh_f16)({a} {sym} {b})", False
                return f"({a} {sym} {b})", False
            if op in (AluOp.Idiv, AluOp.Mod):
                if isf:
                    return f"{'jh_fidiv' if op == AluOp.Idiv else 'jh_fmod'}({a}, {b})", False
                if dtype == DType.Bool:
                    raise self._unsupported(node)
                safe = src[1].op == AluOp.Const and src[1].arg not in (0, -1)
                if safe:
                    return f"({a} {'/' if op == AluOp.Idiv else '%'} {b})", False
                suffix = "i32" if dtype == DType.Int32 else "u32"
                return f"jh_{'idiv' if op == AluOp.Idiv else 'mod'}_{suffix}({a}, {b})", False
            if op in (AluOp.Min, AluOp.Max):
                lo = op == AluOp.Min
                if dtype == DType.Bool:
                    return f"({a} {'&&' if lo else '||'} {b})", False
                if isf:
                    return f"jh_{'fmin' if lo else 'fmax'}<{ct}>({a}, {b})", False
                suffix = "i32" if dtype == DType.Int32 else "u32"
                return f"jh_{'min' if lo else 'max'}_{suffix}({a}, {b})", False
            if op == AluOp.BitCombine:
                if dtype == DType.Bool:
                    return {"and": f"({a} && {b})", "or": f"({a} || {b})", "xor": f"({a} != {b})"}[arg], False
                sym = {"and": "&", "or": "|", "xor": "^"}[arg]
                return f"({a} {sym} {b})", False
            if op == AluOp.BitShift:
                suffix = "i32" if dtype == DType.Int32 else "u32"
                cast_b = f"(int)({b})" if dtype == DType.Int32 else f"(jh_u32)({b})"
                return f"jh_{arg}_{suffix}({a}, {cast_b})", False
            if op == AluOp.Cmplt:
                if src[0].dtype == DType.Bool:
                    return f"(!{a} && {b})", False
                return f"({a} < {b})", False
            if op == AluOp.Cmpne:
                return f"({a} != {b})", False

        if op in AluGroup.Unary:
            a = S[0]
            sdt = src[0].dtype
            fns = {AluOp.Sin: "sin", AluOp.Cos: "cos", AluOp.Asin: "asin", AluOp.Atan: "atan", AluOp.Exp: "exp",
                   AluOp.Log: "log", AluOp.Erf: "erf", AluOp.Erfc: "erfc"}
            if op in fns:
                call = f"jh_{fns[op]}_f32((float)({a}))" if dtype != DType.Float32 else f"jh_{fns[op]}_f32({a})"
                if dtype == DType.Float16 and op in (AluOp.Exp, AluOp.Log):
                    call = f"jh_{fns[op]}_f16((float)({a}))"  # hardware exp2/log2: float16 has no Wasm polynomial to follow
                if dtype == DType.Float64 and self.numerics == "native" and op not in (AluOp.Erf, AluOp.Erfc):
                    return f"__ocml_{fns[op]}_f64({a})", False
                return (call if dtype == DType.Float32 else f"({ct})({call})"), False
            if op == AluOp.Sqrt:
                if dtype == DType.Float64:
                    return f"__builtin_sqrt({a})", False
                if dtype == DType.Float16:
                    return f"(jh_f16)__builtin_sqrtf((float)({a}))", False
                return f"__builtin_sqrtf({a})", False
            if op in (AluOp.Floor, AluOp.Ceil):
                nm = "floor" if op == AluOp.Floor else "ceil"
                if dtype == DType.Float64:
                    return f"__builtin_{nm}({a})", False
                if dtype == DType.Float16:
                    return f"(jh_f16)__builtin_{nm}f((float)({a}))", False
                return f"__builtin_{nm}f({a})", False
            if op == AluOp.Reciprocal:
                if dtype == DType.Float32:
                    return f"jh_rcp_f32({a})", False  # IEEE division, or v_rcp_f32 under the fast numerics
                one = {DType.Float64: "1.0", DType.Float16: "(jh_f16)1.0f"}[dtype]
                return f"({ct})({one} / {a})", False
            if op == AluOp.Cast:
                if dtype == sdt:
                    return a, True
                if dtype == DType.Bool:
                    return f"({a} != 0)", False
                if isf:
                    # f16*f16 feeding a wider accumulator is multiplied exactly in the wider type
                    # (what an MFMA does), so every kernel class agrees on the product.
                    s0 = src[0]
                    if (s0.op == AluOp.Mul and s0.dtype == DType.Float16 and dtype in (DType.Float32, DType.Float64)
                            and self._refs.get(id(s0), 0) <= 1):
                        x, y = (self._ctx[id(t)] for t in s0.src)
                        return f"(({ct})({x}) * ({ct})({y}))", False
                    return f"({ct})({a})", False
                if isFloatDtype(sdt):
                    return f"{'jh_f2i_sat' if dtype == DType.Int32 else 'jh_f2u_sat'}({a})", False
                return f"({ct})({a})", False
            if op == AluOp.Bitcast:
                if dtype == sdt:
                    return a, True
                return f"__builtin_bit_cast({ct}, {a})", False

        if op == AluOp.Where:
            return f"({S[0]} ? {S[1]} : {S[2]})", False
        if op == AluOp.Threefry2x32:
            tmp = self.gensym()
            self.emit(f"const jh_u32x2 {tmp} = jh_threefry2x32({S[0]}, {S[1]}, {S[2]}, {S[3]});")
            if arg == "xor":
                return f"({tmp}.x ^ {tmp}.y)", False
            if arg == 0:
                return f"{tmp}.x", True
            if arg == 1:
                return f"{tmp}.y", True
            raise self._unsupported(node, arg)
        if op == AluOp.Const:
            return const_literal(dtype, arg), True
        if op == AluOp.Special:
            name = arg[0]
            if name not in self.names:
                raise KeyError(f"unbound special {name}")
            return self.names[name], True
        if op == AluOp.Variable:
            if arg not in self.names:
                raise KeyError(f"unbound variable {arg}")
            return self.names[arg], True
        if op == AluOp.GlobalIndex:
            if id(node) in self.loads:
                text = self.loads[id(node)]
            else:
                gid, length = arg
                idx = S[0]
                if length <= 0:
                    return const_literal(dtype, 0), True
                text = f"{self.args[gid]}[{idx}]"
                if not (src[0].min >= 0 and src[0].max < length):
                    # A load whose index may leave the buffer sits under a mask (padding, a window's edge); the clamp makes
                    # it safe anywhere.  A float16 one gets a statement of its own ahead of the select: left inside the
                    # select's arm it is compiled as a branch around the load with a wait behind it, one load in flight
                    # (grouped 3x3 convolution [8,64,56,56], 72 taps unrolled: 83 -> 53 us).  float32 loads the compiler
                    # hoists by itself, and schedules better than when told to (35 us against 46).
                    text = f"{self.args[gid]}[jh_guard_index({idx}, {length})]"
                    if dtype == DType.Float16:
                        tmp = self.gensym()
                        self.emit(f"const auto {tmp} = {text};")
                        text = tmp
            if dtype == DType.Bool:
                text = f"({text} != 0)"
            return text, False
        if op == AluOp.GlobalView:
            raise ValueError("GlobalView must be lowered before code generation")
        raise self._unsupported(node, arg)


def strip_parens(text: str) -> str:
    if text.startswith("(") and text.endswith(")"):
        depth = 0
        for i, ch in enumerate(text):
            if ch == "(":
                depth += 1
            elif ch == ")":
                depth -= 1
                if depth == 0 and i != len(text) - 1:
                    return text
        return text[1:-1]
    return text
