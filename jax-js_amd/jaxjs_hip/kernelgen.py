"""Splice a tuned Kernel into the hand-written HIP templates of `csrc/templates/`.

The counterpart of `pipelineSource` in the reference's WebGPU backend (src/backend/webgpu.ts:285-530):
take the tuner's result, declare the buffer arguments, generate the fused expression body (and the
reduction epilogue) and return complete source text plus the launch geometry.  One function per
kernel class; the text of the classes themselves lives in the `.hip.inc` files.
"""

from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .alu import AluExp, AluOp, AluVar, DType, Kernel, Reduction, byteWidth
from .codegen import CTYPE, SOURCE_OPTION, STORAGE_CTYPE, HipExpCodegen, const_literal, strip_parens
from .errors import UnsupportedOpError
from .shape import prod
from .tuner import TuneResult, tuneHip

_TEMPLATE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc", "templates")
_templates: Dict[str, str] = {}


def template(name: str) -> str:
    if name not in _templates:
        with open(os.path.join(_TEMPLATE_DIR, name), "r") as f:
            _templates[name] = f.read()
    return _templates[name]


def fill(text: str, subs: Dict[str, object]) -> str:
    for k, v in subs.items():
        text = text.replace(f"@@{k}@@", str(v))
    if "@@" in text:
        start = text.index("@@")
        raise KeyError(f"unfilled template field near: {text[start:start + 40]!r}")
    return text


@dataclass
class LaunchStep:
    """One kernel launch of a prepared executable."""

    name: str
    grid: Tuple[int, int, int]
    block: Tuple[int, int, int]
    shared: int
    # ("in", gid) | ("out", 0) | ("scratch", index)
    args: List[Tuple[str, int]]
    module: int = 0  # index into KernelSource.sources


@dataclass
class KernelSource:
    sources: List[str]
    steps: List[LaunchStep]
    scratch_bytes: List[int] = field(default_factory=list)
    klass: str = ""
    # Minimum byte size each input slot must have (from the lengths the index analysis assumed).
    min_input_bytes: Dict[int, int] = field(default_factory=dict)
    info: Dict[str, object] = field(default_factory=dict)
    # Scratch buffers (indices) that must hold zeros before the executable's first launch; the kernels leave them zeroed.
    zeroed_scratch: List[int] = field(default_factory=list)


def _used_args(nargs: int, *exps: Optional[AluExp]) -> List[Optional[DType]]:
    used: List[Optional[DType]] = [None] * nargs
    for e in exps:
        if e is None:
            continue
        for n in e.collect(lambda x: x.op == AluOp.GlobalIndex):
            used[n.arg[0]] = n.dtype
    return used


def _min_bytes(*exps: Optional[AluExp]) -> Dict[int, int]:
    need: Dict[int, int] = {}
    for e in exps:
        if e is None:
            continue
        for n in e.collect(lambda x: x.op == AluOp.GlobalIndex):
            gid, length = n.arg
            need[gid] = max(need.get(gid, 0), length * byteWidth(n.dtype))
    return need


def _params(used: List[Optional[DType]], out_t: str, out_name: str = "out") -> Tuple[str, List[str]]:
    names = [f"in{i}" for i in range(len(used))]
    parts = [f"const {STORAGE_CTYPE[d or DType.Float32]}* __restrict__ {n}" for d, n in zip(used, names)]
    parts.append(f"{out_t}* __restrict__ {out_name}")
    return ", ".join(parts), names


def _in_params(used: List[Optional[DType]]) -> Tuple[str, str]:
    """The input pointers as a parameter list and as the matching argument list (for a generated loader function)."""
    names = [f"in{i}" for i in range(len(used))]
    return ("".join(f"const {STORAGE_CTYPE[d or DType.Float32]}* __restrict__ {n}, " for d, n in zip(used, names)),
            "".join(f"{n}, " for n in names))


def _reduce_text(op: AluOp, dtype: DType) -> str:
    ct = CTYPE[dtype]
    if dtype == DType.Bool:
        return "(a) || (b)" if op in (AluOp.Add, AluOp.Max) else "(a) && (b)"
    if op in (AluOp.Add, AluOp.Mul):
        sym = "+" if op == AluOp.Add else "*"
        if dtype == DType.Int32:
            return f"jh_{'add' if op == AluOp.Add else 'mul'}_i32((a), (b))"
        if dtype == DType.Float16:
            return f"(jh_f16)((a) {sym} (b))"
        return f"(a) {sym} (b)"
    lo = op == AluOp.Min
    if dtype in (DType.Float32, DType.Float16, DType.Float64):
        return f"jh_{'fmin' if lo else 'fmax'}<{ct}>((a), (b))"
    return f"jh_{'min' if lo else 'max'}_{'i32' if dtype == DType.Int32 else 'u32'}((a), (b))"


class _Body:
    """Generates the three renderings of one expression a template needs: the hoisted vector /
    uniform loads at lane 0, the per-lane body that consumes them, and a plain scalar body."""

    def __init__(self, exp: AluExp, args: List[str], names: Dict[str, str], lane_sym: str, lane_base: str,
                 V: int, classes: Dict[int, str], numerics: str, indent: str, tag: str = ""):
        self.exp, self.args, self.names = exp, args, names
        self.lane_sym, self.lane_base, self.V, self.classes = lane_sym, lane_base, V, classes
        self.numerics, self.indent, self.tag = numerics, indent, tag

    def hoisted(self) -> Tuple[str, Dict[int, str]]:
        names0 = dict(self.names)
        names0[self.lane_sym] = self.lane_base
        cg = HipExpCodegen(self.args, names0, self.indent, prefix=f"h{self.tag}", numerics=self.numerics)
        nodes = [n for n in self.exp.collect(lambda x: x.op == AluOp.GlobalIndex) if id(n) in self.classes]
        for n in nodes:
            cg.countReferences(n.src[0])
        loads: Dict[int, str] = {}
        for k, n in enumerate(nodes):
            idx = strip_parens(cg.run(n.src[0]))
            st = STORAGE_CTYPE[n.dtype]
            ptr = self.args[n.arg[0]]
            if self.classes[id(n)] in ("vector", "vector_u", "vector_nt"):
                var = f"v{self.tag}{k}"
                load = {"vector": "jh_vload", "vector_u": "jh_vload_u", "vector_nt": "jh_vload_nt"}[self.classes[id(n)]]
                cg.emit(f"const jh_pack<{st}, {self.V}> {var} = {load}<{st}, {self.V}>({ptr} + ({idx}));")
                loads[id(n)] = f"{var}.v[lane]"
            elif self.classes[id(n)] in ("vector_g", "vector_gm"):
                # a group that is inside the buffer or outside it as a whole: one load from the group's place, or from
                # element 0 when it is outside, where every lane then holds element 0 as a guarded scalar load would
                var = f"v{self.tag}{k}"
                sign = ""
                if self.classes[id(n)] == "vector_gm":  # index x % C: a negative x puts the whole group outside
                    sign = f"({strip_parens(cg.run(n.src[0].src[0]))}) >= 0 && "
                cg.emit(f"const bool {var}_in = {sign}(jh_u32)({idx}) < (jh_u32){n.arg[1]};")
                cg.emit(f"jh_pack<{st}, {self.V}> {var} = jh_vload<{st}, {self.V}>({ptr} + ({var}_in ? ({idx}) : 0));")
                cg.emit(f"if (!{var}_in) {{ for (int jh_i = 1; jh_i < {self.V}; ++jh_i) {var}.v[jh_i] = {var}.v[0]; }}")
                loads[id(n)] = f"{var}.v[lane]"
            else:
                var = f"u{self.tag}{k}"
                cg.emit(f"const {st} {var} = {ptr}[{idx}];")
                loads[id(n)] = var
        return "\n".join(cg.take_lines()), loads

    def batched(self, holder: str = "Lc") -> Tuple[str, str, Dict[int, str]]:
        """The hoisted loads as a value type: (field declarations of a struct, body of a function that performs the
        loads at `lane_base` and returns the struct, the names under which the per-lane body finds them in an instance
        called `holder`).  A template fills an array of such structs first and consumes it afterwards, which is what
        puts several loads per lane in flight: left to itself the compiler issues a load, waits for it and folds it into
        the accumulator chain before it issues the next."""
        text, loads = self.hoisted()
        fields, names = [], []
        nodes = [n for n in self.exp.collect(lambda x: x.op == AluOp.GlobalIndex) if id(n) in self.classes]
        out: Dict[int, str] = {}
        for n in nodes:
            ref = loads[id(n)]
            var = ref.split(".")[0]
            st = STORAGE_CTYPE[n.dtype]
            if var not in names:
                names.append(var)
                fields.append(f"jh_pack<{st}, {self.V}> {var};" if ref.endswith(".v[lane]") else f"{st} {var};")
            out[id(n)] = f"{holder}.{ref}"
        body = text + ("\n" if text else "") + self.indent + "return jh_loads{" + ", ".join(names) + "};"
        return " ".join(fields), body, out

    def lanes(self, loads: Dict[int, str]) -> Tuple[str, str]:
        cg = HipExpCodegen(self.args, self.names, self.indent + "  ", prefix=f"l{self.tag}", numerics=self.numerics)
        cg.loads = loads
        cg.countReferences(self.exp)
        value = strip_parens(cg.run(self.exp))
        return "\n".join(cg.take_lines()), value

    def lanes_of(self, loads: Dict[int, str], exps: List[AluExp]) -> Tuple[str, List[str]]:
        """`lanes` for several expressions that share one statement list (the two factors of a product)."""
        cg = HipExpCodegen(self.args, self.names, self.indent + "  ", prefix=f"l{self.tag}", numerics=self.numerics)
        cg.loads = loads
        for e in exps:
            cg.countReferences(e)
        values = [strip_parens(cg.run(e)) for e in exps]
        return "\n".join(cg.take_lines()), values

    def scalar(self, indent: Optional[str] = None, prefix: str = "s") -> Tuple[str, str]:
        cg = HipExpCodegen(self.args, self.names, indent or self.indent, prefix=f"{prefix}{self.tag}",
                           numerics=self.numerics)
        cg.countReferences(self.exp)
        value = strip_parens(cg.run(self.exp))
        return "\n".join(cg.take_lines()), value


# "wasm": the reference Wasm backend's polynomial transcendentals, operation for operation (f32 maps within 2 ulp of
# the checker).  "fast": the same, except exp and reciprocal on the hardware's exp2 / rcp instructions (within rel
# 1e-5 of the checker; what keeps a fused softmax-style row kernel off the VALU limit).  "native": device libm.
NUMERICS = ("wasm", "fast", "native")


def _prelude(numerics: str) -> str:
    if numerics not in NUMERICS:
        raise ValueError(f"numerics must be one of {NUMERICS}")
    return (f"#define JH_WASM_NUMERICS {1 if numerics in ('wasm', 'fast') else 0}\n#define JH_FAST_NUMERICS {1 if numerics == 'fast' else 0}\n"
            + template("prelude.hip.inc") + "\n")


def _compile_options_of(kernel: Kernel, t: TuneResult) -> str:
    """Leading source lines that `runtime.compile_source` turns into compiler options.  Kernels that touch float16 are
    compiled without the SLP vectorizer: it pairs the unrolled lanes' float32 intermediates (the argument of a
    logarithm, a mean) into two-float vectors, the backend then moves a float16 negation or subtraction in front of
    the rounding, and instruction selection aborts the process on the two-float negation it made itself (packed
    float32 arithmetic is switched off for this target).  `logSigmoid`, `acos`, a variance along axis 0 and
    log-softmax over rows of 50257 in float16 all ran into it."""
    halves = kernel.dtype == DType.Float16 or any(
        e is not None and e.collect(lambda n: n.dtype == DType.Float16) for e in (t.exp, t.epilogue))
    return SOURCE_OPTION + "-fno-slp-vectorize\n" if halves else ""


_F16_PLAIN = (AluOp.Add, AluOp.Mul, AluOp.Max, AluOp.Min, AluOp.Where, AluOp.Cast, AluOp.Const, AluOp.GlobalIndex)


def epilogue_compile_options(epilogue: Optional[AluExp]) -> str:
    """The same for the matrix templates, whose per-element epilogue is inlined once per accumulator register: only
    when the epilogue does more in float16 than add, multiply by something that is not a negative constant, clamp,
    select and cast (bias, residual and ReLU keep the vectorizer; `-(a @ b)`, GELU or `logSigmoid` behind a product do
    not)."""
    if epilogue is None:
        return ""

    def risky(n: AluExp) -> bool:
        if n.dtype != DType.Float16 or n.op in (AluOp.Variable, AluOp.Special):
            return False
        if n.op == AluOp.Mul:
            return any(c.op == AluOp.Const and float(c.arg) < 0 for c in n.src)
        return n.op not in _F16_PLAIN

    return SOURCE_OPTION + "-fno-slp-vectorize\n" if epilogue.collect(risky) else ""


IDENT = {"gidx": "gidx", "ridx": "ridx"}


def generate(kernel: Kernel, numerics: str = "wasm", tune: Optional[TuneResult] = None, name: str = "jh_kernel",
             **tune_opts) -> KernelSource:
    """Full source text and launch plan for a Kernel."""
    if kernel.size >= (1 << 31) or (kernel.reduction is not None and kernel.reduction.size >= (1 << 31)):
        raise ValueError("kernel extents must stay below 2^31 (indices are int32, src/alu.ts:1463-1464)")
    t = tune or tuneHip(kernel, **tune_opts)
    if t.klass == "map":
        return _gen_map(kernel, t, numerics, name)
    if t.klass == "map_t":
        return _gen_map_transposed(kernel, t, numerics, name)
    if t.klass == "reduce_row":
        return _gen_reduce(kernel, t, numerics, name, row=True)
    if t.klass == "reduce_col":
        return _gen_reduce(kernel, t, numerics, name, row=False)
    if t.klass == "gemm":
        from .gemm import gen_gemm

        return gen_gemm(kernel, t, numerics, name)
    raise ValueError(f"unknown kernel class {t.klass}")


def _gen_map(kernel: Kernel, t: TuneResult, numerics: str, name: str) -> KernelSource:
    V, block, grid = t.params["V"], t.params["block"], t.params["grid"]
    used = _used_args(kernel.nargs, t.exp)
    out_t = STORAGE_CTYPE[kernel.dtype]
    params, args = _params(used, out_t)
    body = _Body(t.exp, args, IDENT, "gidx", "g0", V, t.vector_loads, numerics, "  ")
    load_fields, hoisted, loads = body.batched()
    body.indent = "        "
    lane_body, lane_value = body.lanes(loads)
    scalar_body, scalar_value = body.scalar("    ")
    src = _compile_options_of(kernel, t) + _prelude(numerics) + fill(template("map.hip.inc"), dict(
        SIZE=kernel.size, V=V, BLOCK=block, UNROLL=t.params.get("unroll", 1), NT_STORE=t.params.get("nt_store", 0), NAME=name, PARAMS=params, OUT_T=out_t,
        LOAD_FIELDS=load_fields, LOAD_PARAMS=_in_params(used)[0], LOAD_ARGS=_in_params(used)[1],
        VECTOR_LOADS=hoisted, LANE_BODY=lane_body, LANE_VALUE=lane_value,
        SCALAR_BODY=scalar_body, SCALAR_VALUE=scalar_value))
    step = LaunchStep(name, (grid, 1, 1), (block, 1, 1), 0,
                      [("in", i) for i in range(kernel.nargs)] + [("out", 0)])
    return KernelSource([src], [step], [], "map", _min_bytes(t.exp), dict(t.params))


def _gen_map_transposed(kernel: Kernel, t: TuneResult, numerics: str, name: str) -> KernelSource:
    """64 x 64 tiles through LDS for a map whose operand runs along another axis than its output (map_t.hip.inc)."""
    p = t.params
    shape, strides, j = p["shape"], p["strides"], p["j"]
    n = len(shape)
    ostr = [1] * n
    for i in range(n - 2, -1, -1):
        ostr[i] = ostr[i + 1] * shape[i + 1]
    used = _used_args(kernel.nargs, t.exp)
    out_t = STORAGE_CTYPE[kernel.dtype]
    params, args = _params(used, out_t)
    (load,) = t.exp.collect(lambda x: x.op == AluOp.GlobalIndex)
    cg = HipExpCodegen(args, IDENT, "        ", prefix="m", numerics=numerics)
    cg.loads = {id(load): "jh_x"}
    cg.countReferences(t.exp)
    value = strip_parens(cg.run(t.exp))
    body = "\n".join(cg.take_lines())
    outer = [i for i in range(n - 1) if i != j]
    decode = []
    for i in reversed(outer):
        decode.append(f"  {{ const long long d = rem % {shape[i]}ll; rem /= {shape[i]}ll; in_base += d * {strides[i]}ll; out_base += d * {ostr[i]}ll; }}")
    blocks = prod([shape[i] for i in outer]) * -(-shape[j] // 64) * -(-shape[-1] // 64)
    src = _compile_options_of(kernel, t) + _prelude(numerics) + fill(template("map_t.hip.inc"), dict(
        NJ=shape[j], NC=shape[-1], SC=strides[-1], OSJ=ostr[j], NAME=name, PARAMS=params, OUT_T=out_t,
        IN_T=STORAGE_CTYPE[load.dtype], IN_PTR=args[p["gid"]], IN_OFF=p["offset"], OUTER_DECODE="\n".join(decode), BODY=body, VALUE=value))
    step = LaunchStep(name, (blocks, 1, 1), (256, 1, 1), 0, [("in", i) for i in range(kernel.nargs)] + [("out", 0)])
    return KernelSource([src], [step], [], "map_t", _min_bytes(t.exp), dict(tile=64, blocks=blocks, j=j, shape=shape))


def _exact_product(exp: AluExp, re: Reduction) -> Optional[Tuple[AluExp, AluExp]]:
    """The two float16 factors when a float32 sum adds up products of float16 values widened to float32.  Such a
    product is exact in float32 (11-bit significands, exponents far inside the range), so `fma(a, b, acc)` rounds once,
    exactly where `acc + a * b` rounds: the same bits from one instruction (v_fma_mix_f32 converts both halves on the
    way in) instead of two conversions, a multiply and an add."""
    if re.op != AluOp.Add or re.dtype != DType.Float32 or exp.dtype != DType.Float32:
        return None

    def widened(e: AluExp) -> Optional[AluExp]:
        return e.src[0] if e.op == AluOp.Cast and e.dtype == DType.Float32 and e.src[0].dtype == DType.Float16 else None

    if exp.op == AluOp.Mul:
        a, b = widened(exp.src[0]), widened(exp.src[1])
        if a is not None and b is not None:
            return a, b
    if exp.op == AluOp.Cast and exp.src[0].op == AluOp.Mul and exp.src[0].dtype == DType.Float16:
        return exp.src[0].src[0], exp.src[0].src[1]  # multiplied in float32 by convention (see codegen, Cast of a product)
    return None


def _lane_accumulate(body: "_Body", loads: Dict[int, str], exp: AluExp, re: Reduction, acc_t: str, acc: str) -> Tuple[str, str]:
    """(statements, expression for the accumulator's new value) of one lane's step of the fold."""
    pair = _exact_product(exp, re)
    if pair is not None:
        text, (a, b) = body.lanes_of(loads, list(pair))
        return text, f"__builtin_fmaf((float)({a}), (float)({b}), {acc})"
    text, value = body.lanes(loads)
    return text, f"JH_REDUCE({acc}, ({acc_t})({value}))"


def _partial_pitch(size: int, V: int) -> int:
    """Row pitch of the slice-major partial buffer: the vector stores of each slice must stay aligned."""
    return -(-size // max(V, 1)) * max(V, 1)


def _gen_reduce(kernel: Kernel, t: TuneResult, numerics: str, name: str, row: bool) -> KernelSource:
    re = kernel.reduction
    assert re is not None and t.epilogue is not None
    p = dict(t.params)
    V, T, split = p["V"], p["T"], p.get("split", 1)
    R, size = re.size, kernel.size
    if re.dtype == DType.Bool:
        split = 1
    acc_t = CTYPE[re.dtype]
    out_t = STORAGE_CTYPE[kernel.dtype]
    used = _used_args(kernel.nargs, t.exp, t.epilogue if split == 1 else None)
    ident = const_literal(re.dtype, re.identity)

    if split > 1:
        unit = T * V if row else T * p.get("unroll", 1)  # column class: whole batches of loads per row slot
        slice_len = -(-R // split)
        slice_len = -(-slice_len // unit) * unit
        split = -(-R // slice_len)
    if split <= 1:
        split, slice_len = 1, R
    p["split"] = split

    params, args = _params(used, acc_t if split > 1 else out_t, "partial" if split > 1 else "out")

    if row:
        body = _Body(t.exp, args, IDENT, "ridx", "r0", V, t.vector_loads, numerics, "  ")
        load_fields, hoisted, loads = body.batched()
        body.indent = "          "
        lane_body, lane_value = _lane_accumulate(body, loads, t.exp, re, acc_t, "acc")
        scalar_body, scalar_value = body.scalar("        ")
        epi = _Body(t.epilogue, args, {"gidx": "gidx", "acc": "acc"}, "gidx", "gidx", 1, {}, numerics, "      ", "e")
        epi_body, epi_value = epi.scalar("      ", "e") if split == 1 else ("", "0")
        src = _compile_options_of(kernel, t) + _prelude(numerics) + fill(template("reduce_row.hip.inc"), dict(
            SIZE=size, R=R, V=V, T=T, BLOCK=p["block"], ROWS=p["rows"], SPLIT=split, SLICE=slice_len,
            UNROLL=p.get("unroll", 4), REDUCE=_reduce_text(re.op, re.dtype), NAME=name, PARAMS=params, ACC_T=acc_t, OUT_T=out_t,
            LOAD_FIELDS=load_fields, LOAD_PARAMS=_in_params(used)[0], LOAD_ARGS=_in_params(used)[1],
            IDENTITY=ident, VECTOR_LOADS=hoisted, LANE_BODY=lane_body, LANE_ACCUM=lane_value,
            SCALAR_BODY=scalar_body, SCALAR_VALUE=scalar_value, EPILOGUE_BODY=epi_body, EPILOGUE_VALUE=epi_value))
        grid_x = p["grid"]
        block = p["block"]
    else:
        body = _Body(t.exp, args, IDENT, "gidx", "g0", V, t.vector_loads, numerics, "  ")
        load_fields, hoisted, loads = body.batched()
        body.indent = "          "
        lane_body, lane_value = _lane_accumulate(body, loads, t.exp, re, acc_t, "acc[lane]")
        scalar_body, scalar_value = body.scalar("      ")
        epi = _Body(t.epilogue, args, {"gidx": "gidx", "acc": "accv"}, "gidx", "g0", V, t.epi_vector_loads,
                    numerics, "      ", "e")
        if split == 1:
            epi_hoisted, epi_loads = epi.hoisted()
            epi_body, epi_value = epi.lanes(epi_loads)
            tail_body, tail_value = epi.scalar("    ", "te")
        else:
            epi_hoisted = epi_body = tail_body = ""
            epi_value = tail_value = "0"
        src = _compile_options_of(kernel, t) + _prelude(numerics) + fill(template("reduce_col.hip.inc"), dict(
            SIZE=size, R=R, V=V, T=T, LX=p["lx"], SPLIT=split, SLICE=slice_len, PITCH=_partial_pitch(size, V),
            UNROLL=p.get("unroll", 4), INTERLEAVE=p.get("interleave", 0),
            LOAD_FIELDS=load_fields, LOAD_PARAMS=_in_params(used)[0], LOAD_ARGS=_in_params(used)[1],
            REDUCE=_reduce_text(re.op, re.dtype), NAME=name, PARAMS=params, ACC_T=acc_t, OUT_T=out_t,
            IDENTITY=ident, VECTOR_LOADS=hoisted, LANE_BODY=lane_body, LANE_ACCUM=lane_value,
            SCALAR_BODY=scalar_body, SCALAR_VALUE=scalar_value,
            EPI_VECTOR_LOADS=epi_hoisted, EPILOGUE_BODY=epi_body, EPILOGUE_VALUE=epi_value,
            TAIL_EPILOGUE_BODY=tail_body, TAIL_EPILOGUE_VALUE=tail_value))
        grid_x = p["grid"]
        block = p["lx"] * T

    klass = "reduce_row" if row else "reduce_col"
    need = _min_bytes(t.exp, t.epilogue)
    if split == 1:
        step = LaunchStep(name, (grid_x, 1, 1), (block, 1, 1), 0,
                          [("in", i) for i in range(kernel.nargs)] + [("out", 0)])
        return KernelSource([src], [step], [], klass, need, p)

    # Two-stage: slices -> scratch[size*split] (reduction dtype), then a small second reduce over the
    # slices that applies the caller's epilogue.  The second stage is itself a Kernel over the IR.
    grid_x = max(1, min(grid_x, (256 * 16) // split + 1))
    step1 = LaunchStep(name, (grid_x, split, 1), (block, 1, 1), 0,
                       [("in", i) for i in range(kernel.nargs)] + [("scratch", 0)])
    pitch = 1 if row else _partial_pitch(size, V)
    ks2, steps2, partial_len = fold_stage(kernel, numerics, name, split, pitch, slice_major=not row)
    p["stage2"] = ks2.info
    need.update({g: b for g, b in ks2.min_input_bytes.items() if g != kernel.nargs})
    return KernelSource([src] + ks2.sources, [step1] + steps2, [partial_len * byteWidth(re.dtype)],
                        klass + "+fold", need, p)


def fold_stage(kernel: Kernel, numerics: str, name: str, split: int, pitch: int, slice_major: bool,
               first_module: int = 1):
    """Second stage of a reduction whose reduce axis was cut into `split` slices: a Kernel over the IR that folds the
    partial accumulators (in scratch buffer 0) in slice order and applies the caller's epilogue.  Partials are laid out
    `[slice][pitch]` (slice-major, `pitch` >= size) or `[output][split]`.  Returns (its KernelSource, its launch steps
    with the scratch buffer bound and module indices shifted by `first_module`, the partial buffer's length in elements)."""
    re = kernel.reduction
    size = kernel.size
    gid_partial = kernel.nargs
    if slice_major:  # partial[slice][gidx], rows padded to the vector width
        idx = AluExp.add(AluExp.mul(AluVar.ridx, AluExp.i32(pitch)), AluVar.gidx)
        partial_len = pitch * split
    else:  # partial[gidx][slice]
        idx = AluExp.add(AluExp.mul(AluVar.gidx, AluExp.i32(split)), AluVar.ridx)
        partial_len = size * split
    stage2 = Kernel(kernel.nargs + 1, size,
                    AluExp.globalIndex(re.dtype, gid_partial, partial_len, idx),
                    Reduction(re.dtype, re.op, split, re.epilogue))
    ks2 = generate(stage2, numerics, name=name + "_fold", allow_gemm=False, allow_split=False)
    steps2 = []
    for s in ks2.steps:
        mapped = [("scratch", 0) if a == ("in", gid_partial) else a for a in s.args]
        steps2.append(LaunchStep(s.name, s.grid, s.block, s.shared, mapped, module=s.module + first_module))
    return ks2, steps2, partial_len
