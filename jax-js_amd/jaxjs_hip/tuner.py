"""Kernel tuning for gfx950: which kernel class runs a `Kernel`, and with which tile/wave shape.

Sibling of the reference's `tuneNullopt` / `tuneWebgpu` (src/tuner.ts:219-240, 243-478).  The WebGPU
heuristics (upcast/unroll/group sizes for 32-wide SIMD groups and a 65535-group grid) do not carry
over; `tuneHip` instead classifies the lowered expression's memory accesses and picks one of the
hand-written CDNA4 templates:

  map         no reduction: V consecutive outputs per lane, 128-bit loads/stores, blocks in buffer order
  reduce_row  reduce axis contiguous in memory: T lanes walk one output's reduce axis with vector
              loads, wave64 shuffle tree (+ LDS across waves) to combine; matvec W[M,K].x is this
              class with one wave per row
  reduce_col  output axis contiguous in memory: each lane owns V consecutive outputs and loops the
              reduce axis, optionally split over the waves of a block and combined through LDS
  (both reduce classes can additionally split the reduce axis over blocks; partials then go to a
   scratch buffer and a second, tiny reduce kernel applies the epilogue -- deterministic, no atomics)
  gemm        dense contraction `sum_k A*B` with strided single-view operands: MFMA tiles

The choice between classes uses a small affine analysis (`lane_form`) of every buffer index with
respect to `gidx` and `ridx`; nothing is decided from the source-level op that produced the kernel.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

from .alu import AluExp, AluGroup, AluOp, AluVar, DType, Kernel, Reduction, byteWidth, isFloatDtype
from .shape import ShapeTracker, unravelAlu

CU_COUNT = 256          # MI355X: 8 XCDs x 32 CUs; replaced by the device's own count once a backend is up
WAVE = 64
MAX_GRID_BLOCKS = CU_COUNT * 16


def set_compute_units(n: int) -> None:
    """Take the CU count from the initialised device (`jh_get_device_info`); 256 stays the value for ahead-of-time
    generation without a device."""
    global CU_COUNT, MAX_GRID_BLOCKS
    if n and n > 0:
        CU_COUNT = int(n)
        MAX_GRID_BLOCKS = CU_COUNT * 16
# Map kernels get one block per 256 lane groups rather than a capped grid-stride launch: blocks are dispatched in
# order, so the chip walks the buffers front to back (open DRAM pages are used up before they close), whereas a
# block that strides by the whole grid touches a new page every trip: 5.0-5.3 -> 5.9-6.3 TB/s on streams of 400 MB
# and more (measured: copy, a+b, exp(x)/2 in f16 and f32; unrolling the strided loop made it slower).
MAP_GRID_BLOCKS = 1 << 22
MAP_BLOCK = 256
MAP_NT_BYTES = 320 << 20  # streams of a map beyond this: nontemporal loads and stores
GEMM_ENABLED = True


@dataclass
class TuneResult:
    """Lowered expression pair plus launch geometry (cf. `TuneResult`, src/tuner.ts:29-59)."""

    exp: AluExp
    epilogue: Optional[AluExp]
    klass: str = "map"
    params: Dict[str, int] = field(default_factory=dict)
    # Index nodes (by id) of `exp` that are read with one vector load per V lanes, or once per group.
    vector_loads: Dict[int, str] = field(default_factory=dict)  # id(node) -> "vector" | "vector_u" | "uniform"
    epi_vector_loads: Dict[int, str] = field(default_factory=dict)
    gemm: Optional[dict] = None


def tuneNullopt(kernel: Kernel) -> TuneResult:
    """Lower views and bind gidx/ridx ranges without any optimisation (src/tuner.ts:219-240)."""
    exp = kernel.exp
    vars_ = {"gidx": AluExp.special(DType.Int32, "gidx", max(kernel.size, 1))}
    re = kernel.reduction
    if re is not None:
        vars_["ridx"] = AluExp.special(DType.Int32, "ridx", max(re.size, 1))
        if exp.dtype != re.dtype:
            exp = AluExp.cast(re.dtype, exp)
    epilogue = None
    if re is not None:
        epilogue = re.epilogue.substitute({"gidx": vars_["gidx"]}).rewriteGlobalViews().reduceExactIndex().simplify()
    return TuneResult(exp=exp.substitute(vars_).rewriteGlobalViews().reduceExactIndex().simplify(), epilogue=epilogue)


# ------------------------------------------------------------------------------------------------
# Affine lane analysis
# ------------------------------------------------------------------------------------------------


def _is_symbol(e: AluExp, name: str) -> bool:
    return (e.op == AluOp.Special and e.arg[0] == name) or (e.op == AluOp.Variable and e.arg == name)


def references(e: AluExp, name: str, memo: Optional[dict] = None) -> bool:
    return e.some(lambda n: _is_symbol(n, name))


def known_divisor(e: AluExp) -> int:
    """An integer that provably divides e's value (0 means "e is 0", i.e. divisible by anything)."""
    if e.op == AluOp.Const:
        return abs(int(e.arg)) if float(e.arg).is_integer() else 1
    if e.op == AluOp.Mul:
        a, b = known_divisor(e.src[0]), known_divisor(e.src[1])
        return a * b
    if e.op in (AluOp.Add, AluOp.Sub):
        return math.gcd(known_divisor(e.src[0]), known_divisor(e.src[1]))
    if e.op == AluOp.Mod and e.src[1].op == AluOp.Const:
        return math.gcd(known_divisor(e.src[0]), abs(int(e.src[1].arg)))
    if e.op == AluOp.Where:
        return math.gcd(known_divisor(e.src[1]), known_divisor(e.src[2]))
    return 1


def _may_wrap(e: AluExp) -> bool:
    """Can the int32 arithmetic of e wrap around (it then holds a loaded value: index arithmetic alone stays in range)?"""
    return not (e.min >= -(1 << 31) and e.max <= (1 << 31) - 1)


def _wrapped(e: AluExp, divisor: int) -> int:
    """What is left of a divisibility claim when e may have wrapped modulo 2^32: its power-of-two part."""
    return (divisor & -divisor) if divisor and _may_wrap(e) else divisor


def lane_form(e: AluExp, sym: str, V: int) -> Optional[Tuple[int, int]]:
    """Describe e when `sym = V*q + lane`, lane in [0,V): returns (stride, align) such that
    e == u + stride*lane with u independent of lane and u % align == 0 (align 0: u is 0), or None
    if e is not affine in the lane.  Only index arithmetic (int32 +,-,*,/,% by constants) is
    understood, plus int32 values loaded at an index the whole group shares (stride 0, no alignment known); everything
    else referencing `sym` is "unknown".  Once a loaded value is involved the arithmetic may wrap modulo 2^32: the
    form then holds modulo 2^32, `align` keeps only its power-of-two part, and a product with a nonzero stride is
    "unknown".
    """
    if not references(e, sym):
        return (0, _wrapped(e, known_divisor(e)))
    if _is_symbol(e, sym):
        return (1, V)
    if e.dtype not in (DType.Int32, DType.Uint32):
        return None
    op = e.op
    if op == AluOp.GlobalIndex:
        # a value loaded at an index the whole group shares (the row id of a table lookup): the same for every lane
        f = lane_form(e.src[0], sym, V)
        return (0, 1) if f is not None and f[0] == 0 else None
    if op in (AluOp.Add, AluOp.Sub):
        a, b = lane_form(e.src[0], sym, V), lane_form(e.src[1], sym, V)
        if a is None or b is None:
            return None
        stride = a[0] + b[0] if op == AluOp.Add else a[0] - b[0]
        return (stride, _wrapped(e, math.gcd(a[1], b[1])))
    if op == AluOp.Mul:
        for i in (0, 1):
            c = e.src[i]
            if c.op == AluOp.Const:
                f = lane_form(e.src[1 - i], sym, V)
                if f is None or (f[0] != 0 and _may_wrap(e)):
                    return None
                return (f[0] * int(c.arg), _wrapped(e, f[1] * abs(int(c.arg))))
        return None
    if op in (AluOp.Idiv, AluOp.Mod) and e.src[1].op == AluOp.Const:
        C = int(e.src[1].arg)
        inner = e.src[0]
        f = lane_form(inner, sym, V)
        if f is None or C <= 0 or inner.min < 0:
            return None
        stride, align = f
        if stride == 0:
            return (0, math.gcd(align, C) if op == AluOp.Mod else 1)
        # (u + s*lane) with 0 <= s*lane < s*V: stays inside one period of C when C | u's alignment
        # step, i.e. when both C and align are multiples of s*V.
        if stride < 0:
            return None
        span = stride * V
        if C % span == 0 and (align == 0 or align % span == 0):
            if op == AluOp.Mod:
                return (stride, math.gcd(align, C))
            return (0, 1)
        return None
    return None


def _load_nodes(exp: Optional[AluExp]) -> List[AluExp]:
    return exp.collect(lambda n: n.op == AluOp.GlobalIndex) if exp is not None else []


def _in_bounds(node: AluExp) -> bool:
    idx = node.src[0]
    return idx.min >= 0 and idx.max < node.arg[1]


def classify_loads(exp: Optional[AluExp], sym: str, V: int, guarded: bool = False) -> Dict[int, str]:
    """id(GlobalIndex node) -> "vector" (V consecutive, aligned elements per lane group), "vector_u" (V consecutive
    elements whose first is not known to sit on a multiple of V: rows of odd length, views shifted by an element) or
    "uniform" (same element for the whole group).  Loads needing a bounds guard stay scalar, except (`guarded`) the
    ones whose groups are inside the buffer or outside it as a whole -- the first index a multiple of V, positive or
    negative, and the buffer a multiple of V long: "vector_g", the pieces of a concatenation or of a padding along an
    outer axis; "vector_gm" when that holds for x in an index x % C (the rows of a table lookup)."""
    out: Dict[int, str] = {}
    if V <= 1:
        return out
    for node in _load_nodes(exp):
        if not _in_bounds(node):
            if guarded and node.arg[1] % V == 0 and V & (V - 1) == 0:
                idx = node.src[0]
                f = lane_form(idx, sym, V)
                if f is not None and f[0] == 1 and f[1] % V == 0:
                    out[id(node)] = "vector_g"
                elif (idx.op == AluOp.Mod and idx.dtype == DType.Int32 and idx.src[1].op == AluOp.Const
                      and int(idx.src[1].arg) > 0 and int(idx.src[1].arg) % V == 0):
                    # x % C with x = x0 + lane, x0 a multiple of V of either sign (a table row chosen by a loaded id):
                    # for x0 >= 0 the remainders are x0 % C + lane; for x0 < 0 every lane's remainder is negative, or
                    # zero in lane 0 alone, and under the guard all of them read element 0
                    f = lane_form(idx.src[0], sym, V)
                    if f is not None and f[0] == 1 and f[1] % V == 0:
                        out[id(node)] = "vector_gm"
            continue
        f = lane_form(node.src[0], sym, V)
        if f is None:
            continue
        stride, align = f
        if stride == 0:
            out[id(node)] = "uniform"
        elif stride == 1:
            out[id(node)] = "vector" if (align == 0 or align % V == 0) else "vector_u"
    return out


def _pow2_floor(x: int) -> int:
    return 1 << (max(int(x), 1).bit_length() - 1)


def _elem_sizes(exp: Optional[AluExp]) -> List[int]:
    return [byteWidth(n.dtype) for n in _load_nodes(exp)]


def _pick_vector_width(kernel: Kernel, t: TuneResult, axis_len: int) -> int:
    """Elements per lane so that the narrowest stream moves 128 bits."""
    sizes = _elem_sizes(t.exp) + _elem_sizes(t.epilogue) + [byteWidth(kernel.dtype)]
    smallest = min(sizes)
    V = max(16 // smallest, 1)
    if max(sizes) == 8:
        V = min(V, 4)
    while V > 1 and axis_len < V:
        V //= 2
    return V


# ------------------------------------------------------------------------------------------------
# GEMM recognition
# ------------------------------------------------------------------------------------------------


def _strip_float_casts(e: AluExp) -> AluExp:
    while e.op == AluOp.Cast and isFloatDtype(e.dtype) and isFloatDtype(e.src[0].dtype):
        e = e.src[0]
    return e


def _flatten_k_split(st) -> Optional[tuple]:
    """(view, k0, sk1) describing the operand as ONE strided view over the broadcast shape.

    A single-view tracker is returned as is (k0 = sk1 = 0).  Two views are accepted when the outer one
    is a plain row-major reshape whose last axis K covers exactly the last two axes (K1, K0) of the
    inner view and whose other axes map one-to-one onto the inner view's leading axes -- what
    `x.transpose(..).reshape([.., K1*K0])` followed by a Dot produces (attention output [B,N,L,H] read
    as [B,L,N*H]).  Then element k of the reduce axis lives at (k // K0) * sk1 + (k % K0) * sk0, and
    the returned view carries sk0 as its last stride."""
    if len(st.views) == 1:
        return st.views[0], 0, 0
    if len(st.views) != 2:
        return None
    inner, outer = st.views
    if inner.mask is not None or outer.mask is not None or outer.offset != 0 or len(inner.shape) < 2:
        return None
    # The outer view must address the inner view's logical space row-major (stride-0 axes aside).
    live = [(i, n) for i, n in enumerate(outer.shape) if n != 1 and outer.strides[i] != 0]
    if not live or live[-1][0] != len(outer.shape) - 1:
        return None
    expect = 1
    for i, n in reversed(live):
        if outer.strides[i] != expect:
            return None
        expect *= n
    lead = live[:-1]
    # Trailing axes of the inner view that are contiguous with each other count as one (the cotangent of a convolution
    # read as [O, N, H, W] -> [O, N*H*W]: H and W merge, N stays a second stride).
    ishape, istrides = list(inner.shape), list(inner.strides)
    while len(ishape) > len(lead) + 2 and istrides[-2] == istrides[-1] * ishape[-1]:
        ishape[-2:] = [ishape[-2] * ishape[-1]]
        istrides[-2:] = [istrides[-1]]
    if len(ishape) != len(inner.shape):
        from .shape import View
        inner = View(tuple(ishape), tuple(istrides), inner.offset, None)
    if len(lead) != len(inner.shape) - 2 or any(n != inner.shape[j] for j, (_, n) in enumerate(lead)):
        return None
    K1, K0 = inner.shape[-2], inner.shape[-1]
    if K1 * K0 != live[-1][1] or expect != math.prod(inner.shape):
        return None
    strides = [0] * len(outer.shape)
    for j, (i, _) in enumerate(lead):
        strides[i] = inner.strides[j]
    strides[-1] = inner.strides[-1]
    from .shape import View
    flat = View(tuple(outer.shape), tuple(strides), inner.offset, None)
    return flat, K0, inner.strides[-2]


def _span(view, k0: int, sk1: int) -> int:
    """One past the largest element index the operand can touch."""
    hi = view.offset
    dims = list(zip(view.shape, view.strides))
    if k0:
        K = view.shape[-1]
        dims = dims[:-1] + [(k0, view.strides[-1]), (K // k0, sk1)]
    for n, s in dims:
        if n > 0 and s > 0:
            hi += (n - 1) * s
    return hi + 1


def match_gemm(kernel: Kernel) -> Optional[dict]:
    """Recognise `sum_k A[..m..,k] * B[..n..,k]` over single-view, unmasked operands.

    Same precondition the reference's WebGPU tuner checks before optimising a reduction
    (src/tuner.ts:255-282): every GlobalView is indexed by `[unravel(gidx)..., ridx]`.  Axes of the
    broadcast shape are then classified by the operands' strides into batch / M / N, adjacent axes
    with compatible strides are merged, and exactly one M and one N axis must remain.
    """
    re = kernel.reduction
    if re is None or re.op != AluOp.Add or re.dtype != DType.Float32:
        return None
    root = _strip_float_casts(kernel.exp)
    if root.op != AluOp.Mul:
        return None
    a, b = _strip_float_casts(root.src[0]), _strip_float_casts(root.src[1])
    if a.op != AluOp.GlobalView or b.op != AluOp.GlobalView or a.dtype != b.dtype:
        return None
    if a.dtype not in (DType.Float16, DType.Float32):
        return None
    # An operand that is not one plain strided view (masked, or several views: the patches of a convolution,
    # a padded or dilated activation) is a *gather* operand: its tile is loaded element by element through
    # its own index expression.  Only its outermost view is looked at here, and only to see which output
    # axes it depends on (stride 0 = independent).
    def describe(gv):
        f = _flatten_k_split(gv.arg[1])
        if f is not None and f[0].mask is None:
            vec = 8 if gv.dtype == DType.Float16 else 4
            # a two-stride k axis is only loadable in runs that hold whole 64-deep slabs; otherwise: element loader
            if not f[1] or (f[0].strides[-1] == 1 and f[1] % 64 == 0 and f[2] % vec == 0 and f[2] > 0):
                return f[0], f[1], f[2], False
        outer = gv.arg[1].views[-1]
        if outer.mask is not None:
            return None
        return outer, 0, 0, True

    da, db = describe(a), describe(b)
    if da is None or db is None:
        return None
    (va, ka0, ka1, ga), (vb, kb0, kb1, gb) = da, db
    # (Both operands may be gather operands: the cotangent of a convolution's activations contracts a patch view of the
    # output cotangent with the filter read through a flip and a transpose.  Both tiles are then built by element
    # loaders -- slower to fill than vector loads, but the products still run on the matrix cores.)
    if va.shape != vb.shape or len(va.shape) < 1:
        return None
    shape = list(va.shape)
    if shape[-1] != re.size or math.prod(shape[:-1]) != kernel.size or kernel.size == 0 or re.size == 0:
        return None
    expected = [u.simplify() for u in unravelAlu(shape[:-1], AluVar.gidx)] + [AluVar.ridx]
    for gv in (a, b):
        if len(gv.src) != len(expected) or any(x.simplify() is not y for x, y in zip(gv.src, expected)):
            return None
    ska, skb = va.strides[-1], vb.strides[-1]
    if shape[-1] > 1 and ((ska == 0 and not ga) or (skb == 0 and not gb)):
        return None
    # Output strides: row-major over shape[:-1].
    outs = [1] * (len(shape) - 1)
    for i in range(len(outs) - 2, -1, -1):
        outs[i] = outs[i + 1] * shape[i + 1]
    axes = []  # (role, size, stride_a, stride_b, stride_out)
    for i in range(len(shape) - 1):
        n = shape[i]
        if n == 1:
            continue
        sa, sb = va.strides[i], vb.strides[i]
        role = "batch" if (sa != 0) == (sb != 0) else ("m" if sa != 0 else "n")
        axes.append([role, n, sa, sb, outs[i]])
    # Merge neighbours of equal role whose strides nest (outer == inner * inner_size).
    merged: List[list] = []
    for ax in axes:
        if merged and merged[-1][0] == ax[0]:
            p = merged[-1]
            nest = [4] + ([] if ga else [2]) + ([] if gb else [3])  # a gather operand's own strides do not matter
            if all(p[k] == ax[k] * ax[1] for k in nest):
                merged[-1] = [p[0], p[1] * ax[1], ax[2], ax[3], ax[4]]
                continue
        merged.append(ax)
    # Several M (or N) axes that do not nest (rows of a transposed activation): keep the innermost as
    # the tile axis and walk the outer ones like batch axes (the other operand's stride there is 0).
    # (For a gather operand, whose strides play no part, the tile axis is the largest of them when the innermost is
    # short: the filter cotangent of a convolution has rows (channels, ky, kx) with the output channels between the two
    # -- 64 rows by channel and 9 taps as batch fill an MFMA tile, 9 rows per channel do not.)
    for role, gathered in (("m", ga), ("n", gb)):
        idx = [i for i, x in enumerate(merged) if x[0] == role]
        keep = idx[-1] if idx else None
        if gathered and len(idx) > 1 and merged[idx[-1]][1] < 32:
            keep = max(idx, key=lambda i: (merged[i][1], i))
        for i in idx:
            if i != keep:
                merged[i][0] = "batch"
    ms = [x for x in merged if x[0] == "m"]
    ns = [x for x in merged if x[0] == "n"]
    bs = [x for x in merged if x[0] == "batch"]
    if len(ms) > 1 or len(ns) > 1 or len(bs) > 3:
        return None
    m = ms[0] if ms else ["m", 1, 0, 0, 0]
    n = ns[0] if ns else ["n", 1, 0, 0, 0]
    info = dict(
        dtype=a.dtype, gid_a=a.arg[0], gid_b=b.arg[0],
        M=m[1], N=n[1], K=shape[-1],
        a_off=va.offset, a_sm=m[2], a_sk=ska, a_k0=ka0 or shape[-1], a_sk1=ka1,
        b_off=vb.offset, b_sn=n[3], b_sk=skb, b_k0=kb0 or shape[-1], b_sk1=kb1,
        c_sm=m[4], c_sn=n[4],
        batch=[(x[1], x[2], x[3], x[4]) for x in bs],
        a_len=_span(va, ka0, ka1), b_len=_span(vb, kb0, kb1),
        a_gather=ga, b_gather=gb, a_node=a, b_node=b,
    )
    if ga:
        info.update(a_off=0, a_sm=0, a_sk=1, a_k0=shape[-1], a_sk1=0, a_len=0)
    if gb:
        info.update(b_off=0, b_sn=0, b_sk=1, b_k0=shape[-1], b_sk1=0, b_len=0)
    # The tile writes C with its lanes along n: when the output is contiguous along m instead (the first
    # operand indexes the fastest output axis), exchange the operands' roles -- A.B^T and B.A^T are the same sums.
    if info["c_sm"] == 1 and info["c_sn"] != 1 and info["N"] > 1:
        sw = dict(info)
        for x, y in (("gid_a", "gid_b"), ("a_off", "b_off"), ("a_sm", "b_sn"), ("a_sk", "b_sk"), ("a_k0", "b_k0"),
                     ("a_sk1", "b_sk1"), ("a_len", "b_len"), ("a_gather", "b_gather"), ("a_node", "b_node"), ("M", "N"),
                     ("c_sm", "c_sn")):
            sw[x], sw[y] = info[y], info[x]
        sw["batch"] = [(n, sb, sa, sc) for n, sa, sb, sc in info["batch"]]
        info = sw
    # Negative strides (flipped views) are left to the generic path.
    if min(info["a_sm"], info["a_sk"], info["b_sn"], info["b_sk"], info["a_off"], info["b_off"]) < 0:
        return None
    ga, gb = info["a_gather"], info["b_gather"]
    if any(min(x[1:]) < 0 for x in info["batch"]) and not (ga or gb):
        return None
    if ga or gb:
        # batch strides of the gather operand are never used; keep the plain operand's and the output's
        info["batch"] = [(n, 0 if ga else sa, 0 if gb else sb, sc) for n, sa, sb, sc in info["batch"]]
        if any(min(x[1:]) < 0 for x in info["batch"]):
            return None
    return info


# ------------------------------------------------------------------------------------------------
# tuneHip
# ------------------------------------------------------------------------------------------------


def _grid_for(blocks_needed: int) -> int:
    return max(1, min(int(blocks_needed), MAX_GRID_BLOCKS))


def match_transposed_map(kernel: Kernel) -> Optional[dict]:
    """A map over exactly one operand, read through one unmasked strided view whose unit-stride axis is not the output's
    fastest axis (a transpose or axis permutation written out): {gid, shape, strides, offset, j} with j the operand's
    unit-stride axis.  Anything else (several operands, masks, position-dependent expressions, small arrays) is None."""
    if kernel.reduction is not None or kernel.size < (1 << 16):
        return None
    exp = kernel.exp
    views = exp.collect(lambda n: n.op == AluOp.GlobalView)
    if len(views) != 1 or exp.collect(lambda n: n.op == AluOp.GlobalIndex):
        return None
    node = views[0]
    gid, st = node.arg
    if len(st.views) != 1 or st.views[0].mask is not None or node.dtype not in (DType.Float16, DType.Float32, DType.Int32, DType.Uint32):
        return None
    v = st.views[0]
    shape, strides = list(v.shape), list(v.strides)
    if len(shape) < 2 or math.prod(shape) != kernel.size or strides[-1] in (0, 1) or any(x < 0 for x in strides):
        return None
    expected = [u.simplify() for u in unravelAlu(shape, AluVar.gidx)]
    if len(node.src) != len(expected) or any(x.simplify() is not y for x, y in zip(node.src, expected)):
        return None
    rest = exp.rewrite(lambda n: AluExp.const(n.dtype, 0) if n is node else None)
    if references(rest, "gidx"):
        return None  # the expression also depends on the position itself
    js = [i for i in range(len(shape) - 1) if strides[i] == 1 and shape[i] >= 32]
    if not js or shape[-1] < 32:
        return None
    return dict(gid=gid, shape=shape, strides=strides, offset=v.offset, j=js[-1])


def tuneHip(kernel: Kernel, *, allow_gemm: bool = True, allow_split: bool = True,
            gemm_tile: Optional[tuple] = None, col_strip: Optional[tuple] = None,
            row_lanes: Optional[int] = None, row_unroll: Optional[int] = None, row_nt: Optional[int] = None, col_nt: Optional[int] = None,
            map_unroll: Optional[int] = None, map_nt: Optional[int] = None) -> TuneResult:
    """Pick the kernel class and its parameters for one Kernel on MI355X."""
    t = tuneNullopt(kernel)
    re = kernel.reduction
    size = kernel.size

    if re is None:
        tm = match_transposed_map(kernel)
        if tm is not None:
            t.klass = "map_t"
            t.params = dict(tm)
            return t
        V = _pick_vector_width(kernel, t, size)
        t.klass = "map"
        t.vector_loads = classify_loads(t.exp, "gidx", V, guarded=True)
        groups = max(size // V, 1)
        # Groups per lane (their loads all issued before the first is consumed).  One by default: with a block per 256
        # groups the resident waves already keep enough loads in flight, and 2-8 groups per lane measured 1-15 % slower
        # on 50-400 MB streams; the option stays for measurements.
        unroll = int(map_unroll) if map_unroll else 1
        blocks = (groups + MAP_BLOCK * unroll - 1) // (MAP_BLOCK * unroll)
        nt_store = 0
        # Streams that together exceed the 256 MB memory-side cache are read with the nontemporal hint (float16 copy of
        # 201 MB: 67 -> 58 us, the softmax maps of a 96 x 1024 x 1024 score tensor 67 -> 56 us; the hint on the stores
        # adds nothing, and plain stores leave the result in that cache for the next kernel); smaller streams keep
        # ordinary loads (268 MB of float32 in and out: 37 us against 41 with the hint).
        if map_nt is None:
            streamed = kernel.bytes + sum(n.arg[1] * byteWidth(n.dtype) for n in _load_nodes(t.exp) if t.vector_loads.get(id(n)) == "vector")
            map_nt = 2 if streamed >= MAP_NT_BYTES else 0  # the loads carry the gain; plain stores leave the result cached
        if map_nt:  # 1: loads and stores, 2: loads only, 3: stores only
            t.vector_loads = dict(t.vector_loads)
            for node in _load_nodes(t.exp):
                if map_nt != 3 and t.vector_loads.get(id(node)) == "vector" and node.arg[1] * 2 >= size and size >= (1 << 22):
                    t.vector_loads[id(node)] = "vector_nt"
            nt_store = 1 if size >= (1 << 22) and map_nt != 2 else 0
        t.params = dict(V=V, block=MAP_BLOCK, unroll=unroll, nt_store=nt_store, grid=max(1, min(blocks, MAP_GRID_BLOCKS)))
        return t

    R = re.size
    if allow_gemm and GEMM_ENABLED:
        g = match_gemm(kernel)
        if g is not None and _gemm_worthwhile(g):
            t.klass = "gemm"
            t.gemm = g
            if gemm_tile:
                t.params["gemm_tile"] = dict(gemm_tile)
            return t

    loads = _load_nodes(t.exp)
    Vr = _pick_vector_width(kernel, t, R)
    along_r = classify_loads(t.exp, "ridx", Vr)
    Vg = _pick_vector_width(kernel, t, size)
    along_g = classify_loads(t.exp, "gidx", Vg)
    n_row = sum(1 for v in along_r.values() if v in ("vector", "vector_u"))
    n_col = sum(1 for v in along_g.values() if v in ("vector", "vector_u"))
    # Which axis do the heavy streams walk at unit stride?  Weight every load by the bytes it can
    # touch, so that a large matrix decides the orientation and a small broadcast vector does not.
    w_row = w_col = 0
    for node in loads:
        weight = node.arg[1] * byteWidth(node.dtype)
        fr = lane_form(node.src[0], "ridx", 1)
        fg = lane_form(node.src[0], "gidx", 1)
        if fr is not None and fr[0] == 1:
            w_row += weight
        elif fg is not None and fg[0] == 1:
            w_col += weight

    row_major = w_row >= w_col and w_row > 0 and R >= 8
    # A short fold (up to 256 steps: what the column template unrolls whole) whose only stream along the reduce axis is a
    # small table, under many outputs (the first layer of a small CNN: 9 or 25 or 75 filter taps per output, one or three
    # input channels, millions of outputs): one lane per output walks the
    # taps, so that consecutive lanes read consecutive pixels, instead of a few lanes sharing every output's taps.
    # (The image itself is unit-stride along both axes -- a window row is a few consecutive pixels --, so it is weighed
    # here by its stride along the outputs.)
    if row_major and R <= 256 and size >= CU_COUNT * 256:
        w_g = w_r_only = 0
        for node in loads:
            fr, fg = lane_form(node.src[0], "ridx", 1), lane_form(node.src[0], "gidx", 1)
            weight = node.arg[1] * byteWidth(node.dtype)
            if fg is not None and 1 <= fg[0] <= 4:  # (a strided window walk reads every 2nd..4th pixel)
                w_g += weight
            elif fr is not None and fr[0] == 1:
                w_r_only += weight
        if w_g >= 8 * w_r_only and w_g > 0:
            row_major = False
    if w_row == 0 and w_col == 0 and size < 4096 and R >= 1024:
        row_major = True  # few outputs, long fold, no coalescing either way: spread the fold over lanes

    if row_major:
        V = Vr if n_row > 0 else 1
        vec_iters = max(R // V, 1)
        t_hi = min(_pow2_floor(vec_iters), 1024)
        # Enough lanes per row that a wave reads long contiguous runs, then ~8 vector loads per lane.  Rows of at most 64
        # vector loads take 8 lanes (sixteen left half of them with one load fewer, and the tree one step longer:
        # 75648 rows of 197 f16 6.7 -> 5.4 us, of 197 f32 11.0 -> 10.1 us, 65536 rows of 200 f16 6.0 -> 5.3 us).
        T = max(min(t_hi, 8 if vec_iters <= 64 else 16), min(_pow2_floor(max(vec_iters // 8, 1)), t_hi))
        while T < t_hi and size * T < CU_COUNT * 512:
            T *= 2
        if row_lanes:  # tuning override: lanes per output row
            T = int(row_lanes)
        block = max(T, 256)
        rows = block // T
        split = 1
        if allow_split:
            lanes_busy = size * T
            if lanes_busy < CU_COUNT * 512 and R // (T * V) >= 64:
                want = (CU_COUNT * 1024) // max(lanes_busy, 1)
                split = max(1, min(want, R // (T * V * 8), 1024))
        t.klass = "reduce_row"
        t.vector_loads = dict(along_r) if V > 1 else {}
        # A stream that this launch reads once (about one element per (output, reduce index) pair: the matrix of a
        # matvec, the rows of a row reduction) is loaded with the nontemporal hint, so that it does not displace the
        # operands every row reuses from L2.
        if row_nt is None or row_nt:
            for node in loads:
                if t.vector_loads.get(id(node)) == "vector" and node.arg[1] * 2 >= size * R and size * R >= (1 << 22):
                    t.vector_loads[id(node)] = "vector_nt"
        # All of a lane's vector loads of a row are issued before the first is consumed when the row is short enough
        # (at most 16 per lane); longer rows go four at a time.
        trips = R // (T * V) if split == 1 else 0
        nvec = max(1, len(t.vector_loads))
        unroll = trips if 1 <= trips <= 16 else 4
        unroll = max(1, min(unroll, 32 // nvec))  # a batch holds unroll x nvec x 4 registers per lane
        if row_unroll:
            unroll = int(row_unroll)
        t.params = dict(V=V, T=T, block=block, rows=rows, split=split, unroll=unroll)
        nrb = (size + rows - 1) // rows
        t.params["grid"] = _grid_for(nrb)
        return t

    V = Vg if n_col > 0 else 1
    groups = max(size // V, 1)
    lx = 64
    # Split the fold over waves (and blocks) when there are too few output groups to fill the chip.
    # Blocks stay small (at most 4 waves) when the fold may also be cut across blocks: many small
    # blocks spread over all 256 CUs, a few 1024-thread blocks leave most of them without work.
    t_max = 4 if allow_split else 16
    T = 1
    while T < t_max and groups * T < CU_COUNT * 256 and R // (T * 2) >= 8:
        T *= 2
    split = 1
    if allow_split and groups * T < CU_COUNT * 512 and R // T >= 64:
        want = (CU_COUNT * 1024) // max(groups * T, 1)
        split = max(1, min(want, R // (T * 16), 1024))
    # Row loads a lane issues before it consumes the first (reduce_col.hip.inc fills a batch, then folds it).
    nvec_g = max(1, sum(1 for c in along_g.values() if c.startswith("vector")))
    unroll, interleave = (8 if nvec_g <= 2 else 4), 0
    if split > 1 and V > 1:
        # Slices over blocks: a lane keeps 16 of its row loads in flight (8 when the expression reads more than two
        # vector streams), and slices are whole batches long (kernelgen rounds them), so no batch is ragged.
        unroll = 16 if nvec_g <= 2 else 8
    if split > 1 and V > 1 and col_strip:
        # Tuning override, kept for measurements: strips of `lanes` x 16 bytes handled by blocks of `block` threads.  The
        # default above -- 1 KiB strips, 4 row slots per block, the rows cut until the launch has about three blocks per
        # CU, partial sums folded by a second launch -- measured 16.0-16.3 us on the transposed float16 matvec
        # [4096, 11008] against 16.9 us for one launch of 172 blocks that each own a 128-byte strip and all rows.
        lx_line = 8  # 8 lanes x 16 bytes = one 128-byte line per row
        blk = 1024
        rows_split = 1
        if col_strip:  # (lanes per strip, block size, unroll[, blocks along the reduce axis[, interleaved rows]]): tuning override
            lx_line, blk, unroll = col_strip[:3]
            rows_split = col_strip[3] if len(col_strip) > 3 else 1
            interleave = col_strip[4] if len(col_strip) > 4 else 0
        strips = -(-groups // lx_line)
        if (strips >= CU_COUNT // 2 or (col_strip and strips * rows_split >= CU_COUNT // 2)) and R // (blk // lx_line) >= 8:
            lx, T, split, unroll = lx_line, blk // lx_line, rows_split, (unroll if col_strip else 8)
    if split == 1 and T % 4 == 0 and V > 1 and lx == 64 and 64 <= groups < 64 * (CU_COUNT // 2) and not col_strip:
        # Few column groups and no cut over blocks (the fold launch behind a cut reduction is the typical case: 11008
        # outputs x 32 slices): 64-lane strips would give a handful of workgroups that each walk their rows alone.
        # Strips of 16 lanes (256 bytes per row) put four times as many CUs on the same bytes, the row slots sharing a
        # wave and meeting through lane exchanges instead of LDS (whole waves only: four row slots or a multiple).
        lx = 16
    t.klass = "reduce_col"
    t.vector_loads = dict(along_g) if V > 1 else {}
    if col_nt is None or col_nt:  # a stream read once by this launch: nontemporal, as in the row class
        for node in loads:
            if t.vector_loads.get(id(node)) == "vector" and node.arg[1] * 2 >= size * R and size * R >= (1 << 22):
                t.vector_loads[id(node)] = "vector_nt"
    t.params = dict(V=V, T=T, lx=lx, block=lx * T, split=split, unroll=unroll, interleave=interleave)
    # The cap on the grid is meant for 256-thread blocks; blocks of one wave (no split of the fold over row slots) get
    # proportionally more of them, or a short fold over many outputs (a depthwise convolution: 6.4 M outputs of 9 terms)
    # runs four waves per SIMD where it wants sixteen.
    t.params["grid"] = max(1, min((groups + lx - 1) // lx, MAX_GRID_BLOCKS * max(1, 256 // (lx * T))))
    t.epi_vector_loads = classify_loads(t.epilogue, "gidx", V) if V > 1 else {}
    return t


GEMM_MIN_K = 32     # a shorter reduce axis than this: the reduction classes
GEMM_MIN_ROWS = 32  # fewer rows (or columns) than this only against a large operand (see _gemm_worthwhile)


def _gemm_worthwhile(g: dict) -> bool:
    """MFMA tiles only pay off for a real dense contraction; thin shapes stream better through the
    row-reduce template (matvec and friends).  The tile loaders move 128-bit vectors along an operand's unit-stride
    axis (k or the row axis); the direct-to-LDS template needs every such vector whole and on the 16-byte grid, the
    general float16 template and the float32 template also take operands where they are not (see `operand_ok`)."""
    thin = min(g["M"], g["N"])
    # (A convolution's gathered operand makes the reduction classes walk its window arithmetic once per output; it
    # pays to pad even a 27-long k axis -- 3 channels x 3 x 3 -- to one slab: 83 -> 14 us.)
    if g["K"] < (GEMM_MIN_K // 2 if g.get("a_gather") or g.get("b_gather") else GEMM_MIN_K) or thin < 2:
        return False  # one row or column is a matvec: the reduction classes stream it at the HBM rate
    if thin < GEMM_MIN_ROWS and (max(g["M"], g["N"]) < 128 or g["K"] < 256 or max(g["M"], g["N"]) * g["K"] < (1 << 20)):
        return False
    # (2..31 rows against a large operand -- a linear layer on a handful of tokens -- do go to the matrix cores: as
    # separate dot products the large operand is read once per row, 202 us for 16 x 14336 x 4096 against 25 us.)
    vec = 8 if g["dtype"] == DType.Float16 else 4
    bstr_a = [b[1] for b in g["batch"]]
    bstr_b = [b[2] for b in g["batch"]]

    def operand_ok(tag, sk, srow, rows, off, bstr, k0):
        """An operand with a unit-stride axis.  `g[tag + "_loose"]` records whether its 128-bit groups are all whole and
        on the 16-byte grid; if not, the general float16 template and the float32 template load them loosely (under-aligned
        addresses, the group across the end of the axis element by element) -- a two-level k axis has no such path."""
        if sk == 1:
            tight = g["K"] % vec == 0 and srow % vec == 0 and off % vec == 0 and all(x % vec == 0 for x in bstr)
        elif srow == 1:
            tight = rows % vec == 0 and sk % vec == 0 and off % vec == 0 and all(x % vec == 0 for x in bstr)
        else:
            return False
        g[tag + "_loose"] = not tight
        return tight or k0 == g["K"]

    def split_ok(k0, sk, sk1):
        # A two-level k axis is only loaded along unit-stride runs, and no k-slab may straddle two runs.
        return k0 == g["K"] or (sk == 1 and k0 % 64 == 0 and sk1 % vec == 0 and sk1 > 0)

    # (Gather operands take any k extent: the element loader and the row-vector loader check every k, and the block
    # loaders of the tap-major order are only chosen when k is a multiple of 8.)
    return ((g.get("a_gather") or operand_ok("a", g["a_sk"], g["a_sm"], g["M"], g["a_off"], bstr_a, g["a_k0"]))
            and (g.get("b_gather") or operand_ok("b", g["b_sk"], g["b_sn"], g["N"], g["b_off"], bstr_b, g["b_k0"]))
            and split_ok(g["a_k0"], g["a_sk"], g["a_sk1"]) and split_ok(g["b_k0"], g["b_sk"], g["b_sk1"]))
