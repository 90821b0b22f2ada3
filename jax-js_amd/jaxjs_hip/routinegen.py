"""Native launch plans for routines (the non-fusable operations, src/routine.ts:20-102).

Every routine runs on the GPU; there is no host path.  A combination without a plan (an element type the
kernels do not cover, an extent beyond a kernel's stated limit) raises `UnsupportedRoutineError` at prepare
time, which is what the Backend interface prescribes for a routine a backend lacks (src/backend.ts:236-240).

  Sort, Argsort                               `sort.hip.inc`     32-bit, float16 and float64 keys
  Scatter                                     `scatter.hip.inc`  float32/float16/float64/int32/uint32/bool updates
  TriangularSolve, Cholesky, LU, JacobiEigh   `linalg.hip.inc`   float32/float64/float16 (arithmetic in double, as the reference)
  Fft                                         `fft.hip.inc`      float32/float64/float16
  Attention (extension, not in the reference) `attention.hip.inc` float16, head size 32 / 64 / 128, any L and S
"""

from __future__ import annotations

from typing import Optional

from .alu import DType, byteWidth
from .kernelgen import KernelSource, LaunchStep, _prelude, fill, template
from .errors import UnsupportedRoutineError
from .routine import Routine, Routines, ScatterOp
from .shape import prod

_SORT_KINDS = {DType.Float32: (0, "float"), DType.Float16: (1, "jh_f16"), DType.Int32: (2, "int"),
               DType.Uint32: (3, "jh_u32"), DType.Bool: (2, "int"), DType.Float64: (4, "double")}
SORT_TILE = 8192  # 64 KB of LDS in 8-byte words: rows up to 8192 elements never leave the CU (4096 in 16-byte words)
SORT_GROUP = 8    # elements a thread sorts in registers at the end of every stage (4 for rows of <= 256: more threads stay busy)
CHOLESKY_PANEL_FROM = 192  # matrix order from which Cholesky runs panel by panel over the whole chip


def _next_pow2(n: int) -> int:
    p = 1
    while p < n:
        p <<= 1
    return p


def generateRoutine(routine: Routine, numerics: str = "wasm") -> KernelSource:
    gen = {Routines.Sort: _gen_sort, Routines.Argsort: _gen_sort, Routines.Scatter: _gen_scatter,
           Routines.TriangularSolve: _gen_trisolve, Routines.Cholesky: _gen_cholesky, Routines.LU: _gen_lu,
           Routines.JacobiEigh: _gen_jacobi, Routines.Fft: _gen_fft, Routines.Attention: _gen_attention}.get(routine.name)
    ks = gen(routine, numerics) if gen is not None else None
    if ks is None:
        raise UnsupportedRoutineError(routine.name, "hip")
    return ks


def _empty(klass: str, **info) -> KernelSource:
    return KernelSource([], [], [], klass, {}, dict(info))


def _round64(n: int, cap: int = 1024) -> int:
    return max(64, min(cap, (n + 63) // 64 * 64))


_LINALG_DEFAULTS = dict(ROUTINE=0, N=1, M=1, THREADS=64, UNIT=0, IN_LDS=0, MAX_SWEEPS=0, TOL="0.0", BATCH=1, AHEAD=16, STAGED=0, RB=1,
                        ELEM="float", CMP="float")
# Element types of the dense routines: C type, the type magnitudes are compared in, bytes per element.
_FLOAT_ELEMS = {DType.Float32: ("float", "float", 4), DType.Float64: ("double", "double", 8), DType.Float16: ("jh_f16", "float", 2)}


def _linalg_source(numerics: str, **params) -> str:
    return _prelude(numerics) + fill(template("linalg.hip.inc"), {**_LINALG_DEFAULTS, **params})


def _float_elem(t):
    """(C type, comparison type, bytes) when every operand has one and the same floating-point type, else None."""
    d = t.inputDtypes[0]
    return _FLOAT_ELEMS.get(d) if all(x == d for x in t.inputDtypes) else None


def _gen_cholesky(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape = list(t.inputShapes[0])
    if len(shape) < 2:
        raise ValueError("cholesky: input must be at least 2D")
    n, m = shape[-2], shape[-1]
    if n != m:
        raise ValueError(f"cholesky: input must be square, got [{n}, {m}]")
    el = _float_elem(t)
    if el is None or n > 8192:
        return None
    ctype, cmp_t, eb = el
    batch = prod(shape[:-2])
    if batch == 0 or n == 0:
        return _empty("cholesky", n=n, batch=batch)
    if n >= CHOLESKY_PANEL_FROM and batch * n * n * 8 <= CHOLESKY_RIGHT_LOOKING_MAX_BYTES:
        # Large matrices, right-looking: the running sums of the whole triangle in a double-precision scratch copy; per
        # 32-column panel one launch that finishes the panel and one that updates the trailing triangle (bit-identical).
        src = _linalg_source(numerics, ROUTINE=5, N=n, M=batch, ELEM=ctype, CMP=cmp_t)
        grid1 = lambda count: (max(1, min((count + 255) // 256, 1 << 16)), 1, 1)  # noqa: E731
        steps = [LaunchStep("jh_chol_init", grid1(batch * n * n), (256, 1, 1), 0, [("in", 0), ("out", 0), ("scratch", 0)])]
        for j0 in range(0, n, 32):
            after = max(0, n - j0 - 32)
            steps.append(LaunchStep("jh_chol_panel", (batch * max(1, (after + 63) // 64), 1, 1), (64, 1, 1), 0,
                                    [("scratch", 0), ("out", 0), ("const", j0)]))
            if after > 0:
                T = (after + 63) // 64
                steps.append(LaunchStep("jh_chol_update", (batch * T * T, 1, 1), (256, 1, 1), 0, [("out", 0), ("scratch", 0), ("const", j0)]))
        return KernelSource([src], steps, [batch * n * n * 8], "cholesky", {0: batch * n * n * eb},
                            dict(n=n, batch=batch, panels=(n + 31) // 32, launches=len(steps), variant="right-looking"))
    if n >= CHOLESKY_PANEL_FROM and batch * n * n < (1 << 31):
        # Large matrices: 32-column panels, two launches each, every launch spread over the chip; the same sums in the
        # same order as the single-workgroup kernel (bit-identical results).
        src = _linalg_source(numerics, ROUTINE=4, N=n, M=batch, ELEM=ctype, CMP=cmp_t)
        grid1 = lambda count: (max(1, min((count + 255) // 256, 1 << 16)), 1, 1)  # noqa: E731
        steps = [LaunchStep("jh_chol_zero", grid1(batch * n * n), (256, 1, 1), 0, [("out", 0)])]
        for j0 in range(0, n, 32):
            steps.append(LaunchStep("jh_chol_bulk", (batch * ((n - j0 + 63) // 64), 1, 1), (256, 1, 1), 0,
                                    [("in", 0), ("out", 0), ("scratch", 0), ("const", j0)]))
            after = max(0, n - j0 - 32)
            steps.append(LaunchStep("jh_chol_panel", (batch * max(1, (after + 63) // 64), 1, 1), (64, 1, 1), 0,
                                    [("scratch", 0), ("out", 0), ("const", j0)]))
        return KernelSource([src], steps, [batch * n * 32 * 8], "cholesky", {0: batch * n * n * eb},
                            dict(n=n, batch=batch, panels=(n + 31) // 32, launches=len(steps)))
    threads = _round64(n)
    src = _linalg_source(numerics, ROUTINE=0, N=n, THREADS=threads, ELEM=ctype, CMP=cmp_t)
    steps = [LaunchStep("jh_cholesky", (batch, 1, 1), (threads, 1, 1), 0, [("in", 0), ("out", 0), ("scratch", 0)])]
    return KernelSource([src], steps, [batch * n * n * eb], "cholesky", {0: batch * n * n * eb}, dict(n=n, batch=batch, threads=threads))


def _gen_trisolve(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    a_shape, b_shape = list(t.inputShapes[0]), list(t.inputShapes[1])
    if len(a_shape) < 2:
        raise ValueError(f"triangular_solve: a must be at least 2D, got {a_shape}")
    if len(b_shape) < 2:
        raise ValueError(f"triangular_solve: b must be at least 2D, got {b_shape}")
    n = a_shape[-2]
    if n != a_shape[-1] or n != b_shape[-1]:
        raise ValueError(f"triangular_solve: incompatible shapes a={a_shape}, b={b_shape}")
    el = _float_elem(t)
    if el is None:
        return None
    ctype, cmp_t, eb = el
    mats, m = prod(a_shape[:-2]), b_shape[-2]
    if prod(b_shape[:-2]) != mats:
        raise ValueError(f"triangular_solve: incompatible shapes a={a_shape}, b={b_shape}")
    if mats == 0 or m == 0 or n == 0:
        return _empty("trisolve", n=n, m=m, batch=mats)
    unit = 1 if (routine.params or {}).get("unitDiagonal", False) else 0
    need = {0: mats * n * n * eb, 1: mats * m * n * eb}
    if TRISOLVE_STAGED_FROM <= n <= TRISOLVE_STAGED_MAX_N:
        # one wave of 64 right-hand sides + three waves staging blocks of rows in LDS as doubles (two buffers <= 128 KB)
        rb = max(1, min(8, TRISOLVE_STAGED_MAX_N // n))
        src = _linalg_source(numerics, ROUTINE=1, N=n, M=m, THREADS=256, UNIT=unit, AHEAD=TRISOLVE_AHEAD, STAGED=1, RB=rb,
                             ELEM=ctype, CMP=cmp_t)
        steps = [LaunchStep("jh_trisolve_staged", (mats * ((m + 63) // 64), 1, 1), (256, 1, 1), 0,
                            [("in", 0), ("in", 1), ("out", 0), ("scratch", 0)])]
        return KernelSource([src], steps, [mats * m * n * 8], "trisolve", need,
                            dict(n=n, m=m, batch=mats, threads=256, staged=True, rows_per_block=rb))
    threads = 64 if m <= 64 else 256
    src = _linalg_source(numerics, ROUTINE=1, N=n, M=m, THREADS=threads, UNIT=unit, AHEAD=TRISOLVE_AHEAD, ELEM=ctype, CMP=cmp_t)
    blocks = mats * ((m + threads - 1) // threads)
    steps = [LaunchStep("jh_trisolve", (blocks, 1, 1), (threads, 1, 1), 0, [("in", 0), ("in", 1), ("out", 0), ("scratch", 0)])]
    return KernelSource([src], steps, [mats * m * n * eb], "trisolve", need, dict(n=n, m=m, batch=mats, threads=threads, staged=False))


def _gen_lu(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape = list(t.inputShapes[0])
    if len(shape) < 2:
        raise ValueError("lu: input must be at least 2D")
    m, n = shape[-2], shape[-1]
    el = _float_elem(t)
    if el is None:
        return None
    ctype, cmp_t, eb = el
    batch = prod(shape[:-2])
    if batch == 0 or m == 0:
        return _empty("lu", m=m, n=n, batch=batch)
    if min(m, n) >= LU_BY_COLUMNS_FROM and batch * m * n < (1 << 31):
        # Large matrices: two launches per column, the rank-1 update of the trailing block over the whole chip; the same
        # operations per element as the single-workgroup kernel (bit-identical).
        src = _linalg_source(numerics, ROUTINE=6, N=n, M=m, THREADS=1024, BATCH=batch, ELEM=ctype, CMP=cmp_t)
        grid1 = lambda count: (max(1, min((count + 255) // 256, 1 << 16)), 1, 1)  # noqa: E731
        steps = [LaunchStep("jh_lu_init", grid1(batch * m * n), (256, 1, 1), 0, [("in", 0), ("out", 0), ("out", 2)])]
        for j in range(min(m, n)):
            steps.append(LaunchStep("jh_lu_col", (batch, 1, 1), (1024, 1, 1), 0,
                                    [("out", 0), ("out", 1), ("out", 2), ("scratch", 0), ("scratch", 1), ("const", j)]))
            rows, cols = m - j - 1, n - j - 1
            if rows > 0 and cols > 0:
                steps.append(LaunchStep("jh_lu_update", (batch * ((cols + 63) // 64) * ((rows + 31) // 32), 1, 1), (256, 1, 1), 0,
                                        [("out", 0), ("scratch", 0), ("scratch", 1), ("const", j)]))
        return KernelSource([src], steps, [batch * m * 8, max(batch * 4, 16)], "lu", {0: batch * m * n * eb},
                            dict(m=m, n=n, batch=batch, launches=len(steps), variant="by columns"))
    if m > 4096:  # single workgroup: the multipliers of one column live in LDS as doubles
        return None
    threads = _round64(max(m, n))
    src = _linalg_source(numerics, ROUTINE=2, N=n, M=m, THREADS=threads, ELEM=ctype, CMP=cmp_t)
    steps = [LaunchStep("jh_lu", (batch, 1, 1), (threads, 1, 1), 0, [("in", 0), ("out", 0), ("out", 1), ("out", 2)])]
    return KernelSource([src], steps, [], "lu", {0: batch * m * n * eb}, dict(m=m, n=n, batch=batch, threads=threads))


def _gen_jacobi(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape = list(t.inputShapes[0])
    if len(shape) < 2:
        raise ValueError("jacobi_eigh: input must be at least 2D")
    n = shape[-1]
    if n != shape[-2]:
        raise ValueError(f"jacobi_eigh: input must be square, got {shape}")
    if t.inputDtypes[0] not in (DType.Float32, DType.Float16, DType.Float64):
        raise TypeError("jacobi_eigh: input must be floating-point")
    el = _float_elem(t)
    if el is None or n > 16384:
        return None
    ctype, cmp_t, eb = el
    batch = prod(shape[:-2])
    if batch == 0 or n == 0:
        return _empty("jacobi", n=n, batch=batch)
    params = routine.params or {}
    threads = _round64(n)
    in_lds = 1 if 2 * n * n * eb <= 150 * 1024 else 0  # both matrices in the CU's 160 KB of LDS: n <= 138 in float32
    src = _linalg_source(numerics, ROUTINE=3, N=n, THREADS=threads, IN_LDS=in_lds, MAX_SWEEPS=int(params["maxSweeps"]),
                         TOL=repr(float(params["tolerance"])), ELEM=ctype, CMP=cmp_t)
    steps = [LaunchStep("jh_jacobi", (batch, 1, 1), (threads, 1, 1), 0, [("in", 0), ("out", 0), ("out", 1)])]
    return KernelSource([src], steps, [], "jacobi", {0: batch * n * n * eb}, dict(n=n, batch=batch, threads=threads, in_lds=bool(in_lds)))


TRISOLVE_STAGED_FROM = 128    # matrix size from which TriangularSolve stages the matrix in LDS with helper waves
TRISOLVE_STAGED_MAX_N = 8192   # two one-row buffers of doubles still fit in LDS
TRISOLVE_AHEAD = 8       # entries of a row that a right-hand side's thread fetches ahead of its subtraction chain
LU_BY_COLUMNS_FROM = 192  # smaller dimension from which LU runs two launches per column over the whole chip
CHOLESKY_RIGHT_LOOKING_MAX_BYTES = 1 << 30  # the double-precision working copy of all matrices
FFT_FUSED_MAX_N = 8192  # 16 bytes of LDS per point: 128 KiB


def _gen_fft(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape = list(t.inputShapes[0])
    if len(shape) < 1:
        raise ValueError("fft: input must be at least 1D")
    n = shape[-1]
    if n < 1:
        raise ValueError(f"fft: final axis must be non-empty, got {n}")
    if t.inputDtypes[0] != t.inputDtypes[1] or t.inputDtypes[0] not in (DType.Float32, DType.Float16, DType.Float64):
        raise ValueError("fft: expected matching floating-point real/imag arrays")
    params = routine.params or {}
    factors = [int(f) for f in params["factors"]]
    if prod(factors) != n or any(f < 1 for f in factors):
        raise ValueError(f"fft: factors {factors} do not multiply to the axis length {n}")
    el = _float_elem(t)
    if el is None or n >= (1 << 30):
        return None
    ctype, _, eb = el
    rows = prod(shape[:-1])
    if rows == 0:
        return _empty("fft", n=n, rows=rows)
    # Rows that fit the LDS twice over (16 bytes per point) run in one launch, one workgroup per row, unless there are
    # too few rows for that to use the chip (a single long row is quicker spread over many workgroups per stage).
    S = len(factors)
    fused_max = FFT_FUSED_MAX_N * 4 // max(eb, 4)  # four buffers of n elements: 128 KiB at most
    fused = S >= 1 and n <= fused_max and (n <= 2048 or rows >= 64)
    if "singleLaunch" in params:  # tests pin either path
        fused = bool(params["singleLaunch"]) and S >= 1 and n <= fused_max
    threads = min(1024, max(64, _round64(n)))
    # Twiddle tables: stage s has span_s entries for (q, j) and radix_s^2 for (q, p), 16 bytes each.
    offsets, spans, prev = [0], [], 1
    for radix in factors:
        spans.append(prev * radix + radix * radix)
        offsets.append(offsets[-1] + spans[-1])
        prev *= radix
    lds_entries = max(spans) if spans and 4 * eb * n + 16 * max(spans) <= 150 * 1024 else 0
    src = _prelude(numerics) + fill(template("fft.hip.inc"), dict(N=n, ROWS=rows, ELEM=ctype, INVERSE=1 if params.get("inverse") else 0,
                                                                  NF=len(factors), FACTORS=", ".join(map(str, factors)) or "1",
                                                                  TW_OFFSETS=", ".join(map(str, offsets if S else [0, 0])),
                                                                  FUSED=1 if fused else 0, FUSED_THREADS=threads,
                                                                  FUSED_TABLE_ENTRIES=lds_entries))
    need = {0: rows * n * eb, 1: rows * n * eb}
    if fused:
        steps = [LaunchStep("jh_fft_rows", (min(rows, 1 << 16), 1, 1), (threads, 1, 1), 0, [("in", 0), ("in", 1), ("out", 0), ("out", 1)])]
        return KernelSource([src], steps, [], "fft", need, dict(n=n, rows=rows, factors=factors, launches=1, fused=True, lds_tables=bool(lds_entries)))
    blocks = max(1, min((rows * n + 255) // 256, 1 << 20))
    out_pair, tmp_pair = [("out", 0), ("out", 1)], [("scratch", 0), ("scratch", 1)]
    target = lambda s: out_pair if (S - 1 - s) % 2 == 0 else tmp_pair  # noqa: E731  (stage -1 is the permutation)
    steps = [LaunchStep("jh_fft_permute", (blocks, 1, 1), (256, 1, 1), 0, [("in", 0), ("in", 1)] + target(-1) + [("scratch", 2)])]
    prev = 1
    for s_, radix in enumerate(factors):
        steps.append(LaunchStep("jh_fft_stage", (blocks, 1, 1), (256, 1, 1), 0,
                                target(s_ - 1) + target(s_) + [("scratch", 2), ("const", prev), ("const", radix),
                                                               ("const", 1 if s_ == S - 1 else 0), ("const", s_)]))
        prev *= radix
    scratch = [rows * n * eb, rows * n * eb, max(offsets[-1], 1) * 16] if S >= 1 else [8, 8, 16]
    return KernelSource([src], steps, scratch, "fft", need, dict(n=n, rows=rows, factors=factors, launches=len(steps), fused=False))


_SCATTER_KINDS = {DType.Float32: (0, "float"), DType.Float16: (1, "jh_f16"), DType.Int32: (2, "int"), DType.Uint32: (3, "jh_u32"),
                  DType.Bool: (4, "int"), DType.Float64: (5, "double")}


def _gen_scatter(routine: Routine, numerics: str) -> Optional[KernelSource]:
    """Index arithmetic of src/routine.ts:226-296, unrolled over the output axes at generation time."""
    t = routine.type
    params = routine.params or {}
    op = ScatterOp(getattr(params["op"], "value", params["op"]))
    out_shape, axes, out_dim = [int(x) for x in params["shape"]], [int(x) for x in params["axis"]], int(params["outDim"])
    unique = bool(params.get("uniqueIndices", False))
    ushape = list(t.inputShapes[0])
    index_shapes = [list(s) for s in t.inputShapes[1:]]
    dtype = t.inputDtypes[0]
    if dtype not in _SCATTER_KINDS or any(d not in (DType.Int32, DType.Uint32) for d in t.inputDtypes[1:]):
        return None
    if len(axes) != len(index_shapes):
        raise ValueError(f"scatter: {len(axes)} indexed axes but {len(index_shapes)} index arrays")
    U, OUT = prod(ushape), prod(out_shape)
    if U >= (1 << 31) or OUT >= (1 << 31):
        return None
    if OUT == 0:
        return _empty("scatter", updates=U, out=OUT)
    index_rank = max((len(s) for s in index_shapes), default=0)
    ustrides = [prod(ushape[d + 1:]) for d in range(len(ushape))]
    ostrides = [prod(out_shape[d + 1:]) for d in range(len(out_shape))]
    free_dims = [d for d in range(len(ushape)) if d < out_dim or d >= out_dim + index_rank]
    if len(free_dims) != len(out_shape) - len(axes):
        raise ValueError(f"scatter: updates of shape {ushape} do not match output {out_shape} indexed on {axes}")
    coord = lambda d: f"((i / {ustrides[d]}ll) % {ushape[d]}ll)"  # noqa: E731
    lines, free_i = [], 0
    for axis, extent in enumerate(out_shape):
        if axis in axes:
            k = axes.index(axis)
            ishape = index_shapes[k]
            istrides = [prod(ishape[j + 1:]) for j in range(len(ishape))]
            first = out_dim + index_rank - len(ishape)
            terms = [f"{coord(first + j)} * {istrides[j]}ll" for j in range(len(ishape)) if ishape[j] != 1]
            cast = "(jh_i64)" if t.inputDtypes[1 + k] == DType.Int32 else "(jh_i64)(jh_u32)"
            lines.append(f"  c = {cast}idx{k}[{' + '.join(terms) or '0'}];")
        else:
            lines.append(f"  c = {coord(free_dims[free_i])};")
            free_i += 1
        lines.append(f"  if (c < 0 || c >= {extent}ll) return -1;")
        lines.append(f"  o += c * {ostrides[axis]}ll;")
    accumulate = op != ScatterOp.Update and not unique
    mode = 2 if accumulate else (0 if unique else 1)
    kind, ctype = _SCATTER_KINDS[dtype]
    nidx = len(index_shapes)
    src = _prelude(numerics) + fill(template("scatter.hip.inc"), dict(
        U=U, OUT=OUT, MODE=mode, KIND=kind, T=ctype, DEST_CODE="\n".join(lines),
        INDEX_PARAMS="".join(f", const int* __restrict__ idx{k}" for k in range(nidx)),
        INDEX_ARGS="".join(f", idx{k}" for k in range(nidx))))
    idx_args = [("in", 1 + k) for k in range(nidx)]
    grid = lambda count: (max(1, min((count + 255) // 256, 1 << 20)), 1, 1)  # noqa: E731
    steps = [LaunchStep("jh_scatter_fill", grid(OUT), (256, 1, 1), 0, [("out", 0), ("scratch", 0)])]
    if U > 0:
        if mode == 1:
            steps.append(LaunchStep("jh_scatter_claim", grid(U), (256, 1, 1), 0, [("scratch", 0)] + idx_args))
        steps.append(LaunchStep("jh_scatter_apply", grid(U), (256, 1, 1), 0, [("in", 0), ("out", 0), ("scratch", 0)] + idx_args))
    need = {0: U * byteWidth(dtype)}
    for k, ishape in enumerate(index_shapes):
        need[1 + k] = prod(ishape) * 4
    return KernelSource([src], steps, [OUT * 4 if mode == 1 else 8], "scatter", need, dict(updates=U, out=OUT, mode=mode, launches=len(steps)))


def _gen_sort(routine: Routine, numerics: str) -> Optional[KernelSource]:
    t = routine.type
    shape, dtype = list(t.inputShapes[0]), t.inputDtypes[0]
    if len(shape) == 0:
        raise ValueError(f"{routine.name.value.lower()}: cannot sort a scalar")
    if dtype not in _SORT_KINDS:
        return None
    n = shape[-1]
    rows = prod(shape[:-1])
    argsort = routine.name == Routines.Argsort
    if n == 0 or rows == 0:
        return KernelSource([], [], [], "sort", {}, dict(n=n, rows=rows))
    if n >= (1 << 30):
        return None
    P = max(_next_pow2(n), 2)
    kind, ctype = _SORT_KINDS[dtype]
    word = (8 if argsort else 4) * (2 if dtype == DType.Float64 else 1)  # bytes per keyed word
    tile = min(P, SORT_TILE * 8 // max(word, 8))
    # A thread moves eight words per pass (three strides at once, or its register group), so tile / 8 threads keep
    # every lane busy and leave room for several blocks per CU, whose barriers then overlap; with few tiles in the
    # launch the wider block (tile / 2) finishes its one tile sooner.
    threads = max(1, min(tile // 2, 1024))
    if rows * (P // tile) >= 8 * 256 and tile >= 512:
        threads = min(tile // 8, 1024)
    src = _prelude(numerics) + fill(template("sort.hip.inc"), dict(N=n, P=P, ROWS=rows, TILE=tile, ARGSORT=1 if argsort else 0,
                                                                   KIND=kind, T=ctype, THREADS=threads, GROUP=SORT_GROUP if P > 256 else 4))
    tiles = rows * (P // tile)
    outs = [("out", 0), ("out", 1)] if argsort else [("out", 0), ("out", 0)]
    steps = [LaunchStep("jh_sort_local", (tiles, 1, 1), (threads, 1, 1), 0, [("in", 0), ("scratch", 0)] + outs)]
    pair_blocks = max(1, min((rows * (P // 2) + 255) // 256, 1 << 20))
    k = tile * 2
    while k <= P:
        j = k // 2
        while j >= tile:
            steps.append(LaunchStep("jh_sort_global", (pair_blocks, 1, 1), (256, 1, 1), 0, [("scratch", 0), ("const", k), ("const", j)]))
            j //= 2
        steps.append(LaunchStep("jh_sort_merge", (tiles, 1, 1), (threads, 1, 1), 0, [("in", 0), ("scratch", 0)] + outs + [("const", k)]))
        k *= 2
    scratch = [rows * P * word] if P > tile else [16]
    need = {0: rows * n * byteWidth(dtype)}
    return KernelSource([src], steps, scratch, "sort", need, dict(n=n, rows=rows, P=P, tile=tile, argsort=argsort, launches=len(steps)))


def _gen_attention(routine: Routine, numerics: str) -> Optional[KernelSource]:
    """Fused attention over [B, L, N, H] / [B, S, N, H] float16 operands with H = 32, 64 or 128 and any L and S >= 1
    (contiguous, or strided views with unit stride along the head dimension)."""
    import math

    t = routine.type
    params = routine.params or {}
    if len(t.inputShapes) != 3 or any(len(s) != 4 for s in t.inputShapes):
        raise ValueError("attention: expected q [B,L,N,H], k [B,S,N,H], v [B,S,N,H]")
    (B, L, N, H), ks, vs = t.inputShapes
    if list(ks) != list(vs) or ks[0] != B or ks[2] != N or ks[3] != H:
        raise ValueError(f"attention: shape mismatch q={t.inputShapes[0]} k={ks} v={vs}")
    S = ks[1]
    if any(d != DType.Float16 for d in t.inputDtypes) or H not in (32, 64, 128):
        return None  # the kernel takes float16 and head sizes of one, two or four 32-row MFMA tiles
    if B * N * L == 0:
        return _empty("attention", B=B, L=L, S=S, N=N)
    if B * N * -(-L // 128) >= (1 << 31) or max(B * L * N * H, B * S * N * H) >= (1 << 31):
        return None
    scale = float(params.get("scale", 1 / math.sqrt(H)))
    # Each operand is a base buffer read through (batch, position, head) strides and an offset: contiguous
    # [B, T, N, H] unless the caller passes a view (`params["views"]`, e.g. the q/k/v slices of one QKV projection).
    views = list(params.get("views") or [None, None, None])
    lay, need = [], {}
    for i, T in enumerate((L, S, S)):
        v = views[i]
        if v is None:
            lay.append((T * N * H, N * H, H, 0))
            need[i] = B * T * N * H * 2
        else:
            sb, sp, sn, sh = v["strides"]
            if (sh != 1 and H > 1) or v["offset"] % 8 or sb % 8 or sp % 8 or sn % 8 or min(sb, sp, sn) < 0 or v["elements"] >= (1 << 31):
                return None
            lay.append((sb, sp, sn, v["offset"]))
            need[i] = v["elements"] * 2
    (qb, ql, qn, qo), (kb, ksp, kn, ko), (vb, vsp, vn, vo) = lay
    src = _prelude(numerics) + fill(template("attention.hip.inc"), dict(
        B=B, NH=N, L=L, S=S, H=H, CAUSAL=1 if params.get("isCausal") else 0, SCALE_LOG2E=repr(scale * math.log2(math.e)),
        FOLD_SCALE=1 if 0 < scale < float("inf") else 0,
        QB=qb, QL=ql, QN=qn, QOFF=qo, KB=kb, KS=ksp, KN=kn, KOFF=ko, VB=vb, VS=vsp, VN=vn, VOFF=vo,
        OB=L * N * H, OL=N * H, ON=H))
    blocks = B * N * -(-L // 128)
    steps = [LaunchStep("jh_attention", (blocks, 1, 1), (256, 1, 1), 0, [("in", 0), ("in", 1), ("in", 2), ("out", 0)])]
    return KernelSource([src], steps, [], "attention", need, dict(B=B, L=L, S=S, N=N, H=H, causal=bool(params.get("isCausal")), blocks=blocks))
