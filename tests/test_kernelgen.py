"""Plan generation on the host (no GPU): properties every kernel plan must have."""
from jaxjs_hip import DType
from jaxjs_hip.kernelgen import generate


def test_every_contraction_shape_gets_a_plan():
    """Plan generation must not raise whatever the extents: rows and columns from 2 to 14336 across the tile sizes, k
    from 32 to 8192 (multiples of the slab depths and not), both layouts of B, float16 and float32.  (A k split folded
    inside the launch used to be chosen for tiles that only the general template can run, which has no such fold.)"""
    import random
    from jaxjs_hip.lowering import matmulKernel
    rng = random.Random(1)
    shapes = [(100, 14336, 4096), (65, 4096, 4096), (127, 14336, 4096), (96, 1000, 4096), (8192, 100, 4096), (300, 300, 8192)]
    rows = [2, 33, 64, 65, 100, 128, 129, 200, 256, 300, 1000, 4096]
    for _ in range(60):
        shapes.append((rng.choice(rows), rng.choice(rows + [14336]), rng.choice([32, 64, 100, 256, 768, 1000, 2048, 4096, 4100, 8192])))
    for dt in (DType.Float16, DType.Float32):
        for shape in shapes:
            for bt in (False, True):
                ks = generate(matmulKernel(*shape, dt, b_transposed=bt), "fast")
                assert ks.steps and ks.sources, (dt, shape, bt)


PINNED_PLANS = [
    # dtype, M, N, K, B stored [N,K] -> what the plan must say
    # whole tiles
    (DType.Float16, 8192, 8192, 8192, False, dict(BM=256, BN=256, direct_lds=True, splitk=1)),
    (DType.Float16, 2048, 2048, 2048, False, dict(BM=128, BN=128, BK=64, stages=4, direct_lds=True, splitk=1)),
    # edge tiles on the direct-to-LDS template: clamped loads
    (DType.Float16, 8000, 8000, 8000, False, dict(BM=256, BN=256, direct_lds=True, splitk=1)),
    (DType.Float16, 1000, 1001, 512, True, dict(BM=128, BN=128, direct_lds=True)),
    (DType.Float16, 100, 14336, 4096, False, dict(BM=128, BN=128, BK=32, direct_lds=True, splitk=2, fused_fold=True)),
    # rows of B off the 16-byte grid: repack pre-pass when the other side has >= 512 rows, the general template below
    (DType.Float16, 8192, 50257, 768, False, dict(BM=256, BN=256, direct_lds=True, repack="b")),
    (DType.Float16, 300, 1001, 512, False, dict(direct_lds=False)),
    # a k axis that is not whole slabs: both operands copied with k padded to 32 (zeros), unless the copies are huge or the
    # shape is small
    (DType.Float16, 4100, 4100, 4100, False, dict(BM=128, BN=256, direct_lds=True, repack="ab")),
    (DType.Float16, 1000, 1000, 1000, True, dict(BM=128, BN=128, direct_lds=True, repack="ab")),
    (DType.Float16, 8192, 768, 50257, False, dict(direct_lds=True, repack="ab")),
    (DType.Float16, 16384, 16384, 16400, False, dict(direct_lds=False, repack=None)),
    (DType.Float16, 300, 300, 1000, False, dict(direct_lds=False, repack=None)),
    # a few rows against a large matrix: clamped rows on 128x128 tiles, k in slices, fold launch
    (DType.Float16, 4, 14336, 4096, False, dict(BM=128, BN=128, BK=32, stages=4, direct_lds=True, splitk=2)),
    (DType.Float16, 31, 4096, 4096, True, dict(BM=128, BN=128, direct_lds=True, splitk=4)),
    (DType.Float16, 16, 14336, 4000, False, dict(BM=64, BN=128, direct_lds=False)),
    # short k under many tiles: shallow stages, several workgroups per CU
    (DType.Float16, 8192, 3072, 768, False, dict(BM=128, BN=256, BK=32, stages=2, direct_lds=True)),
    (DType.Float16, 8192, 768, 3072, False, dict(BM=128, BN=256, stages=4, direct_lds=True)),
    # f32: small shapes in 64x64 tiles with in-launch k slices, the rest unchanged
    (DType.Float32, 256, 256, 256, False, dict(BM=64, BN=64, splitk=4, fused_fold=True)),
    (DType.Float32, 512, 512, 512, True, dict(BM=64, BN=64, splitk=4, fused_fold=True)),
    (DType.Float32, 1024, 1024, 1024, False, dict(BM=128, BN=64, splitk=4, fused_fold=True)),
    (DType.Float32, 4096, 4096, 4096, False, dict(BM=128, BN=128, splitk=1)),
]


def test_gemm_plans_are_pinned():
    """The launch plan the tile chooser picks for the shapes its rules were measured on."""
    from jaxjs_hip.lowering import matmulKernel
    for dt, M, N, K, bt, want in PINNED_PLANS:
        ks = generate(matmulKernel(M, N, K, dt, b_transposed=bt), "fast")
        assert ks.klass.startswith("gemm"), (M, N, K, ks.klass)
        got = {key: ks.info.get(key) for key in want}
        assert got == want, ((dt.value, M, N, K, bt), got, want)
        if want.get("repack"):
            assert [s.name.rsplit("_", 2)[-2] for s in ks.steps][:len(want["repack"])] == ["repack"] * len(want["repack"])
            assert len(ks.scratch_bytes) == len(want["repack"])
        if want.get("repack") == "b" and not bt:
            assert ks.scratch_bytes[0] == K * (-(-N // 8) * 8) * 2


def _direct_lds_load_offsets(rows, bk, nwaves, k_contiguous, row_stride, k_stride, last):
    """Element offsets (from the tile's first row and the slab's first k) of every 16-byte load of one operand slab, as the
    direct-to-LDS template computes them: (tile row or first row of the group, k or first k of the chunk, offset)."""
    out = []
    for q in range(rows * bk * 2 // 1024 // nwaves):
        for wave in range(nwaves):
            inst = q * nwaves + wave
            for lane in range(64):
                if k_contiguous:
                    lpr = bk // 8
                    row = inst * (64 // lpr) + lane // lpr
                    swz = (row >> 2) & 3 if bk == 32 else (row >> 1) & 7
                    lc = (lane % lpr) ^ swz
                    out.append((row, lc * 8, min(row, last) * row_stride + lc * 8))
                else:
                    row_bytes = rows * 2
                    off = lane * 16
                    k = inst * (1024 // row_bytes) + off // row_bytes
                    pc = (off % row_bytes) >> 4
                    lchunk = (((pc >> 2) ^ (k & 3)) << 2) | (pc & 3)
                    lastc = (last + 1) // 8 - 1
                    out.append((lchunk * 8, k, k * k_stride + min(lchunk, lastc) * 8))
    return out


def test_clamped_edge_loads_stay_inside_the_operand():
    """A model of the direct-to-LDS loaders' source addresses (the arithmetic of `jh_lane_offset` with its clamp to the
    last row, or last whole group of eight rows, that exists): for operands whose extent is not whole tiles every
    16-byte load lies inside the operand, and the rows that exist read their own elements."""
    cases = [(8000, 64, 256, 32, 4, True), (8000, 128, 256, 64, 4, True), (8000, 64, 256, 32, 4, False), (136, 64, 128, 32, 4, False),
             (100, 64, 128, 32, 4, True), (50257, 64, 256, 32, 4, True), (50264, 64, 128, 64, 4, False), (8, 64, 128, 32, 4, False),
             (1, 64, 128, 32, 4, True), (4104, 96, 256, 32, 8, False)]
    for extent, K, tile, bk, nwaves, k_contiguous in cases:
        row_stride, k_stride = (K, 1) if k_contiguous else (1, extent)
        for t in range(-(-extent // tile)):
            r0 = t * tile
            last = min(extent - 1 - r0, tile - 1)
            for slab in range(K // bk):
                base = r0 * row_stride + slab * bk * k_stride
                for r, kk, src in _direct_lds_load_offsets(tile, bk, nwaves, k_contiguous, row_stride, k_stride, last):
                    a = base + src
                    assert 0 <= a and a + 8 <= extent * K, (extent, K, tile, t, slab, r, kk)
                    if k_contiguous and r <= last:
                        assert a == (r0 + r) * K + slab * bk + kk
                    if not k_contiguous and r + 7 <= last:
                        assert a == (slab * bk + kk) * extent + r0 + r


def test_interval_form_of_a_mask_matches_the_mask_element_by_element():
    """`gemm.interval_mask_form`: a conjunction of comparisons affine in `e` (coefficient +-1) and terms without `e` is
    rewritten as invariant terms and bounds lo <= e < hi.  Checked against the condition itself on random values of the
    other variables, for every e of a group; conditions outside the form (a coefficient of 2, a comparison of something
    not affine in e) are refused."""
    import random
    from jaxjs_hip.alu import AluExp
    from jaxjs_hip.gemm import interval_mask_form
    I, S = AluExp.i32, AluExp.special
    row, k, e = S(DType.Int32, "row", 4096), S(DType.Int32, "k", 100352), S(DType.Int32, "e", 8)
    NOT = lambda c: AluExp.cmpne(c, AluExp.bool(True))
    x = AluExp.add(AluExp.mod(k, I(56)), AluExp.mod(row, I(3)))          # column of a padded window, before e
    y = AluExp.add(AluExp.mod(AluExp.idiv(k, I(56)), I(56)), AluExp.idiv(row, I(3)))
    conds = {
        "window": AluExp.mul(AluExp.mul(AluExp.cmplt(y, I(57)), NOT(AluExp.cmplt(y, I(1)))),
                             AluExp.mul(AluExp.cmplt(AluExp.add(x, e), I(57)), NOT(AluExp.cmplt(AluExp.add(x, e), I(1))))),
        "flipped": AluExp.mul(AluExp.cmplt(I(3), AluExp.sub(x, e)), NOT(AluExp.cmplt(I(40), AluExp.sub(x, e)))),   # 3 < x - e <= 40
        "both sides": AluExp.cmplt(AluExp.add(e, I(2)), AluExp.sub(x, I(20))),
        "double negation": NOT(NOT(AluExp.cmplt(AluExp.add(e, x), I(30)))),
        "no e at all": AluExp.cmplt(y, I(20)),
    }
    rng = random.Random(5)
    for name, cond in conds.items():
        form = interval_mask_form(cond)
        assert form is not None, name
        inv, lows, highs = form
        for _ in range(300):
            ctx = {"row": rng.randrange(4096), "k": rng.randrange(100352)}
            signed = lambda v: v - (1 << 32) if v >= (1 << 31) else v  # bounds are signed 32-bit values
            lo = max([0] + [signed(b.evaluate(ctx)) for b in lows])
            hi = min([8] + [signed(b.evaluate(ctx)) for b in highs])
            ok = all(bool(t.evaluate(ctx)) for t in inv)
            for ev in range(8):
                want = bool(cond.evaluate(dict(ctx, e=ev)))
                assert want == (ok and lo <= ev < hi), (name, ctx, ev)
    assert interval_mask_form(AluExp.cmplt(AluExp.add(x, AluExp.mul(e, I(2))), I(57))) is None
    assert interval_mask_form(AluExp.cmplt(AluExp.mod(AluExp.add(x, e), I(7)), I(3))) is None


def test_float16_sources_carry_their_compiler_option_and_unknown_options_are_refused():
    """Float16 map and reduce kernels, and matrix kernels with a float16 epilogue beyond bias / ReLU, open with the line
    that switches the SLP vectorizer off for that source; float32 kernels and plain epilogues do not.  The line is
    honoured only for options on the fixed list."""
    import pytest
    from jaxjs_hip import jit as J, library as Lb
    from jaxjs_hip.codegen import SOURCE_OPTION
    from jaxjs_hip.errors import HipRuntimeError
    from jaxjs_hip.jit import ShapedArray
    from jaxjs_hip.runtime import compile_source
    line = SOURCE_OPTION + "-fno-slp-vectorize\n"

    def sources(fn, shapes, dtype):
        prog = J.jit(fn, [ShapedArray(s, dtype) for s in shapes])
        return [generate(k, "fast") for k in prog.kernels]

    for dtype, expect in ((DType.Float16, True), (DType.Float32, False)):
        gens = sources(lambda x: Lb.logSoftmax(x, -1), [(16, 1001)], dtype)
        assert {g.klass for g in gens} == {"reduce_row", "map"}
        assert all(g.sources[0].startswith(line) == expect for g in gens)
    mm = [(256, 256), (256, 256)]
    (neg,) = sources(lambda a, b: J.neg(Lb.matmul(a, b)), mm, DType.Float16)
    (relu,) = sources(lambda a, b: Lb.relu(Lb.matmul(a, b)), mm, DType.Float16)
    (neg32,) = sources(lambda a, b: J.neg(Lb.matmul(a, b)), mm, DType.Float32)
    assert neg.klass == relu.klass == neg32.klass == "gemm"
    assert neg.sources[0].startswith(line) and not relu.sources[0].startswith(line) and not neg32.sources[0].startswith(line)
    with pytest.raises(HipRuntimeError, match="not on the list"):
        compile_source(SOURCE_OPTION + "-O0\nextern \"C\" __global__ void k() {}\n", use_cache=False)


def test_wide_load_of_a_looked_up_row_reads_what_the_guarded_element_loads_read():
    """The claim behind the `vector_gm` load class, by brute force over int32 ids (extremes, multiples of the table
    length of either sign, values whose product with the row width wraps): with x = wrap(wrap(id * W) + r0 + lane),
    element loads read `x % C` (C remainder, sign of x) when it lies in [0, C) and element 0 otherwise; the wide load
    reads `x0 % C + lane` when x0 >= 0 and the remainder is in range, element 0 in every lane otherwise."""
    import numpy as np
    from jaxjs_hip import jit as J, library as Lb
    from jaxjs_hip.jit import ShapedArray

    def wrap(v):
        return (v + 2**31) % 2**32 - 2**31

    def crem(a, b):
        return a - b * int(a / b)  # truncating division, exact for |a| < 2^53

    rng = np.random.default_rng(5)
    for rows, W, V in ((50257, 768, 8), (77, 64, 8), (1000, 8, 4), (3, 16, 8)):
        C = rows * W
        ids = [0, 1, -1, rows - 1, rows, -rows, 2 * rows, -2 * rows, 2**31 - 1, -2**31, 2**31 // W, -(2**31 // W), 2**32 // W + 1]
        ids += [int(v) for v in rng.integers(-2**31, 2**31, 200)] + [int(v) for v in rng.integers(-3 * rows, 3 * rows, 200)]
        for i in ids:
            for r0 in range(0, W, V):
                x0 = wrap(wrap(i * W) + r0)
                each = [crem(wrap(x0 + lane), C) for lane in range(V)]
                each = [f if 0 <= f < C else 0 for f in each]
                f0 = crem(x0, C)
                inside = x0 >= 0 and 0 <= f0 < C
                assert each == ([f0 + lane for lane in range(V)] if inside else [0] * V), (rows, W, i, r0)
    prog = J.jit(lambda t, i: Lb.take(t, i, 0), [ShapedArray((1000, 768), DType.Float16), ShapedArray((64,), DType.Int32)])
    from jaxjs_hip.tuner import tuneHip
    assert "vector_gm" in tuneHip(prog.kernels[0]).vector_loads.values()
