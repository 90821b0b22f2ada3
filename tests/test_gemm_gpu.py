"""Kernel class (d): MFMA GEMM parity.  f16 operands / f32 accumulation; bars: integer-valued inputs exact,
otherwise |gpu - f64| <= 2*K*eps32*sum|a||b| on the accumulator plus half an ulp of the f16 result."""
import numpy as np
import pytest

from jaxjs_hip import AluExp, AluOp, AluVar, DType, Kernel, Reduction, ShapeTracker, unravelAlu
from jaxjs_hip.lowering import matmulKernel, reduceKernel
from gpu_util import device_run
from oracle import oracle

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(77)


def _check(got, A, B, K, out_f16=True):
    ref = A.astype(np.float64) @ B.astype(np.float64)
    mag = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    bound = 2 * K * np.finfo(np.float32).eps * mag
    if out_f16:
        bound = bound + np.abs(ref) * 2.0**-11 + 2.0**-24
    err = np.abs(got.astype(np.float64).reshape(ref.shape) - ref)
    assert np.all(err <= bound), f"max excess {np.max(err - bound)}"


SHAPES = [(128, 128, 64), (256, 256, 128), (200, 264, 136), (32, 32, 32), (512, 384, 1000 // 8 * 8), (96, 1024, 72),
          (1024, 1024, 1024), (128, 128, 32), (256, 512, 96), (2048, 256, 160), (1024, 64, 1024), (512, 768, 768)]


@pytest.mark.parametrize("M,N,K", SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
def test_gemm_f16_layouts(M, N, K, layout):
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    if layout == "TN":
        if M % 8:
            pytest.skip("A stored [K,M] needs M % 8 == 0 for the vector loader; other shapes take the generic class")
        full = [M, N, K]
        stA = ShapeTracker.fromShape([K, M]).permute([1, 0]).reshape([M, 1, K]).expand(full)
        stB = ShapeTracker.fromShape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
        k = reduceKernel(full, [(DType.Float16, stA), (DType.Float16, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
        bufs = [np.ascontiguousarray(A.T), B]
    else:
        k = matmulKernel(M, N, K, DType.Float16, b_transposed=(layout == "NT"))
        bufs = [A, np.ascontiguousarray(B.T) if layout == "NT" else B]
    got, ks = device_run(k, bufs)
    if layout != "NN" or N % 8 == 0:
        assert ks.klass.startswith("gemm"), ks.klass
    _check(got, A, B, K)


def test_gemm_integer_valued_is_exact():
    """Products and partial sums of small integers are exact in f32 whatever the order (the
    200-256-200 style cases of test/numpy.test.ts:1510-1660)."""
    M, N, K = 200, 200, 256
    A = RNG.integers(-4, 5, (M, K)).astype(np.float16)
    B = RNG.integers(-4, 5, (K, N)).astype(np.float16)
    got, ks = device_run(matmulKernel(M, N, K, DType.Float16), [A, B])
    assert ks.klass.startswith("gemm")
    np.testing.assert_array_equal(got.reshape(M, N).astype(np.float64), A.astype(np.float64) @ B.astype(np.float64))
    got, _ = device_run(matmulKernel(64, 64, 64, DType.Float16), [np.ones((64, 64), np.float16)] * 2)
    np.testing.assert_array_equal(got, np.full(64 * 64, 64, np.float16))


def test_gemm_matches_checker_small():
    M, N, K = 64, 96, 64
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    k = matmulKernel(M, N, K, DType.Float16)
    got, ks = device_run(k, [A, B])
    assert ks.klass.startswith("gemm")
    want = oracle.run_kernel(k, [A, B], oracle.MODE_CPU)
    np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-2, atol=1e-3)


def test_gemm_batched_two_batch_axes():
    """Attention-score layout: einsum("BLNH,BSNH->BNLS") has two batch axes that cannot be merged
    (strides from src/library/numpy/einsum.ts:345-353)."""
    Bt, Nh, L, S, H = 2, 3, 64, 96, 32
    q = RNG.normal(0, 1, (Bt, L, Nh, H)).astype(np.float16)
    kk = RNG.normal(0, 1, (Bt, S, Nh, H)).astype(np.float16)
    full = [Bt, Nh, L, S, H]
    stq = ShapeTracker.fromShape([Bt, L, Nh, H]).permute([0, 2, 1, 3]).reshape([Bt, Nh, L, 1, H]).expand(full)
    stk = ShapeTracker.fromShape([Bt, S, Nh, H]).permute([0, 2, 1, 3]).reshape([Bt, Nh, 1, S, H]).expand(full)
    k = reduceKernel(full, [(DType.Float16, stq), (DType.Float16, stk)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    got, ks = device_run(k, [q, kk])
    assert ks.klass.startswith("gemm") and ks.info["nbatch"] == Bt * Nh
    ref = np.einsum("blnh,bsnh->bnls", q.astype(np.float64), kk.astype(np.float64))
    np.testing.assert_allclose(got.reshape(ref.shape).astype(np.float64), ref, rtol=2e-3, atol=2e-2)


def test_gemm_fused_epilogue_bias_relu_f32_out():
    """Epilogue reads another buffer at the output position and changes dtype (src/frontend/jit.ts:816-889)."""
    M, N, K = 192, 320, 128
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    bias = RNG.uniform(-1, 1, N).astype(np.float32)
    base = matmulKernel(M, N, K, DType.Float16)
    acc = AluVar.acc(DType.Float32)
    n_idx = unravelAlu([M, N], AluVar.gidx)[1]
    b = AluExp.globalView(DType.Float32, 2, ShapeTracker.fromShape([N]), [n_idx])
    epi = AluExp.max(AluExp.add(acc, b), AluExp.f32(0))
    k = Kernel(3, M * N, base.exp_raw, Reduction(DType.Float32, AluOp.Add, K, epi))
    got, ks = device_run(k, [A, B, bias])
    assert ks.klass.startswith("gemm") and got.dtype == np.float32
    ref = np.maximum(A.astype(np.float64) @ B.astype(np.float64) + bias, 0)
    np.testing.assert_allclose(got.reshape(M, N), ref, rtol=1e-4, atol=1e-4)


def _random_gemm_cases():
    """Seeded shapes around the tile chooser's decision points: few tiles with a long k axis (k splits folded inside
    the launch), tile counts around the CU count, short k, ragged extents; f16 (NN and NT) and f32, with a row-bias
    + ReLU epilogue on every other case (the fold applies the caller's epilogue, loads included)."""
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(36):
        dt = DType.Float32 if i % 3 == 2 else DType.Float16
        if i % 4 == 0:  # small grids, long k: split candidates
            M, N, K = int(rng.choice([128, 256, 384])), int(rng.choice([128, 256, 512, 1024])), int(rng.choice([2048, 4096, 8192]))
        elif i % 4 == 1:  # around one tile per CU
            M, N, K = int(rng.choice([1024, 2048, 1536])), int(rng.choice([2048, 1024, 2560])), int(rng.choice([256, 512, 1024]))
        elif i % 4 == 2:  # ragged
            M, N, K = int(rng.integers(33, 700)), int(rng.integers(5, 90)) * 8, int(rng.integers(3, 60)) * 8
        else:  # short k, many tiles
            M, N, K = int(rng.choice([4096, 2048])), int(rng.choice([512, 768, 2304])), int(rng.choice([64, 96, 192]))
        cases.append((dt, M, N, K, bool(i % 2 and dt == DType.Float16 and i % 4 != 2), bool(i % 2 == 0)))
    return cases


@pytest.mark.parametrize("dt,M,N,K,bt,bias", _random_gemm_cases(), ids=lambda v: v.value if isinstance(v, DType) else str(int(v)) if not isinstance(v, bool) else ("T" if v else "F"))
def test_gemm_random_shapes_with_and_without_epilogue(dt, M, N, K, bt, bias):
    npdt = np.float16 if dt == DType.Float16 else np.float32
    A = RNG.uniform(-1, 1, (M, K)).astype(npdt)
    B = RNG.uniform(-1, 1, (K, N)).astype(npdt)
    base = matmulKernel(M, N, K, dt, b_transposed=bt)
    bufs = [A, np.ascontiguousarray(B.T) if bt else B]
    if bias:
        bv = RNG.uniform(-1, 1, N).astype(np.float32)
        acc = AluVar.acc(DType.Float32)
        n_idx = unravelAlu([M, N], AluVar.gidx)[1]
        b = AluExp.globalView(DType.Float32, 2, ShapeTracker.fromShape([N]), [n_idx])
        k = Kernel(3, M * N, base.exp_raw, Reduction(DType.Float32, AluOp.Add, K, AluExp.max(AluExp.add(acc, b), AluExp.f32(0))))
        bufs.append(bv)
    else:
        k = base
    got, ks = device_run(k, bufs)
    assert ks.klass.startswith("gemm") or K < 32, (ks.klass, ks.info)  # a k axis shorter than one slab is a plain row reduction
    ref = A.astype(np.float64) @ B.astype(np.float64)
    mag = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    bound = 2 * K * np.finfo(np.float32).eps * mag
    if bias:
        ref = np.maximum(ref + bv, 0)
        bound = bound + 4 * np.finfo(np.float32).eps * (np.abs(ref) + 1)
    elif dt == DType.Float16:
        bound = bound + np.abs(ref) * 2.0**-11 + 2.0**-24
    err = np.abs(got.astype(np.float64).reshape(ref.shape) - ref)
    assert np.all(err <= bound), f"max excess {np.max(err - bound)} with {ks.info}"


def _fuzz_gemm_cases(count=72, seed=5):
    """Seeded random contractions over everything the tile chooser branches on: extents from 2 to 5000 (few rows or
    columns against a long k included), k whole slabs or not, all four storage layouts of A and B, views that start a
    few elements into their buffer, float16 and float32."""
    rng = np.random.default_rng(seed)

    def pick():
        return int(rng.choice([rng.integers(2, 40), rng.integers(40, 300), rng.integers(300, 1500), rng.choice([64, 128, 256, 512, 1024, 2048]),
                               rng.integers(1500, 5000)]))

    cases = []
    while len(cases) < count:
        r = rng.integers(0, 6)
        M, N = pick(), pick()
        K = int(rng.choice([rng.integers(32, 200), rng.integers(200, 3000), rng.choice([64, 128, 256, 768, 1024, 2048, 4096, 8192]), rng.integers(3000, 9000),
                            8 * rng.integers(4, 600), 32 * rng.integers(1, 200)]))
        if r == 0:
            M, N, K = int(rng.integers(2, 65)), int(rng.choice([4096, 14336, 1000, 2048])), int(rng.choice([1024, 2048, 4096, 4104, 8192]))
        if r == 1:
            N, M, K = int(rng.integers(2, 65)), int(rng.choice([4096, 2048, 1001])), int(rng.choice([1024, 2048, 4096]))
        if M * N * K > 3e10 or M * N > 2e7:
            continue
        layout = str(rng.choice(["NN", "NT", "TN", "TT"]))
        dt = DType.Float16 if rng.random() < 0.75 else DType.Float32
        offs = tuple((int(rng.integers(1, 9)) if rng.random() < 0.25 else 0) for _ in range(2))
        cases.append((M, N, K, layout, dt, offs))
    return cases


@pytest.mark.parametrize("M,N,K,layout,dt,offs", _fuzz_gemm_cases(), ids=lambda v: v.value if isinstance(v, DType) else "o%d%d" % v if isinstance(v, tuple) else str(v))
def test_gemm_random_shapes_layouts_and_offsets_are_exact(M, N, K, layout, dt, offs):
    """Whatever plan a shape gets (direct-to-LDS with edge tiles, repacked operands, k slices folded in or after the launch,
    few-row tiles, the general templates, or a reduction class for thin shapes): entries in {-1, 0, 1}, the f32
    accumulator stored as it is, every element equal to the host product."""
    npdt = np.float16 if dt == DType.Float16 else np.float32
    A = RNG.integers(-1, 2, (M, K)).astype(npdt)
    B = RNG.integers(-1, 2, (K, N)).astype(npdt)
    full = [M, N, K]
    va = ShapeTracker.fromShape([M * K + offs[0]]).shrink([(offs[0], M * K + offs[0])])
    vb = ShapeTracker.fromShape([K * N + offs[1]]).shrink([(offs[1], K * N + offs[1])])
    stA = (va.reshape([K, M]).permute([1, 0]) if layout[0] == "T" else va.reshape([M, K])).reshape([M, 1, K]).expand(full)
    stB = (vb.reshape([N, K]) if layout[1] == "T" else vb.reshape([K, N]).permute([1, 0])).reshape([1, N, K]).expand(full)
    k = reduceKernel(full, [(dt, stA), (dt, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    if dt == DType.Float16:
        k = _f32_out(k, K)
    abuf = np.concatenate([np.zeros(offs[0], npdt), (A.T if layout[0] == "T" else A).ravel()])
    bbuf = np.concatenate([np.zeros(offs[1], npdt), (B.T if layout[1] == "T" else B).ravel()])
    got, ks = device_run(k, [abuf, bbuf])
    np.testing.assert_array_equal(got.reshape(M, N), A.astype(np.float32) @ B.astype(np.float32), err_msg=f"{ks.klass} {ks.info}")


def _tile_row_sample(n, bm=256):
    """Three rows of every block-tile row: the first, one in the second 128-row wave half, the last."""
    return sorted({t * bm + r for t in range(n // bm) for r in (0, bm // 2 + 3, bm - 1)})


def test_gemm_8192_cubed_sampled():
    """Headline shape.  Full f64 verification would take minutes on the host; rows are independent, so rows
    t*256 + {0, 131, 255} for every one of the 32 tile rows (both 128-row wave halves, every column, so every
    workgroup of the launch) are compared with exact dot products."""
    n = 8192
    A = RNG.uniform(-1, 1, (n, n)).astype(np.float16)
    B = RNG.uniform(-1, 1, (n, n)).astype(np.float16)
    got, ks = device_run(matmulKernel(n, n, n, DType.Float16), [A, B])
    assert ks.klass.startswith("gemm") and (ks.info["BM"], ks.info["BN"]) == (256, 256) and ks.info["direct_lds"], ks.info
    rows = _tile_row_sample(n)
    assert len(rows) == 96
    _check(got.reshape(n, n)[rows], A[rows], B, n)


def test_gemm_8192_cubed_nt_sampled():
    """The same shape with B stored [N, K]: both operands run along k, which takes the 64-deep slabs and the
    five-unit LDS ring."""
    n = 8192
    A = RNG.uniform(-1, 1, (n, n)).astype(np.float16)
    Bt = RNG.uniform(-1, 1, (n, n)).astype(np.float16)
    got, ks = device_run(matmulKernel(n, n, n, DType.Float16, b_transposed=True), [A, Bt])
    assert ks.klass.startswith("gemm") and ks.info["BK"] == 64 and ks.info["ring"] == 5, ks.info
    rows = _tile_row_sample(n)
    _check(got.reshape(n, n)[rows], A[rows], Bt.T, n)


def _f32_out(base, K):
    """The same contraction with the f32 accumulator stored as it is (no rounding to the operand type)."""
    return Kernel(base.nargs, base.size, base.exp_raw, Reduction(DType.Float32, AluOp.Add, K, AluVar.acc(DType.Float32)))


def test_gemm_8192_cubed_every_element_exact():
    """Entries in {-1, 0, 1}: every product and every partial sum is an integer below 2^24, so the f32 accumulator is
    exact in any summation order and the whole 8192 x 8192 result must equal the host product bit for bit (the
    integer-exact style of test/numpy.test.ts:1510-1660), in both layouts of B."""
    n = 8192
    A = RNG.integers(-1, 2, (n, n)).astype(np.float16)
    B = RNG.integers(-1, 2, (n, n)).astype(np.float16)
    ref = A.astype(np.float32) @ B.astype(np.float32)  # exact for these inputs whatever the BLAS blocking
    assert np.array_equal(ref[:4].astype(np.float64), A[:4].astype(np.float64) @ B.astype(np.float64))
    got, ks = device_run(_f32_out(matmulKernel(n, n, n, DType.Float16), n), [A, B])
    assert ks.klass.startswith("gemm") and got.dtype == np.float32 and ks.info["tiles"] == 1024, ks.info
    np.testing.assert_array_equal(got.reshape(n, n), ref)
    got, ks = device_run(_f32_out(matmulKernel(n, n, n, DType.Float16, b_transposed=True), n), [A, np.ascontiguousarray(B.T)])
    assert ks.klass.startswith("gemm") and ks.info["ring"] == 5, ks.info
    np.testing.assert_array_equal(got.reshape(n, n), ref)


def test_gemm_full_size_edge_tiles_and_repacked_operands_are_exact():
    """The shapes the edge-tile and repack paths were measured on, at full size with entries in {-1, 0, 1} (every sum an
    integer below 2^24: exact in the f32 accumulator, stored as f32): 8000^3 (edge tiles along both axes of the
    direct-to-LDS template), 8192 x 50257 x 768 (B's rows off the 16-byte grid: repack pre-pass, 197 tile columns the last
    one 81 wide) and 4100 x 4100 x 4100 (ragged k: both operands copied with k padded).  Rows from every tile row, the
    last rows and the last columns included, against exact host products."""
    for (M, N, K, want_repack) in ((8000, 8000, 8000, None), (8192, 50257, 768, "b"), (4100, 4100, 4100, "ab")):
        A = RNG.integers(-1, 2, (M, K)).astype(np.float16)
        B = RNG.integers(-1, 2, (K, N)).astype(np.float16)
        got, ks = device_run(_f32_out(matmulKernel(M, N, K, DType.Float16), K), [A, B])
        assert ks.klass == "gemm" and ks.info["direct_lds"] and ks.info.get("repack") == want_repack, ks.info
        bm = ks.info["BM"]
        rows = sorted({min(t * bm + r, M - 1) for t in range(-(-M // bm)) for r in (0, bm // 2 + 3, bm - 1)} | {M - 1, M - 2})
        if len(rows) > 200:
            rows = rows[::len(rows) // 150] + [M - 2, M - 1]
        ref = A[rows].astype(np.float32) @ B.astype(np.float32)
        np.testing.assert_array_equal(got.reshape(M, N)[rows], ref, err_msg=str((M, N, K)))
        del got


def test_gemm_output_just_under_two_to_the_31_elements():
    """46336 x 46336 outputs (2,147,024,896 float16 values, 4.3 GB) over a short k axis: tile origins, the tile walk and the
    store addresses near the end of the int32 index range.  Integer entries keep every value exact; rows from the first, a
    middle and the last two block-tile rows are read back by range and compared bit for bit, in both layouts of B."""
    from gpu_util import WARM_ONLY, backend
    n, K = 46336, 64
    assert 2 ** 31 - 2 ** 20 < n * n < 2 ** 31
    A = RNG.integers(-2, 3, (n, K)).astype(np.float16)
    B = RNG.integers(-2, 3, (K, n)).astype(np.float16)
    rows = [0, 1, 255, 256, 23167, 23168, 46079, 46080, 46081, 46207, 46334, 46335]
    for bt in (False, True):
        k = matmulKernel(n, n, K, DType.Float16, b_transposed=bt)
        if WARM_ONLY:
            from jaxjs_hip.kernelgen import generate
            from jaxjs_hip.runtime import compile_source
            for src in generate(k).sources:
                compile_source(src)
            if bt:
                pytest.skip("warm-up run: compiled only")
            continue
        be = backend()
        exe = be.prepareKernelSync(k)
        assert exe.data.ks.klass.startswith("gemm"), exe.data.ks.info
        Bh = np.ascontiguousarray(B.T) if bt else B
        a, b, out = be.malloc(A.nbytes, A.tobytes()), be.malloc(Bh.nbytes, Bh.tobytes()), be.malloc(k.bytes)
        try:
            be.dispatch(exe, [a, b], [out])
            for r in rows:
                got = np.frombuffer(be.readSync(out, r * n * 2, n * 2), np.float16)
                np.testing.assert_array_equal(got.astype(np.float32), A[r].astype(np.float32) @ B.astype(np.float32), err_msg=f"row {r} {exe.data.ks.info}")
        finally:
            for s_ in (a, b, out):
                be.decRef(s_)


# ---- operands off the 16-byte grid: extents that are not multiples of the 128-bit groups, odd row pitches, shifted starts

LOOSE_CASES = [
    # dtype, M, N, K, B stored [N,K], batch
    (DType.Float16, 130, 257, 100, False, ()), (DType.Float16, 130, 257, 100, True, ()), (DType.Float16, 333, 1001, 515, False, ()),
    (DType.Float16, 333, 1001, 515, True, ()), (DType.Float16, 64, 50257 // 16, 768, False, ()), (DType.Float16, 257, 129, 66, False, (3,)),
    (DType.Float16, 400, 1027, 1029, False, ()), (DType.Float16, 200, 72, 4100, True, ()),
    (DType.Float32, 130, 257, 101, False, ()), (DType.Float32, 130, 257, 101, True, ()), (DType.Float32, 333, 1001, 515, False, ()),
    (DType.Float32, 129, 66, 257, True, (2,)), (DType.Float32, 1025, 1027, 1029, False, ()),
]


@pytest.mark.parametrize("dt,M,N,K,bt,batch", LOOSE_CASES, ids=lambda v: v.value if isinstance(v, DType) else str(v))
def test_gemm_operands_off_the_vector_grid_are_exact(dt, M, N, K, bt, batch):
    """np.matmul with extents like 1001 or 50257 (row pitches that are not multiples of 16 bytes, a last 128-bit group
    that crosses the end of the axis): still the matrix-core class -- the loaders take whole groups from under-aligned
    addresses and the crossing group element by element -- and, with small integer entries, exact in every element."""
    npdt = np.float16 if dt == DType.Float16 else np.float32
    A = RNG.integers(-2, 3, batch + (M, K)).astype(npdt)
    B = RNG.integers(-2, 3, batch + (K, N)).astype(npdt)
    k = matmulKernel(M, N, K, dt, b_transposed=bt, batch=batch)
    if dt == DType.Float16:
        k = _f32_out(k, K)
    got, ks = device_run(k, [A, np.ascontiguousarray(np.swapaxes(B, -1, -2)) if bt else B])
    assert ks.klass.startswith("gemm") and not ks.info.get("direct_lds"), (ks.klass, ks.info)
    np.testing.assert_array_equal(got.reshape(batch + (M, N)).astype(np.float32), A.astype(np.float32) @ B.astype(np.float32), err_msg=str(ks.info))


@pytest.mark.parametrize("dt", [DType.Float16, DType.Float32], ids=lambda d: d.value)
def test_gemm_operands_that_start_off_the_vector_grid(dt):
    """Full tiles (256 x 256 x 128) but both operands are views that start one and three elements into their buffers:
    nothing is ragged, every 128-bit group is misaligned, and the direct-to-LDS template must not be picked."""
    M, N, K = 256, 256, 128
    npdt = np.float16 if dt == DType.Float16 else np.float32
    abuf = RNG.integers(-2, 3, M * K + 1).astype(npdt)
    bbuf = RNG.integers(-2, 3, K * N + 3).astype(npdt)
    full = [M, N, K]
    stA = ShapeTracker.fromShape([M * K + 1]).shrink([(1, M * K + 1)]).reshape([M, 1, K]).expand(full)
    stB = ShapeTracker.fromShape([K * N + 3]).shrink([(3, K * N + 3)]).reshape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
    k = reduceKernel(full, [(dt, stA), (dt, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    if dt == DType.Float16:
        k = _f32_out(k, K)
    got, ks = device_run(k, [abuf, bbuf])
    assert ks.klass.startswith("gemm") and not ks.info.get("direct_lds"), (ks.klass, ks.info)
    want = abuf[1:].reshape(M, K).astype(np.float32) @ bbuf[3:].reshape(K, N).astype(np.float32)
    np.testing.assert_array_equal(got.reshape(M, N).astype(np.float32), want)


# ---- an operand that runs along its rows with rows off the grid, against >= 512 rows of the other: copied once into scratch

REPACK_CASES = [
    # M, N, K, layout, element offset of the off-grid operand's view, tile options
    (520, 1001, 512, "NN", 0, dict()), (1024, 50257 // 16, 768, "NN", 0, dict()), (1001, 520, 256, "TN", 0, dict()),
    (512, 256, 128, "NN", 3, dict()), (640, 777, 96, "NN", 1, dict(BM=256, BN=256)), (513, 1001, 64, "NN", 0, dict(BM=256, BN=128, SADDR=0)),
    # a k axis that is not whole slabs: both operands copied, k padded with zeros
    (520, 600, 1000, "NN", 0, dict()), (1000, 1000, 1000, "NT", 0, dict()), (515, 1001, 333, "NT", 0, dict()), (1001, 520, 100, "TN", 0, dict()),
    (600, 520, 72, "NN", 1, dict(BM=256, BN=256)), (1027, 1025, 1029, "NN", 0, dict()),
]


@pytest.mark.parametrize("M,N,K,layout,off,tile", REPACK_CASES, ids=lambda v: "-".join(f"{k}{x}" for k, x in v.items()) or "default" if isinstance(v, dict) else str(v))
def test_gemm_f16_rows_off_the_grid_are_repacked(M, N, K, layout, off, tile):
    """np.matmul against a [K, 1001] matrix: every row of B starts at an odd element.  With enough rows on the other side a
    pre-pass copies B into scratch as [K][1008] and the direct-to-LDS template runs on the copy (edge tiles clamped, the
    padding never stored); a k axis that is not whole 32-deep slabs takes copies of both operands with k padded by
    zeros.  Small integer entries: exact in every element."""
    A = RNG.integers(-2, 3, (M, K)).astype(np.float16)
    B = RNG.integers(-2, 3, (K, N)).astype(np.float16)
    full = [M, N, K]
    if layout == "TN":  # A stored [K, M], M off the grid
        abuf = np.concatenate([np.zeros(off, np.float16), np.ascontiguousarray(A.T).ravel()])
        stA = ShapeTracker.fromShape([K * M + off]).shrink([(off, K * M + off)]).reshape([K, M]).permute([1, 0]).reshape([M, 1, K]).expand(full)
        bbuf = B
        stB = ShapeTracker.fromShape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
        want = "a"
    elif layout == "NT":  # B stored [N, K]
        abuf = A
        stA = ShapeTracker.fromShape([M, K]).reshape([M, 1, K]).expand(full)
        bbuf = np.concatenate([np.zeros(off, np.float16), np.ascontiguousarray(B.T).ravel()])
        stB = ShapeTracker.fromShape([N * K + off]).shrink([(off, N * K + off)]).reshape([1, N, K]).expand(full)
        want = "b"
    else:
        abuf = A
        stA = ShapeTracker.fromShape([M, K]).reshape([M, 1, K]).expand(full)
        bbuf = np.concatenate([np.zeros(off, np.float16), B.ravel()])
        stB = ShapeTracker.fromShape([K * N + off]).shrink([(off, K * N + off)]).reshape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
        want = "b"
    if K % 32:
        want = "ab"
    k = _f32_out(reduceKernel(full, [(DType.Float16, stA), (DType.Float16, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add), K)
    opts = dict(gemm_tile=tuple(sorted(tile.items()))) if tile else {}
    got, ks = device_run(k, [abuf, bbuf], **opts)
    assert ks.klass == "gemm" and ks.info["direct_lds"] and ks.info.get("repack") == want, (ks.klass, ks.info)
    np.testing.assert_array_equal(got.reshape(M, N).astype(np.float32), A.astype(np.float32) @ B.astype(np.float32), err_msg=str(ks.info))


# ---- a handful of rows (or columns) against a large operand: a linear layer on a few tokens

THIN_CASES = [
    # dtype, M, N, K, B stored [N,K], expected tile and k split
    # (f16 rows that the direct-to-LDS loads can clamp take its 128x128 tiles; a k axis that is not whole slabs keeps 64x128)
    (DType.Float16, 2, 14336, 4096, False, dict(BM=128, BN=128, splitk=2, direct_lds=True)), (DType.Float16, 16, 14336, 4096, True, dict(BM=128, BN=128, splitk=2, direct_lds=True)),
    (DType.Float16, 31, 4096, 4096, False, dict(BM=128, BN=128, splitk=4, direct_lds=True)), (DType.Float16, 64, 14336, 4096, False, dict(BM=128, BN=128, splitk=2, direct_lds=True)),
    (DType.Float16, 16, 14336, 4000, False, dict(BM=64, BN=128, splitk=1, direct_lds=False)),
    (DType.Float16, 14336, 16, 4096, False, dict(BM=128, BN=64, splitk=4)), (DType.Float16, 7, 1000, 4100, True, dict(BM=64, BN=128)),
    (DType.Float32, 4, 14336, 4096, False, dict(BM=64, BN=64, splitk=2)), (DType.Float32, 14336, 16, 4096, False, dict(BM=64, BN=64, splitk=2)),
    # 65..127 rows, few 128x128 tiles, long k: the tile is not whole (edge loads clamp); two slices folded inside the launch
    (DType.Float16, 100, 14336, 4096, False, dict(BM=128, BN=128, splitk=2, direct_lds=True, fused_fold=True)), (DType.Float16, 65, 4096, 4096, True, dict(BM=128, BN=128, splitk=4, direct_lds=True)),
    (DType.Float16, 300, 300, 8192, False, dict(BM=128, BN=128, splitk=8)), (DType.Float16, 8192, 100, 4096, False, dict(BM=128, BN=128, splitk=8)),
]


@pytest.mark.parametrize("dt,M,N,K,bt,want", THIN_CASES, ids=lambda v: v.value if isinstance(v, DType) else str(v) if not isinstance(v, dict) else "")
def test_gemm_with_a_handful_of_rows_runs_on_the_matrix_cores(dt, M, N, K, bt, want):
    """2..64 rows against a large B (or columns against a large A): as separate dot products the large operand would be
    read once per row; as one GEMM with 64-row tiles and the k axis cut over several workgroups it is read once.  The
    plan is pinned, the result (small integers) exact."""
    npdt = np.float16 if dt == DType.Float16 else np.float32
    A = RNG.integers(-1, 2, (M, K)).astype(npdt)
    B = RNG.integers(-1, 2, (K, N)).astype(npdt)
    k = matmulKernel(M, N, K, dt, b_transposed=bt)
    got, ks = device_run(k, [A, np.ascontiguousarray(B.T) if bt else B])
    assert ks.klass.startswith("gemm") and all(ks.info.get(a) == b for a, b in want.items()), (ks.klass, ks.info)
    np.testing.assert_array_equal(got.reshape(M, N).astype(np.float32), A.astype(np.float32) @ B.astype(np.float32), err_msg=str(ks.info))


def test_single_rows_and_small_operands_stay_with_the_reduction_classes():
    from jaxjs_hip.tuner import tuneHip
    for M, N, K in ((1, 14336, 4096), (14336, 1, 4096), (5, 300, 700), (16, 64, 64), (8, 100, 2048)):
        assert tuneHip(matmulKernel(M, N, K, DType.Float16)).klass.startswith("reduce"), (M, N, K)


# The dense-GEMM sweep of the benchmark configuration: square 2048 / 4096 / 8192 and the skinny 128 x 14336 x 4096,
# in f16 and f32.  Each case pins the launch shape the tuner picks for it (block tile, k split, workgroups) and is
# checked against f64 dot products under the K-scaled bound on a row sample that meets every block-tile row.
SWEEP = [
    (DType.Float16, 2048, 2048, 2048, dict(BM=128, BN=128, BK=64, stages=4, tiles=256, splitk=1, direct_lds=True)),
    (DType.Float16, 4096, 4096, 4096, dict(BM=256, BN=256, BK=32, tiles=256, splitk=1, direct_lds=True)),
    # fewer tiles than CUs: the k axis is cut over blockIdx.y, f32 partials in scratch, folded inside the launch
    (DType.Float16, 128, 14336, 4096, dict(BM=128, BN=128, BK=32, stages=4, tiles=112, splitk=2, direct_lds=True, fused_fold=True)),
    # f32 k splits are folded inside the launch by the last slice to arrive at the tile's counter
    (DType.Float32, 1024, 1024, 1024, dict(BM=128, BN=64, BK=32, tiles=128, splitk=4, fused_fold=True)),
    (DType.Float32, 2048, 2048, 2048, dict(BM=128, BN=64, BK=32, tiles=512, splitk=1)),
    (DType.Float32, 4096, 4096, 4096, dict(BM=128, BN=128, BK=32, tiles=1024, splitk=1)),
    (DType.Float32, 8192, 8192, 8192, dict(BM=128, BN=128, BK=32, tiles=4096, splitk=1)),
    (DType.Float32, 128, 14336, 4096, dict(BM=128, BN=64, BK=32, tiles=224, splitk=2, fused_fold=True)),
]


@pytest.mark.parametrize("dt,M,N,K,want", SWEEP, ids=lambda v: v.value if isinstance(v, DType) else (None if isinstance(v, dict) or v is None else str(v)))
def test_gemm_sweep_shapes(dt, M, N, K, want):
    from jaxjs_hip.kernelgen import generate

    npdt = np.float16 if dt == DType.Float16 else np.float32
    A = RNG.uniform(-1, 1, (M, K)).astype(npdt)
    B = RNG.uniform(-1, 1, (K, N)).astype(npdt)
    k = matmulKernel(M, N, K, dt)
    got, ks = device_run(k, [A, B])
    assert ks.klass.startswith("gemm"), ks.klass
    assert {key: ks.info[key] for key in want} == want, ks.info
    assert ks.info == generate(k).info  # the launch that ran is the tuner's default choice
    bm = ks.info["BM"]
    rows = _tile_row_sample(M, bm) if M >= 2 * bm else list(range(M))
    if len(rows) > 128:
        rows = rows[::len(rows) // 96]
    _check(got.reshape(M, N)[rows], A[rows], B, K, out_f16=(dt == DType.Float16))


@pytest.mark.parametrize("M,N,K,split,bt", [(384, 640, 1024, 4, False), (128, 1792, 2048, 2, False), (256, 256, 4096, 8, True), (640, 128, 512, 2, True),
                                            (200, 392, 2048, 2, False), (100, 1001, 1024, 2, True)])
def test_gemm_f16_in_launch_fold_matches_the_fold_kernel_bit_for_bit(M, N, K, split, bt):
    """The same check for the direct-to-LDS f16 template (15, 14, 4 and 5 tiles; B stored [K,N] and [N,K]; the last two
    shapes have edge tiles along both axes)."""
    from gpu_util import WARM_ONLY, backend
    k = matmulKernel(M, N, K, DType.Float16, b_transposed=bt)
    tiles = dict(BM=128, BN=128, SPLITK=split)
    opts = [dict(gemm_tile=tuple(sorted(dict(tiles, FUSEK=f).items()))) for f in (0, 1)]
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        from jaxjs_hip.tuner import tuneHip
        for o in opts:
            for src in generate(k, tune=tuneHip(k, **o)).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    Bs = np.ascontiguousarray(B.T) if bt else B
    sa, sb, so = be.malloc(A.nbytes, A.tobytes()), be.malloc(Bs.nbytes, Bs.tobytes()), be.malloc(k.bytes)
    try:
        two, one = (be.prepareKernelSync(k, **o) for o in opts)
        assert two.data.ks.klass == "gemm+fold" and one.data.ks.klass == "gemm" and one.data.ks.info["fused_fold"]
        assert one.data.ks.info["direct_lds"] and one.data.ks.info["splitk"] == split and len(one.data.ks.steps) == 1
        be.dispatch(two, [sa, sb], [so])
        want = np.frombuffer(be.readSync(so), np.float16).copy()
        _check(want.reshape(M, N), A, B, K)
        for it in range(40):
            be.dispatch(one, [sa, sb], [so])
            if it % 8 == 7 or it < 2:
                got = np.frombuffer(be.readSync(so), np.float16)
                np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16), err_msg=f"launch {it}")
    finally:
        for s_ in (sa, sb, so):
            be.decRef(s_)


@pytest.mark.parametrize("M,N,K,split", [(384, 320, 1024, 4), (1024, 1024, 1024, 4), (128, 192, 2048, 8), (640, 64, 512, 2)])
def test_gemm_f32_in_launch_fold_matches_the_fold_kernel_bit_for_bit(M, N, K, split):
    """A k split folded inside the launch (device-scope partial stores, a ticket per tile, the last slice adds all slices
    in slice order) against the same split folded by the second kernel: the same bits, on every one of 40 launches in
    a row (the counters must come back to zero, and nothing may depend on which slice arrives last).  The tile counts
    15, 128, 3 and 5 put a tile's slices on one XCD (128) and on different ones."""
    from gpu_util import WARM_ONLY, backend
    k = matmulKernel(M, N, K, DType.Float32)
    tiles = dict(BM=128, BN=64, BK=32, SPLITK=split)
    opts = [dict(gemm_tile=tuple(sorted(dict(tiles, FUSEK=f).items()))) for f in (0, 1)]
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source
        from jaxjs_hip.tuner import tuneHip
        for o in opts:
            for src in generate(k, tune=tuneHip(k, **o)).sources:
                compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float32)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float32)
    sa, sb, so = be.malloc(A.nbytes, A.tobytes()), be.malloc(B.nbytes, B.tobytes()), be.malloc(k.bytes)
    try:
        two, one = (be.prepareKernelSync(k, **o) for o in opts)
        assert two.data.ks.klass == "gemm+fold" and one.data.ks.klass == "gemm" and one.data.ks.info["fused_fold"]
        assert one.data.ks.info["splitk"] == split and len(one.data.ks.steps) == 1
        be.dispatch(two, [sa, sb], [so])
        want = np.frombuffer(be.readSync(so), np.float32).copy()
        _check(want.reshape(M, N), A, B, K, out_f16=False)
        for it in range(40):
            be.dispatch(one, [sa, sb], [so])
            if it % 8 == 7 or it < 2:
                got = np.frombuffer(be.readSync(so), np.float32)
                np.testing.assert_array_equal(got, want, err_msg=f"launch {it}")
    finally:
        for s_ in (sa, sb, so):
            be.decRef(s_)


# Direct-to-LDS pipeline variants: (M, N, K, B stored [N, K], tile options).  K values give 1, 2, 3, 5, 6 and 17
# slabs (the ring's period is five slabs); every schedule option is exercised on both slab depths.
DLDS_VARIANTS = [
    (256, 256, 64, True, dict(BK=64, RING=5)), (256, 256, 128, True, dict()), (256, 512, 192, True, dict()),
    (512, 256, 320, True, dict()), (256, 256, 384, False, dict(BK=64, RING=5)), (512, 768, 1088, True, dict()),
    (512, 768, 1088, False, dict(BK=64, RING=5)), (512, 768, 1088, True, dict(RA=2)), (512, 768, 1088, True, dict(LATE=0)),
    (512, 768, 1088, True, dict(PIN=0)), (512, 768, 1088, True, dict(SADDR=0)), (512, 768, 1088, True, dict(BAR_AT=0)),
    (512, 768, 1056, False, dict()), (512, 768, 1056, False, dict(PIN=0, SADDR=0)), (512, 768, 1056, True, dict(BK=32)),
    (512, 768, 1056, False, dict(LATE=0, BAR_AT=4)), (256, 256, 32, False, dict()),
    (512, 512, 1088, True, dict(BM=128, BN=128)), (512, 512, 1088, True, dict(BM=128, BN=128, RA=2)),
    (512, 512, 1088, True, dict(BM=256, BN=128)), (512, 512, 1088, True, dict(BM=128, BN=256, WM=1, WN=4)),
    (512, 512, 192, False, dict(BM=256, BN=128, BK=64, STAGES=3)), (512, 512, 1056, False, dict(BM=128, BN=128)),
    (512, 512, 1024, True, dict(BM=256, BN=128, BK=64, STAGES=2)),
]


@pytest.mark.parametrize("M,N,K,bt,tile", DLDS_VARIANTS, ids=lambda v: "-".join(f"{k}{x}" for k, x in v.items()) or "default" if isinstance(v, dict) else str(v))
def test_gemm_f16_direct_lds_variants(M, N, K, bt, tile):
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    k = matmulKernel(M, N, K, DType.Float16, b_transposed=bt)
    got, ks = device_run(k, [A, np.ascontiguousarray(B.T) if bt else B], gemm_tile=tuple(sorted(tile.items())))
    assert ks.klass.startswith("gemm") and ks.info["direct_lds"], ks.info
    if bt and "BK" not in tile and K % 64 == 0 and K >= 128:
        assert ks.info["BK"] == 64, ks.info
    _check(got, A, B, K)


# Edge tiles of the direct-to-LDS template: extents that are not whole block tiles.  An operand that runs along k is
# clamped to its last row (any extent), one that runs along its rows to its last whole group of eight (extent % 8 == 0);
# what lies past the edge is computed on repeated data and never stored.  (M, N, K, layout, tile options, row bias + ReLU)
EDGE_CASES = [
    (1000, 1000, 1024, "NN", dict(), False), (300, 520, 256, "NN", dict(), False), (1000, 1001, 512, "NT", dict(), False),
    (1000, 336, 512, "TN", dict(), False), (104, 1000, 256, "TN", dict(), False), (2050, 2056, 384, "NN", dict(), False),
    (520, 392, 320, "NT", dict(BM=256, BN=256, BK=64, RING=5), False), (520, 392, 320, "NN", dict(BM=256, BN=256), False),
    (520, 392, 320, "NN", dict(BM=256, BN=128, PIN=0, SADDR=0), False), (520, 392, 320, "NT", dict(BM=128, BN=256, WM=1, WN=4, SADDR=0), False),
    (1000, 1000, 512, "NN", dict(), True), (777, 520, 512, "NN", dict(BM=256, BN=256), True), (333, 136, 256, "NT", dict(), True),
    (129, 136, 64, "NN", dict(BM=128, BN=128), False), (130, 129, 64, "NT", dict(BM=128, BN=128), False),
    (200, 392, 2048, "NN", dict(BM=128, BN=128, SPLITK=4), True), (100, 14336, 4096, "NN", dict(), False),
]


@pytest.mark.parametrize("M,N,K,layout,tile,bias", EDGE_CASES, ids=lambda v: "-".join(f"{k}{x}" for k, x in v.items()) or "default" if isinstance(v, dict) else str(v))
def test_gemm_f16_direct_lds_edge_tiles(M, N, K, layout, tile, bias):
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float16)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float16)
    full = [M, N, K]
    stA = (ShapeTracker.fromShape([K, M]).permute([1, 0]) if layout == "TN" else ShapeTracker.fromShape([M, K])).reshape([M, 1, K]).expand(full)
    stB = (ShapeTracker.fromShape([N, K]) if layout == "NT" else ShapeTracker.fromShape([K, N]).permute([1, 0])).reshape([1, N, K]).expand(full)
    base = reduceKernel(full, [(DType.Float16, stA), (DType.Float16, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    bufs = [np.ascontiguousarray(A.T) if layout == "TN" else A, np.ascontiguousarray(B.T) if layout == "NT" else B]
    if bias:
        bv = RNG.uniform(-1, 1, N).astype(np.float32)
        acc = AluVar.acc(DType.Float32)
        n_idx = unravelAlu([M, N], AluVar.gidx)[1]
        b = AluExp.globalView(DType.Float32, 2, ShapeTracker.fromShape([N]), [n_idx])
        k = Kernel(3, M * N, base.exp_raw, Reduction(DType.Float32, AluOp.Add, K, AluExp.max(AluExp.add(acc, b), AluExp.f32(0))))
        bufs.append(bv)
    else:
        k = base
    opts = dict(gemm_tile=tuple(sorted(tile.items()))) if tile else {}
    got, ks = device_run(k, bufs, **opts)
    assert ks.klass.startswith("gemm") and ks.info["direct_lds"], (ks.klass, ks.info)
    assert M % ks.info["BM"] or N % ks.info["BN"], ks.info  # an edge tile exists
    ref = A.astype(np.float64) @ B.astype(np.float64)
    mag = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    bound = 2 * K * np.finfo(np.float32).eps * mag
    if bias:
        ref = np.maximum(ref + bv, 0)
        bound = bound + 4 * np.finfo(np.float32).eps * (np.abs(ref) + 1)
    else:
        bound = bound + np.abs(ref) * 2.0**-11 + 2.0**-24
    err = np.abs(got.astype(np.float64).reshape(ref.shape) - ref)
    assert np.all(err <= bound), f"max excess {np.max(err - bound)} with {ks.info}"


F32_SHAPES = [(64, 64, 64), (128, 128, 64), (200, 264, 136), (1024, 1024, 1024), (96, 1028, 72), (512, 384, 100)]


@pytest.mark.parametrize("M,N,K", F32_SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
def test_gemm_f32_layouts(M, N, K, layout):
    """Config 1/4 in f32 on v_mfma_f32_32x32x2_f32: |gpu - f64| <= 2*K*eps32*sum|a||b| (f32 rel 1e-5 class)."""
    A = RNG.uniform(-1, 1, (M, K)).astype(np.float32)
    B = RNG.uniform(-1, 1, (K, N)).astype(np.float32)
    if layout == "TN":
        if M % 4:
            pytest.skip("A stored [K,M] needs M % 4 == 0 for the vector loader")
        full = [M, N, K]
        stA = ShapeTracker.fromShape([K, M]).permute([1, 0]).reshape([M, 1, K]).expand(full)
        stB = ShapeTracker.fromShape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
        k = reduceKernel(full, [(DType.Float32, stA), (DType.Float32, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
        bufs = [np.ascontiguousarray(A.T), B]
    else:
        k = matmulKernel(M, N, K, DType.Float32, b_transposed=(layout == "NT"))
        bufs = [A, np.ascontiguousarray(B.T) if layout == "NT" else B]
    got, ks = device_run(k, bufs)
    assert ks.klass.startswith("gemm"), ks.klass
    _check(got, A, B, K, out_f16=False)


def test_gemm_f32_integer_exact_and_checker():
    M, N, K = 200, 256, 200
    A = RNG.integers(-8, 9, (M, K)).astype(np.float32)
    B = RNG.integers(-8, 9, (K, N)).astype(np.float32)
    got, ks = device_run(matmulKernel(M, N, K, DType.Float32), [A, B])
    assert ks.klass.startswith("gemm")
    np.testing.assert_array_equal(got.reshape(M, N), (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
    A = RNG.uniform(-1, 1, (64, 96)).astype(np.float32)
    B = RNG.uniform(-1, 1, (96, 64)).astype(np.float32)
    k = matmulKernel(64, 64, 96, DType.Float32)
    got, _ = device_run(k, [A, B])
    want = oracle.run_kernel(k, [A, B], oracle.MODE_WASM)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", [DType.Float16, DType.Float32], ids=lambda d: d.value)
@pytest.mark.parametrize("split", [2, 4, 8, 16], ids=lambda n: "slices%d" % n)
def test_gemm_k_slices_of_a_two_stride_axis(split, dt):
    """A stored [H, M, D] contracted over (h, d): its k axis is H runs of D elements.  Slices of two runs, of one run, of
    half and of a quarter of a run (a slice inside a run is piece z % r of run z / r) against B [K, N], which runs along
    its rows.  Integer data: every slice count gives the same bits."""
    H, D, M, N = 4, 512, 128, 128
    K = H * D
    npdt = np.float16 if dt == DType.Float16 else np.float32
    A3 = RNG.integers(-2, 3, (H, M, D)).astype(npdt)
    B = RNG.integers(-2, 3, (K, N)).astype(npdt)
    full = [M, N, K]
    stA = ShapeTracker.fromShape([H, M, D]).permute([1, 0, 2]).reshape([M, 1, K]).expand(full)
    stB = ShapeTracker.fromShape([K, N]).permute([1, 0]).reshape([1, N, K]).expand(full)
    k = reduceKernel(full, [(dt, stA), (dt, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    got, ks = device_run(k, [A3, B], gemm_tile=(("BM", 64), ("BN", 64), ("SPLITK", split)))
    assert ks.klass.startswith("gemm") and ks.info["splitk"] == split, (ks.klass, ks.info)
    A = np.ascontiguousarray(A3.transpose(1, 0, 2)).reshape(M, K)
    np.testing.assert_array_equal(got.reshape(M, N).astype(np.float64), A.astype(np.float64) @ B.astype(np.float64))


@pytest.mark.parametrize("H,D", [(4, 64), (3, 128), (2, 192)], ids=str)
def test_gemm_f16_two_level_k_with_deep_slabs(H, D):
    """A stored [H, M, D] and contracted over (h, d) against B stored [N, H*D]: both operands run along k, A in runs of
    D with a jump between heads (the attention output feeding an out-projection whose weights are stored [out, in]).
    D is a multiple of 64, so the 64-deep slabs never straddle two runs."""
    M, N, K = 512, 512, H * D
    A3 = RNG.uniform(-1, 1, (H, M, D)).astype(np.float16)
    Bt = RNG.uniform(-1, 1, (N, K)).astype(np.float16)
    full = [M, N, K]
    stA = ShapeTracker.fromShape([H, M, D]).permute([1, 0, 2]).reshape([M, 1, K]).expand(full)
    stB = ShapeTracker.fromShape([N, K]).reshape([1, N, K]).expand(full)
    k = reduceKernel(full, [(DType.Float16, stA), (DType.Float16, stB)], lambda a, b: AluExp.mul(a, b), AluOp.Add)
    got, ks = device_run(k, [A3, Bt])
    assert ks.klass.startswith("gemm") and ks.info["direct_lds"] and ks.info["BK"] == 64, ks.info
    A = np.ascontiguousarray(A3.transpose(1, 0, 2)).reshape(M, K)
    _check(got, A, Bt.T, K)
