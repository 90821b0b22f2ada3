"""Differential fuzzing of the kernel path: random typed expression trees over a few input buffers, lowered as map
kernels and as reductions in both memory orientations, GPU against the CPU oracle (Wasm mode).  Integer, unsigned and
bool results must be bit-exact; f32 results within the map tolerance (rel 1e-5 + atol 1e-6; reductions K-scaled)."""
import math
import random

import numpy as np
import pytest

import gpu_util
from gpu_util import WARM_ONLY, assert_parity
from jaxjs_hip import AluExp, AluOp, DType, ShapeTracker
from jaxjs_hip.lowering import mapKernel, reduceKernel

pytestmark = pytest.mark.gpu
F32, I32, U32, BOOL = DType.Float32, DType.Int32, DType.Uint32, DType.Bool
# JAXHIP_FUZZ_OFFSET=<n> shifts every seed below by n: the same tests over expressions, shapes and views not seen before.
OFFSET = int(__import__("os").environ.get("JAXHIP_FUZZ_OFFSET", "0"))


@pytest.fixture(params=["wasm", "fast"])
def numerics_mode(request):
    """The float tests run twice: on the Wasm-faithful numerics and on the backend's default ("fast": exp and
    reciprocal on hardware instructions, each within rel 1e-5 of the checker's polynomial forms).  The generators keep
    exp arguments inside [-4, 4], far from both stated exceptions of the fast mode (results below 2^-126, and
    x * log2(e) in [127.5, 128) where the polynomial form already returns Inf)."""
    gpu_util.set_numerics(request.param)
    yield request.param
    gpu_util.set_numerics("wasm")


def rand_exp(rng, leaves, dtype, depth):
    """A random expression of `dtype` over typed leaves {dtype: [AluExp]}; float subtrees stay well conditioned
    (bounded magnitudes, no cancellation-prone transcendentals of large arguments)."""
    if depth == 0 or rng.random() < 0.15:
        if rng.random() < 0.75 and leaves.get(dtype):
            return rng.choice(leaves[dtype])
        if dtype == F32:
            return AluExp.f32(rng.choice([0.0, 1.0, -1.0, 0.5, 2.0, 3.25, -0.75]))
        if dtype == I32:
            return AluExp.i32(rng.choice([0, 1, -1, 2, 3, 7, -5, 100, 65537]))
        if dtype == U32:
            return AluExp.u32(rng.choice([0, 1, 2, 3, 7, 255, 65537, 0x80000001]))
        return AluExp.bool(rng.random() < 0.5)
    sub = lambda dt: rand_exp(rng, leaves, dt, depth - 1)  # noqa: E731
    r = rng.random()
    if dtype == BOOL:
        if r < 0.45:
            dt = rng.choice([F32, I32, U32])
            return (AluExp.cmplt if rng.random() < 0.6 else AluExp.cmpne)(sub(dt), sub(dt))
        if r < 0.6:
            return sub(BOOL).not_()
        if r < 0.8:
            return AluExp.cast(BOOL, sub(rng.choice([I32, U32, F32])))
        return (AluExp.add if rng.random() < 0.5 else AluExp.mul)(sub(BOOL), sub(BOOL))  # or / and
    if r < 0.12:
        return AluExp.where(sub(BOOL), sub(dtype), sub(dtype))
    if r < 0.22:
        src = rng.choice([d for d in (F32, I32, U32, BOOL) if d != dtype])
        inner = sub(src)
        if src == F32 and dtype != F32:
            inner = AluExp.mul(inner, AluExp.f32(rng.choice([1.0, 1000.0, 3e9])))  # exercise saturation too
        return AluExp.cast(dtype, inner)
    if dtype == F32:
        if r < 0.5:
            return rng.choice([AluExp.add, AluExp.sub, AluExp.mul])(sub(F32), sub(F32))
        if r < 0.6:
            return (AluExp.min if rng.random() < 0.5 else AluExp.max)(sub(F32), sub(F32))
        if r < 0.68:
            return AluExp.mul(sub(F32), AluExp.reciprocal(AluExp.add(AluExp.mul(sub(F32), sub(F32)), AluExp.f32(1.0))))
        if r < 0.76:
            return AluExp.sqrt(AluExp.add(AluExp.mul(sub(F32), sub(F32)), AluExp.f32(0.25)))
        if r < 0.84:
            return rng.choice([AluExp.floor, AluExp.ceil])(sub(F32))
        if r < 0.92:  # transcendentals of a bounded argument
            bounded = AluExp.min(AluExp.max(sub(F32), AluExp.f32(-4.0)), AluExp.f32(4.0))
            return rng.choice([AluExp.exp, AluExp.sin, AluExp.cos, AluExp.atan, AluExp.erf])(bounded)
        return AluExp.bitcast(F32, AluExp.bitCombine(AluExp.bitcast(U32, sub(F32)), AluExp.u32(0x7fffffff), "and"))  # |x|
    # integer kinds
    k = AluExp.i32 if dtype == I32 else AluExp.u32
    if r < 0.5:
        return rng.choice([AluExp.add, AluExp.sub, AluExp.mul])(sub(dtype), sub(dtype))
    if r < 0.62:
        return (AluExp.min if rng.random() < 0.5 else AluExp.max)(sub(dtype), sub(dtype))
    if r < 0.74:  # division by a non-zero constant or by (x | 1)
        den = k(rng.choice([1, 2, 3, 7, 10, 255])) if rng.random() < 0.6 else AluExp.bitCombine(sub(dtype), k(1), "or")
        if dtype == I32 and den.op != AluOp.Const:
            den = AluExp.max(den, k(1))  # avoid INT_MIN / -1
        num = sub(dtype)
        if den.op == AluOp.Const and num.op in (AluOp.Mul, AluOp.Add):
            # The reference's simplifier folds (x * A) / B and (x * A + y) / B as index algebra, without regard to
            # wrap-around (src/alu.ts:795-840); the checker evaluates the unsimplified expression.  Data expressions
            # that overflow there are outside what the two agree on (test_parity_gpu covers the fold itself).
            den = AluExp.max(AluExp.bitCombine(num, k(1), "or"), k(1))
        return (AluExp.idiv if rng.random() < 0.5 else AluExp.mod)(num, den)
    if r < 0.86:
        return AluExp.bitCombine(sub(dtype), sub(dtype), rng.choice(["and", "or", "xor"]))
    return AluExp.bitShift(sub(dtype), k(rng.choice([0, 1, 5, 13, 31])), rng.choice(["shl", "shr"]))


def make_inputs(rng, n):
    npr = np.random.default_rng(rng.randrange(1 << 30))
    f = npr.normal(0, 2, n).astype(np.float32)
    f[npr.integers(0, n, max(n // 40, 1))] = 0.0
    i = npr.integers(-1000, 1000, n).astype(np.int32)
    i[npr.integers(0, n, 4)] = [0x7fffffff, -0x80000000, -1, 0]
    u = npr.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    b = npr.integers(0, 2, n).astype(np.int32)
    return [(F32, f), (I32, i), (U32, u), (BOOL, b)]


def leaves_for(views):
    out = {}
    for v in views:
        out.setdefault(v.dtype, []).append(v)
    return out


@pytest.mark.parametrize("seed", range(150))
def test_random_map_kernels(seed, numerics_mode):
    rng = random.Random(1000 + seed + OFFSET)
    n = rng.choice([1, 5, 64, 1000, 4099, 65536 + 3])
    inputs = make_inputs(rng, n)
    out_dt = rng.choice([F32, F32, I32, U32, BOOL])
    st = ShapeTracker.fromShape([n])
    if rng.random() < 0.3 and n > 1:
        st = st.flip([True])
    k = mapKernel([n], [(dt, st) for dt, _ in inputs], lambda *vs: rand_exp(rng, leaves_for(vs), out_dt, rng.choice([3, 4, 5])))
    arrays = [a for _, a in inputs]
    if out_dt == F32:
        assert_parity(k, arrays, rtol=1e-5, atol=1e-6)
    elif numerics_mode == "fast" and k.exp_raw.collect(lambda e: e.op in (AluOp.Exp, AluOp.Reciprocal)):
        # integers derived from exp / reciprocal values: see test_random_reductions
        from gpu_util import device_run
        from oracle import oracle
        got, ks = device_run(k, arrays)
        want = oracle.run_kernel(k, arrays, oracle.MODE_WASM)
        assert (got != want).mean() <= 0.02, f"class {ks.klass} {ks.info}"
    else:
        assert_parity(k, arrays, exact=True)


@pytest.mark.parametrize("seed", range(100))
def test_random_reductions(seed, numerics_mode):
    rng = random.Random(5000 + seed + OFFSET)
    rows, L = rng.choice([(1, 1000), (7, 129), (64, 64), (300, 33), (5, 4097), (1000, 8)])
    inputs = make_inputs(rng, rows * L)
    out_dt = rng.choice([F32, I32, U32, BOOL])
    op = rng.choice([AluOp.Add, AluOp.Max, AluOp.Min] + ([AluOp.Mul] if out_dt in (I32, U32, BOOL) else []))
    if rng.random() < 0.5:
        st = ShapeTracker.fromShape([rows, L])
    else:
        st = ShapeTracker.fromShape([L, rows]).permute([1, 0])  # reduce axis strided in memory
    depth = rng.choice([2, 3])
    k = reduceKernel([rows, L], [(dt, st) for dt, _ in inputs], lambda *vs: rand_exp(rng, leaves_for(vs), out_dt, depth), op,
                     epilogue=(lambda acc: AluExp.add(acc, AluExp.const(out_dt, 1))) if out_dt in (I32, U32, F32) and rng.random() < 0.5 else None)
    arrays = [a for _, a in inputs]
    if numerics_mode == "fast" and out_dt != F32 and k.exp_raw.collect(lambda e: e.op in (AluOp.Exp, AluOp.Reciprocal)):
        # An integer or bool result computed THROUGH exp or reciprocal (a cast or a comparison of their value): the fast
        # mode's results differ from the polynomial forms in the sixth digit, so a term that sits on a rounding or
        # comparison boundary may come out one apart.  Bit-exactness is the contract for integer arithmetic, not for
        # integers derived from transcendentals; such kernels are held to "few terms differ, each by little" here and
        # to exactness in the wasm run of this same seed.
        from gpu_util import device_run
        from oracle import oracle
        got, ks = device_run(k, arrays)
        want = oracle.run_kernel(k, arrays, oracle.MODE_WASM)
        d = (got.astype(np.int64) - want.astype(np.int64) + (1 << 31)) % (1 << 32) - (1 << 31)  # difference modulo 2^32
        if op in (AluOp.Add, AluOp.Max, AluOp.Min):
            assert np.abs(d).max() <= max(1, L // 50) and (d != 0).mean() <= 0.25, f"class {ks.klass} {ks.info}: {got} vs {want}"
        return
    if out_dt == F32:
        if op == AluOp.Add:
            # plus a few float32 rounding units of sum |term| (far inside the K-scaled bound L * 2^-24 * sum |term|): the
            # integer inputs hold +-2^31, which cancel in some rows and leave an error of that order whatever the order
            from jaxjs_hip.alu import Kernel, Reduction
            from oracle import oracle
            e = k.exp_raw
            mag = Kernel(k.nargs, k.size, AluExp.where(AluExp.cmplt(e, AluExp.f32(0.0)), AluExp.sub(AluExp.f32(0.0), e), e), Reduction(F32, AluOp.Add, L))
            total = np.nan_to_num(oracle.run_kernel(mag, arrays, oracle.MODE_CPU).astype(np.float64), nan=0.0, posinf=0.0)
            from gpu_util import device_run
            got, ks = device_run(k, arrays)
            want = oracle.run_kernel(k, arrays, oracle.MODE_WASM)
            assert got.dtype == want.dtype and got.shape == want.shape and np.array_equal(np.isnan(got), np.isnan(want))
            bound = 1e-4 * L + 8.0 * 2.0 ** -24 * total + 2e-5 * max(1.0, math.sqrt(L)) * np.abs(want.astype(np.float64))
            ok = np.isnan(want) | (got == want) | (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= bound)
            assert ok.all(), f"class {ks.klass} {ks.info}: {np.flatnonzero(~ok)[:5]} {got[~ok][:5]} vs {want[~ok][:5]}"
        else:
            assert_parity(k, arrays, rtol=1e-5, atol=1e-6)
    else:
        assert_parity(k, arrays, exact=True)


def _random_view(rng):
    """A random chain of movement ops on an int32 base array; returns (tracker, base, numpy view)."""
    shape = [rng.choice([1, 2, 3, 8, 17, 40]) for _ in range(rng.choice([1, 2, 3]))]
    base = np.arange(1, int(np.prod(shape)) + 1, dtype=np.int32)
    ref = base.reshape(shape)
    st = ShapeTracker.fromShape(shape)
    for _ in range(rng.choice([1, 2, 3, 4, 5])):
        op = rng.choice(["permute", "flip", "pad", "shrink", "reshape", "expand"])
        nd = ref.ndim
        if op == "permute":
            perm = list(range(nd))
            rng.shuffle(perm)
            st, ref = st.permute(perm), ref.transpose(perm)
        elif op == "flip":
            fl = [rng.random() < 0.5 for _ in range(nd)]
            st = st.flip(fl)
            ref = ref[tuple(slice(None, None, -1) if f else slice(None) for f in fl)]
        elif op == "pad":
            pads = [(rng.choice([0, 1, 3]), rng.choice([0, 2])) for _ in range(nd)]
            st, ref = st.pad(pads), np.pad(ref, pads)
        elif op == "shrink":
            arg = []
            for s in ref.shape:
                b = rng.randrange(0, s)
                arg.append((b, rng.randrange(b + 1, s + 1)))
            st = st.shrink(arg)
            ref = ref[tuple(slice(b, e) for b, e in arg)]
        elif op == "reshape":
            n = ref.size
            divs = [d for d in range(1, n + 1) if n % d == 0]
            a = rng.choice(divs)
            new = [a, n // a] if rng.random() < 0.7 else [n]
            st, ref = st.reshape(new), ref.reshape(new)
        elif op == "expand" and ref.size < 20000:
            k = rng.choice([1, 2, 5])
            st = st.reshape([1] + list(ref.shape)).expand([k] + list(ref.shape))
            ref = np.broadcast_to(ref.reshape((1,) + ref.shape), (k,) + ref.shape)
    return st, base, np.ascontiguousarray(ref)


@pytest.mark.parametrize("seed", range(80))
def test_random_view_chains_in_maps_and_reductions(seed):
    """Movement ops are pure index arithmetic (multi-view trackers, masks, negative strides): the GPU result must
    equal numpy's on the same chain, bit for bit, as an elementwise kernel and under a row reduction."""
    rng = random.Random(9000 + seed + OFFSET)
    st, base, ref = _random_view(rng)
    shape = list(st.shape)
    k = mapKernel(shape, [(I32, st)], lambda v: AluExp.add(AluExp.mul(v, AluExp.i32(3)), AluExp.i32(1)))
    got, _, _ = assert_parity(k, [base], exact=True)
    np.testing.assert_array_equal(got.reshape(ref.shape), ref * 3 + 1)
    if len(shape) >= 1 and shape[-1] >= 1:
        op = rng.choice([AluOp.Add, AluOp.Max, AluOp.Min])
        kr = reduceKernel(shape, [(I32, st)], lambda v: v, op)
        got, _, _ = assert_parity(kr, [base], exact=True)
        want = {AluOp.Add: ref.sum(-1, dtype=np.int64).astype(np.int32), AluOp.Max: ref.max(-1), AluOp.Min: ref.min(-1)}[op]
        np.testing.assert_array_equal(got.reshape(want.shape), want)


@pytest.mark.parametrize("seed", range(60))
def test_random_contractions(seed):
    """Random contraction shapes and operand layouts (either operand stored k-major or row-major, optional batch
    axis shared or broadcast, optional fused bias/cast epilogue) with small integer data: every class the tuner may
    pick (direct-LDS / general / f32 GEMM, swapped roles, or a plain reduction for thin shapes) must be exact."""
    from jaxjs_hip.lowering import reduceKernel as rk
    rng = random.Random(7000 + seed + OFFSET)
    dim = lambda: rng.choice([1, 8, 31] if rng.random() < 0.15 else [64, 100, 128, 160, 256, 300, 512])  # noqa: E731
    M, N = dim(), dim()
    K = rng.choice([8, 32, 40, 64, 96, 128, 136, 512])
    batch = rng.choice([[], [], [3], [2, 2]])
    dt, npdt = rng.choice([(DType.Float16, np.float16), (DType.Float32, np.float32)])
    npr = np.random.default_rng(seed + OFFSET)
    full = batch + [M, N, K]
    nb = len(batch)
    a_t, b_t = rng.random() < 0.3, rng.random() < 0.5
    b_shared = bool(batch) and rng.random() < 0.4
    lim = 2 if dt == DType.Float16 else 3  # |sum| <= lim^2 * K stays exactly representable in the output type
    A = npr.integers(-lim, lim + 1, batch + ([K, M] if a_t else [M, K])).astype(npdt)
    B = npr.integers(-lim, lim + 1, ([] if b_shared else batch) + ([N, K] if b_t else [K, N])).astype(npdt)
    stA = ShapeTracker.fromShape(list(A.shape))
    if a_t:
        stA = stA.permute(list(range(nb)) + [nb + 1, nb])
    stA = stA.reshape(batch + [M, 1, K]).expand(full)
    stB = ShapeTracker.fromShape(list(B.shape))
    if not b_t:
        off = 0 if b_shared else nb
        stB = stB.permute(list(range(off)) + [off + 1, off])
    stB = stB.reshape(([1] * nb if b_shared else batch) + [1, N, K]).expand(full)
    with_bias = rng.random() < 0.4
    bias = npr.integers(-5, 6, [N]).astype(npdt)
    inputs = [(dt, stA), (dt, stB)]
    epilogue = None
    if with_bias:
        from jaxjs_hip import AluVar
        from jaxjs_hip.shape import unravelAlu
        def epilogue(acc):
            n_idx = unravelAlu(batch + [M, N], AluVar.gidx)[-1]
            return AluExp.add(acc, AluExp.globalIndex(dt, 2, N, n_idx))
    k = rk(full, inputs, lambda a, b: AluExp.mul(a, b), AluOp.Add, epilogue=epilogue)
    arrays = [A, B] + ([bias] if with_bias else [])
    if with_bias:
        from jaxjs_hip import Kernel
        k = Kernel(3, k.size, k.exp_raw, k.reduction)
    got, want, ks = assert_parity(k, arrays, exact=True)
    Am = A.astype(np.float64)
    Bm = B.astype(np.float64)
    if a_t:
        Am = np.swapaxes(Am, -1, -2)
    if b_t:
        Bm = np.swapaxes(Bm, -1, -2)
    ref = Am @ Bm + (bias.astype(np.float64) if with_bias else 0)
    np.testing.assert_array_equal(got.astype(np.float64).reshape(ref.shape), ref.astype(npdt).astype(np.float64), err_msg=str(ks.info))


# ---- float16 -----------------------------------------------------------------------------------------------------
F16 = DType.Float16


def rand_f16_exp(rng, leaves, depth):
    """A random float16 expression: every operation rounds to float16 (as the reference's float16 arrays do), so the
    GPU's native half arithmetic and the checker agree bit for bit except where a transcendental or a division is
    involved (one float16 ulp); magnitudes stay small enough that nothing overflows."""
    if depth == 0 or rng.random() < 0.2:
        if rng.random() < 0.8:
            return rng.choice(leaves[F16])
        return AluExp.const(F16, rng.choice([0.0, 1.0, -1.0, 0.5, 2.0, -0.75]))
    sub = lambda: rand_f16_exp(rng, leaves, depth - 1)  # noqa: E731
    r = rng.random()
    if r < 0.4:
        return rng.choice([AluExp.add, AluExp.sub, AluExp.mul])(sub(), sub())
    if r < 0.5:
        return (AluExp.min if rng.random() < 0.5 else AluExp.max)(sub(), sub())
    if r < 0.6:
        return AluExp.where(AluExp.cmplt(sub(), sub()), sub(), sub())
    bounded = AluExp.min(AluExp.max(sub(), AluExp.const(F16, -3.0)), AluExp.const(F16, 3.0))
    if r < 0.7:
        return AluExp.exp(bounded)
    if r < 0.78:
        return AluExp.log(AluExp.add(AluExp.mul(bounded, bounded), AluExp.const(F16, 0.5)))
    if r < 0.86:
        return AluExp.sqrt(AluExp.add(AluExp.mul(bounded, bounded), AluExp.const(F16, 0.25)))
    if r < 0.93:
        return AluExp.reciprocal(AluExp.add(AluExp.mul(bounded, bounded), AluExp.const(F16, 1.0)))
    if r < 0.97:
        return AluExp.cast(F16, AluExp.mul(AluExp.cast(F32, bounded), rng.choice(leaves[F32])))
    return AluExp.cast(F16, AluExp.cast(I32, AluExp.mul(bounded, AluExp.const(F16, 4.0))))


@pytest.mark.parametrize("seed", range(60))
def test_random_f16_kernels(seed, numerics_mode):
    """Maps and reductions over float16 buffers (packs of 8 halves, f32 accumulation of f16 sums, native half
    arithmetic) against the checker, within the float16 tolerance (rel 1e-2)."""
    rng = random.Random(9000 + seed + OFFSET)
    npr = np.random.default_rng(seed + OFFSET)
    reduce_ = seed % 3 == 2
    if reduce_:
        rows, L = rng.choice([(1, 1000), (7, 129), (64, 64), (300, 33), (5, 2049)])
        n = rows * L
        st = ShapeTracker.fromShape([rows, L]) if rng.random() < 0.5 else ShapeTracker.fromShape([L, rows]).permute([1, 0])
    else:
        n = rng.choice([1, 7, 64, 1000, 4099, 65536 + 5])
        st = ShapeTracker.fromShape([n])
        if rng.random() < 0.3 and n > 1:
            st = st.flip([True])
    h1, h2 = (npr.normal(0, 1.5, n).astype(np.float16) for _ in range(2))
    f = npr.uniform(-2, 2, n).astype(np.float32)
    ins = [(F16, st), (F16, st), (F32, st)]
    body = lambda *vs: rand_f16_exp(rng, {F16: list(vs[:2]), F32: [vs[2]]}, rng.choice([2, 3, 4]))  # noqa: E731
    if reduce_:
        op = rng.choice([AluOp.Add, AluOp.Max, AluOp.Min])
        k = reduceKernel([rows, L], ins, body, op)
        tol = dict(rtol=1e-2, atol=1e-2 * (math.sqrt(L) if op == AluOp.Add else 1.0))
    else:
        k = mapKernel([n], ins, body)
        tol = dict(rtol=1e-2, atol=1e-2)
    assert k.dtype == F16
    assert_parity(k, [h1, h2, f], **tol)
