"""Library compositions over the tracing primitives, restating how the reference's numpy/nn/lax
layers spell the operations the benchmark configurations use -- the spelling decides which Kernels
the backend is handed, so it is kept literally:

  square, sigmoid, tanh, gelu, softmax, standardize   src/library/numpy.ts:2579-2582, 3054-3060;
                                                      src/library/nn.ts:65-67, 222-238, 291-301, 386-412
  lax.dot / matmul / two-operand einsum               src/library/lax.ts:40-129; numpy.ts:1729-1747, 1935-1990
  arange / tri (lazy constants)                       src/frontend/array.ts:1570-1627
  argmax                                              src/library/numpy.ts:533-556
  dotProductAttention                                 src/library/nn.ts:478-583
  sort / argsort along an axis                        src/frontend/core.ts:1043-1075
  linalg: cholesky, triangularSolve, solve            src/library/lax-linalg.ts:35-50, 212-244; numpy-linalg.ts:274-318
  eigh (unsorted), fft along an axis                  src/library/lax-linalg.ts:52-100; numpy-fft.ts:50-66, 126-157
  stack, take, takeAlongAxis, absolute, clip, log1p   src/library/numpy.ts:971-985, 1493-1567, 2433-2452, 2854-2884
  random: bits, split, uniform, exponential, normal   src/library/random.ts:53-135, 350-356, 511-525
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

from . import jit as J
from .alu import AluExp, AluOp, AluVar, DType
from .jit import ConstArray, Tracer
from .shape import prod as _int_prod, unravelAlu


def square(x):
    return J.mul(x, x)


def sigmoid(x):
    return J.reciprocal(J.exp(J.neg(x)).add(1))


def tanh(x):
    """(e^{-2|x|} - 1) / (e^{-2|x|} + 1) * negsgn, avoiding overflow (numpy.ts:3054-3060)."""
    negsgn = J.where(J.less(x, 0), 1, -1)
    en2x = J.exp(x.mul(negsgn).mul(2))
    return en2x.sub(1).div(en2x.add(1)).mul(negsgn)


def gelu(x, approximate: bool = True):
    if approximate:
        c = math.sqrt(2 / math.pi)
        return x.mul(0.5).mul(tanh(x.mul(x.mul(x).mul(0.044715).add(1)).mul(c)).add(1))
    return x.mul(0.5).mul(J.erfc(J.neg(x.mul(math.sqrt(0.5)))))


def softmax(x, axis: int = -1):
    xMax = x.max(axis, keepdims=True)
    unnormalized = J.exp(x.sub(J.stopGradient(xMax)))
    return unnormalized.div(unnormalized.sum(axis, keepdims=True))


def standardize(x, axis: int = -1, epsilon: float = 1e-5):
    """Var[X] = E[X^2] - E[X]^2, like the reference (nn.ts:386-412)."""
    mu = x.mean(axis, keepdims=True)
    sigma2 = square(x).mean(axis, keepdims=True).sub(square(mu))
    return x.sub(mu).div(J.sqrt(sigma2.add(epsilon)))


def lax_dot(lhs: Tracer, rhs: Tracer, lc: Sequence[int], rc: Sequence[int], lb: Sequence[int] = (), rb: Sequence[int] = ()):
    """General contraction: transpose to [batch, free, contract], reshape so the free axes of the two
    operands interleave as size-1 axes, then one `Dot` (lax.ts:40-129)."""
    norm = lambda ax, n: [a + n if a < 0 else a for a in ax]
    lc, lb = norm(lc, lhs.ndim), norm(lb, lhs.ndim)
    rc, rb = norm(rc, rhs.ndim), norm(rb, rhs.ndim)
    lf = [a for a in range(lhs.ndim) if a not in lc and a not in lb]
    rf = [a for a in range(rhs.ndim) if a not in rc and a not in rb]
    lhs2 = lhs.transpose(lb + lf + lc)
    rhs2 = rhs.transpose(rb + rf + rc)
    if not lc:
        return J.mul(lhs2.reshape([lhs.shape[a] for a in lb] + [lhs.shape[a] for a in lf] + [1] * len(rf)),
                     rhs2.reshape([rhs.shape[a] for a in rb] + [1] * len(lf) + [rhs.shape[a] for a in rf]))
    kx, ky = [lhs.shape[a] for a in lc], [rhs.shape[a] for a in rc]
    if kx != ky:
        raise ValueError(f"dot: shapes not aligned along contracting dims: {kx} != {ky}")
    return J.dot(
        lhs2.reshape([lhs.shape[a] for a in lb] + [lhs.shape[a] for a in lf] + [1] * len(rf) + [_int_prod(kx)]),
        rhs2.reshape([rhs.shape[a] for a in rb] + [1] * len(lf) + [rhs.shape[a] for a in rf] + [_int_prod(ky)]))


def matmul(x: Tracer, y: Tracer):
    if y.ndim == 1:
        return J.dot(x, y)
    nb = min(max(x.ndim, 2), y.ndim) - 2
    batch = list(range(-2 - nb, -2))
    return lax_dot(x, y, [-1], [-2], batch, batch)


def einsum(subscripts: str, a: Tracer, b: Tracer):
    """Two-operand einsum without repeated or summed-alone indices: batch = shared kept indices,
    contraction = shared dropped indices, then a transpose to the requested order
    (numpy.ts:1935-1990)."""
    lhs, out = subscripts.replace(" ", "").split("->")
    ia, ib = lhs.split(",")
    if len(set(ia)) != len(ia) or len(set(ib)) != len(ib):
        raise NotImplementedError("einsum: repeated indices")
    reduced = [c for c in ia if c in ib and c not in out]
    if any((c not in out) and not (c in ia and c in ib) for c in ia + ib):
        raise NotImplementedError("einsum: index summed over a single operand")
    batch = [c for c in ia if c in ib and c not in reduced]
    res = lax_dot(a, b, [ia.index(c) for c in reduced], [ib.index(c) for c in reduced],
                  [ia.index(c) for c in batch], [ib.index(c) for c in batch])
    order = batch + [c for c in ia if c not in ib] + [c for c in ib if c not in ia]
    return res.transpose([order.index(c) for c in out])


def padtypeToPads(inShape, filterShape, strides, dilation, padding: str):
    """"VALID" / "SAME" / "SAME_LOWER" to explicit pads (src/library/lax.ts:133-165)."""
    kind = padding.upper()
    if kind == "VALID":
        return [(0, 0)] * len(inShape)
    if kind not in ("SAME", "SAME_LOWER"):
        raise ValueError(f"Unknown padding type: {kind}")
    out = [-(-size // s) for size, s in zip(inShape, strides)]
    sizes = [max(0, (o - 1) * s + 1 + (k - 1) * d - i) for o, s, k, d, i in zip(out, strides, filterShape, dilation, inShape)]
    if kind == "SAME":
        return [(sz >> 1, sz - (sz >> 1)) for sz in sizes]
    return [(sz - (sz >> 1), sz >> 1) for sz in sizes]


def convGeneralDilated(lhs: Tracer, rhs: Tracer, windowStrides: Sequence[int], padding, lhsDilation=None, rhsDilation=None):
    """`lax.conv_general_dilated` with one feature group: lhs `[N, C, *xs]`, rhs `[O, C, *ks]` (lax.ts:268-343)."""
    n = lhs.ndim - 2
    rd = list(rhsDilation) if rhsDilation is not None else [1] * n
    ld = list(lhsDilation) if lhsDilation is not None else [1] * n
    if isinstance(padding, str):
        if any(d != 1 for d in ld):
            raise ValueError("String padding is not supported for transposed convolutions")
        padding = padtypeToPads(lhs.shape[2:], rhs.shape[2:], windowStrides, rd, padding)
    from .convolution import ConvParams
    return J.conv(lhs, rhs, ConvParams(0, list(windowStrides), [tuple(p) for p in padding], ld, rd))


def reduceWindow(x: Tracer, op: AluOp, window: Sequence[int], strides: Optional[Sequence[int]] = None):
    """`lax.reduceWindow` for a plain reduction: Pool view, then reduce the window axes (lax.ts:479-502)."""
    strides = list(strides) if strides is not None else [1] * len(window)
    p = J.poolWindows(x, window, strides)
    return J.reduce(p, op, list(range(p.ndim - len(window), p.ndim)))


def arange_const(start: int, stop: int, step: int = 1, dtype: DType = DType.Int32, shape: Optional[Sequence[int]] = None) -> ConstArray:
    """`arange(...)` (optionally reshaped): start + cast(idx)*step, realised by a nullary kernel."""
    size = max(0, -(-(stop - start) // step)) if step > 0 else max(0, -((start - stop) // step))
    exp = AluExp.add(AluExp.const(dtype, start), AluExp.mul(AluExp.cast(dtype, AluVar.gidx), AluExp.const(dtype, step)))
    return ConstArray(tuple(shape) if shape is not None else (size,), dtype, exp)


def tri_const(n: int, m: Optional[int] = None, k: int = 0) -> ConstArray:
    """Boolean lower-triangular mask `rows.reshape([n,1]) >= cols` (array.ts:1614-1627)."""
    m = n if m is None else m
    r, c = unravelAlu([n, m], AluVar.gidx)
    rows = AluExp.add(AluExp.i32(k), AluExp.mul(AluExp.cast(DType.Int32, r), AluExp.i32(1)))
    cols = AluExp.add(AluExp.i32(0), AluExp.mul(AluExp.cast(DType.Int32, c), AluExp.i32(1)))
    return ConstArray((n, m), DType.Bool, J.aluCompare(cols, rows, "LessEqual"))


def argmax(a: Tracer, axis: int):
    """First index of the maximum: max over isMax * (length - i), then length - that (numpy.ts:533-556)."""
    axis = axis + a.ndim if axis < 0 else axis
    n = a.shape[axis]
    isMax = J.equal(a, a.max(axis, keepdims=True))
    length = J.scalar(n, DType.Int32)
    rev = arange_const(n, 0, -1, DType.Int32, shape=[n] + [1] * (a.ndim - axis - 1))
    idx = isMax.astype(DType.Int32).mul(rev)
    return length.sub(idx.max(axis))


def argmin(a: Tracer, axis: int):
    """First index of the minimum: the same construction on `a == min(a)` (numpy.ts:497-524)."""
    axis = axis + a.ndim if axis < 0 else axis
    n = a.shape[axis]
    isMin = J.equal(a, a.min(axis, keepdims=True))
    length = J.scalar(n, DType.Int32)
    rev = arange_const(n, 0, -1, DType.Int32, shape=[n] + [1] * (a.ndim - axis - 1))
    idx = isMin.astype(DType.Int32).mul(rev)
    return length.sub(idx.max(axis))


def logsumexp(x: Tracer, axis=None, keepdims: bool = False):
    """max + log(sum(exp(x - max))) (nn.ts:332-345)."""
    xMax = x.max(axis, keepdims=True)
    shifted = x.sub(xMax)
    result = xMax.add(J.log(J.exp(shifted).sum(axis, keepdims=True)))
    if keepdims:
        return result
    ax = J._normalize_axis(axis, x.ndim)
    return result.reshape([n for i, n in enumerate(x.shape) if i not in ax])


def dotProductAttention(query: Tracer, key: Tracer, value: Tracer, isCausal: bool = False, scale: Optional[float] = None,
                        fused: bool = False):
    """[B,L,N,H] attention with equal query and key/value head counts (nn.ts:478-583).  `fused=True` hands the whole
    chain to the backend as one `Attention` routine when the shapes fit its kernel (float16, head size 64, L a multiple
    of 128, S of 64) -- a front-end switch the reference does not have; otherwise the reference's composition is
    traced."""
    B, L, N, H = query.shape
    S = key.shape[1]
    if key.shape != value.shape or key.shape[0] != B or key.shape[3] != H or key.shape[2] != N:
        raise ValueError("dotProductAttention: shape mismatch")
    scale = 1 / math.sqrt(H) if scale is None else scale
    if (fused and H == 64 and L % 128 == 0 and S % 64 == 0
            and all(t.dtype == DType.Float16 for t in (query, key, value))):
        return J.attention(query, key, value, scale, isCausal)
    scores = einsum("BLNH,BSNH->BNLS", query, key).mul(scale)
    if isCausal:
        scores = J.where(tri_const(L, S, 0), scores, -math.inf)
    attn = softmax(scores, -1)
    return einsum("BNLS,BSNH->BLNH", attn, value)


def _axis_to_last(ndim: int, axis: int):
    axis = axis + ndim if axis < 0 else axis
    perm = [d for d in range(ndim) if d != axis] + [axis]
    inv = [perm.index(d) for d in range(ndim)]
    return axis, perm, inv


def sort(a: Tracer, axis: int = -1):
    """Sort along `axis`: the routine sorts the last axis, other axes are moved there and back."""
    axis, perm, inv = _axis_to_last(a.ndim, axis)
    if a.shape[axis] <= 1:
        return a
    if axis == a.ndim - 1:
        return J.sort(a)
    return J.sort(a.transpose(perm)).transpose(inv)


def argsort(a: Tracer, axis: int = -1):
    axis, perm, inv = _axis_to_last(a.ndim, axis)
    if axis == a.ndim - 1:
        return J.argsort(a)[1]
    return J.argsort(a.transpose(perm))[1].transpose(inv)


def _swap_last_two(x: Tracer):
    return x.transpose(list(range(x.ndim - 2)) + [x.ndim - 1, x.ndim - 2])


def cholesky(a: Tracer, upper: bool = False):
    L = J.cholesky(a)
    return _swap_last_two(L) if upper else L


def triangularSolve(a: Tracer, b: Tracer, leftSide: bool = False, lower: bool = False, transposeA: bool = False,
                    unitDiagonal: bool = False):
    """`a @ x = b` (leftSide) or `x @ a = b`: reduced to the primitive's `a @ x.T = b.T` by transposes."""
    if not leftSide:
        transposeA = not transposeA
    else:
        b = _swap_last_two(b)
    if transposeA:
        a = _swap_last_two(a)
        lower = not lower
    x = J.triangularSolve(a, b, lower=lower, unitDiagonal=unitDiagonal)
    return _swap_last_two(x) if leftSide else x


def solve(a: Tracer, b: Tracer):
    """`numpy.linalg.solve` for equal batch dimensions: LU with partial pivoting, the permutation applied as a 0/1
    matrix product, then a unit-lower and an upper triangular solve."""
    n = a.shape[-1]
    if a.ndim < 2 or a.shape[-2] != n:
        raise ValueError(f"solve: a must be a batch of square matrices, got {a.shape}")
    b_is_1d = b.ndim == 1
    if b_is_1d:
        b = b.reshape(list(b.shape) + [1])
    if b.shape[-2] != n or tuple(a.shape[:-2]) != tuple(b.shape[:-2]):
        raise ValueError(f"solve: leading dimension of b must match size of a, got a={a.shape}, b={b.shape}")
    lu, _pivots, permutation = J.lu(a)
    P = J.equal(arange_const(0, n), permutation.reshape(list(permutation.shape) + [1])).astype(b.dtype)
    LPb = triangularSolve(lu, matmul(P, b), leftSide=True, lower=True, unitDiagonal=True)
    x = triangularSolve(lu, LPb, leftSide=True, lower=False)
    return x.reshape(list(x.shape[:-1])) if b_is_1d else x


def eigh_unsorted(x: Tracer, symmetrizeInput: bool = True):
    """Eigenvectors (columns) and the diagonalised matrix, without the final sort by eigenvalue (which is a
    gather in the reference); sweep count and tolerance as in the reference's wrapper."""
    n = x.shape[-1]
    if symmetrizeInput:
        x = x.add(_swap_last_two(x)).mul(0.5)
    d, v = J.jacobiEigh(x, maxSweeps=max(8, 2 * n), tolerance=1e-6)
    return v, d


def diagonal(x: Tracer, offset: int = 0, axis1: int = 0, axis2: int = 1):
    """The diagonal as a view, appended as the last axis: move the two axes last, flatten them, pad or shrink to
    `diag * (m + 1)` elements, reshape to `[diag, m + 1]` and keep column `offset` (src/frontend/core.ts:958-1000)."""
    if offset < 0:
        return diagonal(x, -offset, axis2, axis1)
    axis1, axis2 = (a + x.ndim if a < 0 else a for a in (axis1, axis2))
    if axis1 == axis2:
        raise ValueError("axis1 and axis2 must not be equal")
    if offset >= x.shape[axis2]:
        raise ValueError("offset exceeds axis size")
    if (axis1, axis2) != (x.ndim - 2, x.ndim - 1):
        x = x.transpose([i for i in range(x.ndim) if i not in (axis1, axis2)] + [axis1, axis2])
    batch = list(x.shape[:-2])
    n, m = x.shape[-2:]
    diag = min(n, m - offset)
    x = x.reshape(batch + [n * m])
    npad = diag * (m + 1) - n * m
    if npad > 0:
        x = J.pad(x, [(0, 0)] * len(batch) + [(0, npad)])
    elif npad < 0:
        x = J.shrink(x, [(0, d) for d in batch] + [(0, n * m + npad)])
    x = x.reshape(batch + [diag, m + 1])
    return J.shrink(x, [(0, d) for d in batch + [diag]] + [(offset, offset + 1)]).reshape(batch + [diag])


def eigh(x: Tracer, lower: bool = True, sortEigenvalues: bool = True, symmetrizeInput: bool = True):
    """`(eigenvectors, eigenvalues)` of a batch of symmetric matrices, eigenvalues ascending: the Jacobi routine, then
    argsort of the diagonal and two gathers (src/library/lax-linalg.ts:52-89)."""
    n = x.shape[-1]
    if x.ndim < 2 or x.shape[-2] != n:
        raise ValueError(f"eigh: expected a batch of square matrices, got {list(x.shape)}")
    if symmetrizeInput:
        x = x.add(_swap_last_two(x)).mul(0.5)
    elif not lower:
        x = _swap_last_two(x)
    d, v = J.jacobiEigh(x, maxSweeps=max(8, 2 * n), tolerance=1e-6)
    values = diagonal(d, 0, -2, -1)
    if not sortEigenvalues:
        return v, values
    order = argsort(values)
    return takeAlongAxis(v, order.reshape(list(x.shape[:-2]) + [1, n]), -1), takeAlongAxis(values, order, -1)


def svd(a: Tracer, computeUv: bool = True, fullMatrices: bool = False):
    """Thin singular value decomposition through the symmetric eigendecomposition of the smaller Gram matrix
    (src/library/lax-linalg.ts:102-163): `s = sqrt(max(flip(eigenvalues), 0))`, the other factor from one more product
    scaled by `1/s` (0 where s is 0)."""
    if a.ndim < 2:
        raise ValueError(f"svd: input must be at least 2D, got {list(a.shape)}")
    m, n = a.shape[-2:]
    if fullMatrices and m != n:
        raise ValueError("svd: fullMatrices=true is only supported for square input")
    batch, k = list(a.shape[:-2]), min(m, n)
    singular = lambda values: J.sqrt(J.maximum(J.flip(values, -1), 0.0))  # noqa: E731
    inverse = lambda s: J.where(J.greater(s, 0.0), J.reciprocal(s), 0.0)  # noqa: E731
    if m >= n:
        v, values = eigh(matmul(_swap_last_two(a), a), symmetrizeInput=False)
        s = singular(values)
        if not computeUv:
            return s
        vDesc = J.flip(v, -1)
        u = matmul(a, vDesc).mul(inverse(s).reshape(batch + [1, k]))
        return u, s, _swap_last_two(vDesc)
    u, values = eigh(matmul(a, _swap_last_two(a)), symmetrizeInput=False)
    s = singular(values)
    if not computeUv:
        return s
    uDesc = J.flip(u, -1)
    vh = matmul(_swap_last_two(uDesc), a).mul(inverse(s).reshape(batch + [k, 1]))
    return uDesc, s, vh


def svdvals(a: Tracer):
    return svd(a, computeUv=False)


def factorFftSize(n: int) -> List[int]:
    factors: List[int] = []
    for radix in (4, 2, 3, 5, 7):
        while n % radix == 0:
            factors.append(radix)
            n //= radix
    radix = 11
    while radix * radix <= n:
        while n % radix == 0:
            factors.append(radix)
            n //= radix
        radix += 2
    if n > 1:
        factors.append(n)
    return factors


def fft(real: Tracer, imag: Tracer, axis: int = -1, inverse: bool = False):
    axis, perm, inv = _axis_to_last(real.ndim, axis)
    n = real.shape[axis]
    if axis != real.ndim - 1:
        real, imag = real.transpose(perm), imag.transpose(perm)
    re, im = J.fft(real, imag, factorFftSize(n), inverse)
    if axis != real.ndim - 1:
        re, im = re.transpose(inv), im.transpose(inv)
    return re, im


def stack(xs: Sequence[Tracer], axis: int = 0):
    xs = [J._raise(x) for x in xs]
    if not xs:
        raise ValueError("Need at least one array to stack")
    if any(tuple(x.shape) != tuple(xs[0].shape) for x in xs):
        raise ValueError(f"Cannot stack arrays with different shapes: {[list(x.shape) for x in xs]}")
    nd = xs[0].ndim + 1
    axis = axis + nd if axis < 0 else axis
    newShape = list(xs[0].shape[:axis]) + [1] + list(xs[0].shape[axis:])
    return J.concatenate([x.reshape(newShape) for x in xs], axis)


def take(a: Tracer, indices: Tracer, axis: Optional[int] = None):
    if axis is None:
        a, axis = a.reshape([-1]), 0
    axis = axis + a.ndim if axis < 0 else axis
    return J.gather(a, [indices], [axis], axis)


def takeAlongAxis(a: Tracer, indices: Tracer, axis: int = -1):
    """One index array per axis: the given one on `axis`, aranges elsewhere, all broadcast to the output shape."""
    if a.ndim != indices.ndim:
        raise ValueError(f"takeAlongAxis: input and indices must have the same rank, got {list(a.shape)} and {list(indices.shape)}")
    axis = axis + a.ndim if axis < 0 else axis
    outShape = list(indices.shape)
    for i in range(a.ndim):
        if i == axis:
            continue
        if a.shape[i] != indices.shape[i] and a.shape[i] != 1 and indices.shape[i] != 1:
            raise ValueError(f"takeAlongAxis: non-axis dimensions must broadcast, got {list(a.shape)} and {list(indices.shape)}")
        outShape[i] = max(a.shape[i], indices.shape[i])
    coords = []
    for i in range(a.ndim):
        if i == axis:
            c = indices
        else:
            shape = [1] * a.ndim
            shape[i] = a.shape[i]
            c = J._raise(arange_const(0, a.shape[i], 1, DType.Int32, shape=shape))
        coords.append(J.broadcast(c, outShape, []) if list(c.shape) != outShape else c)
    return J.gather(a, coords, list(range(a.ndim)), 0)


def absolute(x: Tracer):
    return J.where(J.less(x, 0), x.mul(-1), x)


def clip(a: Tracer, lo=None, hi=None):
    if hi is not None:
        a = J.minimum(a, hi)
    if lo is not None:
        a = J.maximum(a, lo)
    return a


def log1p(x: Tracer):
    """Series through x^10 (Horner) for |x| <= 0.2, log(1 + x) elsewhere."""
    cutoff = 0.2
    useSeries = J.lessEqual(absolute(x), cutoff)
    sx = clip(x, -cutoff, cutoff)
    series = (sx.mul(-1 / 10).add(1 / 9).mul(sx).sub(1 / 8).mul(sx).add(1 / 7).mul(sx).sub(1 / 6).mul(sx).add(1 / 5).mul(sx)
              .sub(1 / 4).mul(sx).add(1 / 3).mul(sx).sub(1 / 2).mul(sx).add(1).mul(sx))
    return J.where(useSeries, series, J.log(x.add(1)))


def _key_halves(key: Tracer):
    if key.dtype != DType.Uint32 or key.ndim < 1 or key.shape[-1] != 2:
        raise ValueError(f"Invalid key shape: {list(key.shape)}. Expected last dimension to be 2 with uint32 type.")
    keyShape = list(key.shape[:-1])
    k0, k1 = J.split(key, -1, [1, 1])
    return k0.reshape(keyShape), k1.reshape(keyShape)


def random_bits(key: Tracer, shape: Sequence[int] = ()):
    k0, k1 = _key_halves(key)
    return J.randomBits(k0, k1, list(shape))


def random_split(key: Tracer, num=2):
    shape = [num] if isinstance(num, int) else list(num)
    if any(n <= 0 for n in shape):
        raise ValueError(f"Invalid split length: {shape}. Must be positive integers.")
    k0, k1 = _key_halves(key)
    return stack([J.randomBits(k0, k1, shape, 0), J.randomBits(k0, k1, shape, 1)], -1)


def random_uniform(key: Tracer, shape: Sequence[int] = (), minval: float = 0.0, maxval: float = 1.0):
    """23 random mantissa bits under the exponent of 1.0, minus 1: uniform in [0, 1)."""
    if minval >= maxval:
        raise ValueError(f"Invalid range: [{minval}, {maxval}).")
    mantissa = random_bits(key, shape).div(J.scalar(1 << 9, DType.Uint32))
    float12 = mantissa.add(J.scalar(0x3F800000, DType.Uint32))
    rand = J.bind1("Bitcast", [float12], dict(dtype=DType.Float32)).sub(1)
    if minval == 0 and maxval == 1:
        return rand
    return rand.mul(maxval - minval).add(minval)


def random_exponential(key: Tracer, shape: Sequence[int] = ()):
    return J.neg(log1p(J.neg(random_uniform(key, shape))))


def random_normal(key: Tracer, shape: Sequence[int] = ()):
    """Box-Muller, first variate only."""
    keys = random_split(key, 2)
    ka, kb = J.split(keys, 0, [1, 1])
    u1 = random_uniform(ka.reshape([2]), shape)
    u2 = random_uniform(kb.reshape([2]), shape)
    radius = J.sqrt(log1p(J.neg(u1)).mul(-2))
    theta = u2.mul(2 * math.pi)
    return radius.mul(J.bind1("Cos", [theta]))


# ---- reductions and scans of the numpy surface (src/library/numpy.ts) ---------------------------------

def prod(a: Tracer, axis=None, keepdims: bool = False):
    """Product over `axis` (numpy.ts:376-382): one Mul reduction."""
    return J.reduce(a, AluOp.Mul, axis, keepdims)


def any_(a: Tracer, axis=None, keepdims: bool = False):
    """`astype(bool).max(axis)` (core.ts:911-913)."""
    return J.reduce(J._raise(a).astype(DType.Bool), AluOp.Max, axis, keepdims)


def all_(a: Tracer, axis=None, keepdims: bool = False):
    """`astype(bool).min(axis)` (core.ts:906-908)."""
    return J.reduce(J._raise(a).astype(DType.Bool), AluOp.Min, axis, keepdims)


def ptp(a: Tracer, axis=None, keepdims: bool = False):
    """`max - min` (numpy.ts:431-438)."""
    return a.max(axis, keepdims).sub(a.min(axis, keepdims))


def countNonzero(a: Tracer, axis=None, keepdims: bool = False):
    """`sum(astype(a != 0, int32))` (numpy.ts:367-373)."""
    return J.notEqual(a, 0).astype(DType.Int32).sum(axis, keepdims)


def var_(x: Tracer, axis=None, keepdims: bool = False, correction: float = 0):
    """`sum(square(x - mean)) * 1/(n - correction)` with the mean kept as its own reduction (numpy.ts:3103-3121)."""
    ax = J._normalize_axis(axis, x.ndim)
    n = 1
    for a in ax:
        n *= x.shape[a]
    if n == 0:
        raise ValueError("var: cannot compute variance over zero-length axis")
    mu = x.mean(ax, keepdims=True)
    return square(x.sub(mu)).sum(ax, keepdims).mul(1 / (n - correction))


def std(x: Tracer, axis=None, keepdims: bool = False, correction: float = 0):
    return J.sqrt(var_(x, axis, keepdims, correction))


def average(a: Tracer, axis=None, weights: Optional[Tracer] = None, keepdims: bool = False):
    """Weighted mean `sum(a*w) / sum(w)`; weights of lower rank line up with `axis` (numpy.ts:456-489)."""
    if weights is None:
        return a.mean(axis, keepdims)
    ax = J._normalize_axis(axis, a.ndim)
    w = J._raise(weights)
    if tuple(w.shape) != tuple(a.shape):
        if w.ndim != len(ax) or any(w.shape[i] != a.shape[d] for i, d in enumerate(ax)):
            raise ValueError("average: weights must match the array or the reduced axes")
        shape = [a.shape[d] if d in ax else 1 for d in range(a.ndim)]
        w = w.reshape(shape)
    return a.mul(w).sum(ax, keepdims).div(J.broadcast(w, a.shape, []).sum(ax, keepdims) if tuple(w.shape) != tuple(a.shape) else w.sum(ax, keepdims))


def moveaxis(a: Tracer, src: int, dst: int):
    src = src + a.ndim if src < 0 else src
    dst = dst + a.ndim if dst < 0 else dst
    perm = [i for i in range(a.ndim) if i != src]
    perm.insert(dst, src)
    return a if perm == list(range(a.ndim)) else a.transpose(perm)


def _cumulative_quadratic(op: AluOp, a: Tracer, padValue, k: int = 0):
    """`reduce(where(tri(n, n, k), a[..., None, :], pad), op, -1)` (numpy.ts:562-575): n^2 work, one kernel."""
    n = a.shape[-1]
    wide = J.broadcast(a, list(a.shape) + [n], [a.ndim - 1])
    pad = J.scalar(padValue, a.dtype)
    return J.reduce(J.where(tri_const(n, n, k), wide, pad), op, -1)


def _cumulative(op: AluOp, a: Tracer, axis):
    """Scan along `axis`: quadratic up to 512 elements, else chunks of 256 scanned independently and offset by an
    exclusive scan of the chunk totals (numpy.ts:577-614)."""
    padValue = 0 if op == AluOp.Add else 1
    a = J._raise(a)
    if a.ndim == 0:
        a = a.reshape([1])
    if axis is None:
        a, axis = a.reshape([-1]), 0
    (axis,) = J._normalize_axis(axis, a.ndim)
    a = moveaxis(a, axis, -1)
    n = a.shape[-1]
    split = 256
    if n <= split * 2:
        return moveaxis(_cumulative_quadratic(op, a, padValue), -1, axis)
    batch = list(a.shape[:-1])
    m = -(-n // split)
    a = J.pad(a, [(0, 0)] * len(batch) + [(0, m * split - n)])
    scans = _cumulative_quadratic(op, a.reshape(batch + [m, split]), padValue)
    totals = J.shrink(scans, [(0, d) for d in batch] + [(0, m), (split - 1, split)]).reshape(batch + [m])
    offsets = _cumulative_quadratic(op, totals, padValue, -1)
    off = offsets.reshape(batch + [m, 1])
    out = scans.add(off) if op == AluOp.Add else scans.mul(off)
    result = J.shrink(out.reshape(batch + [m * split]), [(0, d) for d in batch] + [(0, n)])
    return moveaxis(result, -1, axis)


def cumsum(a: Tracer, axis=None):
    return _cumulative(AluOp.Add, a, axis)


def cumprod(a: Tracer, axis=None):
    return _cumulative(AluOp.Mul, a, axis)


def diff(a: Tracer, n: int = 1, axis: int = -1, prepend=None, append=None):
    """n-th difference along `axis`: `a[1:] - a[:-1]` n times, `!=` on booleans (numpy.ts:724-763)."""
    a = J._raise(a)
    if n < 0:
        raise ValueError(f"diff: order must be a non-negative integer, got {n}")
    if n == 0:
        return a
    if a.ndim == 0:
        raise ValueError("diff: input must be at least one-dimensional")
    (axis,) = J._normalize_axis(axis, a.ndim)
    if prepend is not None or append is not None:
        edge = [1 if i == axis else d for i, d in enumerate(a.shape)]
        parts = [a]
        for value, front in ((prepend, True), (append, False)):
            if value is None:
                continue
            # A scalar edge becomes a constant *array* (its own buffer): a literal has no view for Concatenate's padding
            # to mask, and would be added to every element (the reference's eager path pads the constant's own tracker).
            v = J._raise(value) if not isinstance(value, (int, float)) else J._raise(ConstArray(tuple(edge), a.dtype, AluExp.const(a.dtype, value)))
            parts.insert(0, v) if front else parts.append(v)
        a = J.concatenate(parts, axis)
    for _ in range(min(n, a.shape[axis])):
        length = a.shape[axis]
        upper = J.shrink(a, [(1, length) if i == axis else (0, d) for i, d in enumerate(a.shape)])
        lower = J.shrink(a, [(0, length - 1) if i == axis else (0, d) for i, d in enumerate(a.shape)])
        a = J.notEqual(upper, lower) if a.dtype == DType.Bool else upper.sub(lower)
    return a


# ---- views, products and predicates of the numpy surface -----------------------------------------------

def swapaxes(a: Tracer, axis1: int, axis2: int):
    perm = list(range(a.ndim))
    perm[axis1], perm[axis2] = perm[axis2], perm[axis1]
    return a.transpose(perm)


def rot90(m: Tracer, k: int = 1, axes: Sequence[int] = (0, 1)):
    """Rotation by k quarter turns in the plane of `axes`: flips and an axis swap, all views (numpy.ts rot90)."""
    if len(axes) != 2:
        raise ValueError("rot90: axes must contain exactly two axes")
    a1, a2 = [ax + m.ndim if ax < 0 else ax for ax in axes]  # in the given order
    if a1 == a2:
        raise ValueError("rot90: axes must be different")
    k = k % 4
    if k == 0:
        return m
    if k == 1:
        return swapaxes(J.flip(m, a2), a1, a2)
    if k == 2:
        return J.flip(m, [a1, a2])
    return J.flip(swapaxes(m, a1, a2), a2)


def roll(a: Tracer, shift, axis=None):
    """Circular shift: split at n - shift and concatenate the two parts the other way round, per axis (numpy.ts roll)."""
    if axis is None:
        return roll(a.reshape([-1]), shift, 0).reshape(list(a.shape))
    axes = [ax + a.ndim if ax < 0 else ax for ax in ([axis] if isinstance(axis, int) else list(axis))]  # in the given order
    shifts = [shift] * len(axes) if isinstance(shift, int) else list(shift)
    if len(shifts) != len(axes):
        raise ValueError(f"roll: shift and axis must have the same length, got shift={shifts} and axis={axes}")
    for s, ax in zip(shifts, axes):
        n = a.shape[ax]
        s1 = s % n
        if s1:
            head, tail = J.split(a, ax, [n - s1, s1])
            a = J.concatenate([tail, head], ax)
    return a


def sign(x: Tracer):
    """`where(x != 0, where(x < 0, -1, 1), 0)` (numpy.ts sign)."""
    return J.where(J.notEqual(x, 0), J.where(J.less(x, 0), -1, 1), 0)


def isnan(x: Tracer):
    return J.notEqual(x, x)


def isposinf(x: Tracer):
    return J.equal(x, math.inf)


def isneginf(x: Tracer):
    return J.equal(x, -math.inf)


def isinf(x: Tracer):
    """Bool `+` is OR (numpy.ts isinf)."""
    return J.add(isposinf(x), isneginf(x))


def isfinite(x: Tracer):
    """`!isnan & !isinf` spelt with the comparisons the IR has: x - x == 0 fails exactly for NaN and the infinities."""
    return J.equal(x.sub(x), 0)


def trapezoid(y: Tracer, x: Optional[Tracer] = None, dx=1.0, axis: int = -1):
    """Trapezoidal rule: `sum((y[1:] + y[:-1]) * 0.5 * dx, -1)` after moving `axis` last (numpy.ts trapezoid).  `dx`
    may be a number or an array aligned to the trailing axes of y; `x` gives sample points (1-D, or shaped like y's
    trailing axes)."""
    y = J._raise(y)
    (ax,) = J._normalize_axis(axis, y.ndim)

    def sl(a, d, lo, hi):
        return J.shrink(a, [(lo if i == d else 0, (hi if hi > 0 else n + hi) if i == d else n) for i, n in enumerate(a.shape)])

    if x is None:
        if y.dtype not in (DType.Float32, DType.Float16, DType.Float64):
            y = y.astype(DType.Float32)
        if isinstance(dx, (int, float)):
            spacing = dx
        else:
            spacing = J._raise(dx)
            if spacing.ndim < y.ndim:
                spacing = spacing.reshape([1] * (y.ndim - spacing.ndim) + list(spacing.shape))
            spacing = moveaxis(spacing, axis, -1)
    else:
        x = J._raise(x)
        dt = J.promoteTypes(y.dtype, x.dtype)
        if dt not in (DType.Float32, DType.Float16, DType.Float64):
            dt = DType.Float32
        y, x = y.astype(dt), x.astype(dt)
        xa = 0 if x.ndim == 1 else J._normalize_axis(axis, x.ndim)[0]
        d = sl(x, xa, 1, x.shape[xa]).sub(sl(x, xa, 0, -1))
        spacing = d if x.ndim == 1 else moveaxis(d, xa, -1)
    y = moveaxis(y, ax, -1)
    last = y.ndim - 1
    avg = sl(y, last, 1, y.shape[last]).add(sl(y, last, 0, -1)).mul(0.5)
    return avg.mul(spacing).sum(-1)


def outer(x: Tracer, y: Tracer):
    x, y = x.reshape([-1]), y.reshape([-1])
    return J.mul(x.reshape([x.shape[0], 1]), y)


def inner(x: Tracer, y: Tracer):
    return lax_dot(x, y, [-1], [-1])


def tensordot(x: Tracer, y: Tracer, axes=2):
    if isinstance(axes, int):
        axes = (list(range(-axes, 0)), list(range(axes)))
    return lax_dot(x, y, list(axes[0]), list(axes[1]))


def vdot(x: Tracer, y: Tracer):
    return J.dot(x.reshape([-1]), y.reshape([-1]))


def vecdot(x: Tracer, y: Tracer, axis: int = -1):
    return J.dot(moveaxis(x, axis, -1), moveaxis(y, axis, -1))


def matvec(x1: Tracer, x2: Tracer):
    """`...mn,...n->...m` with broadcasting batch axes: one Dot of [..., m, n] against [..., 1, n]."""
    if x1.ndim < 2 or x2.ndim < 1:
        raise ValueError("matvec: x1 must be at least 2D and x2 at least 1D")
    return J.dot(x1, x2.reshape(list(x2.shape[:-1]) + [1, x2.shape[-1]]))


def vecmat(x1: Tracer, x2: Tracer):
    """`...n,...nm->...m`: one Dot of [..., 1, n] against the matrix with its last two axes swapped."""
    if x1.ndim < 1 or x2.ndim < 2:
        raise ValueError("vecmat: x1 must be at least 1D and x2 at least 2D")
    return J.dot(x1.reshape(list(x1.shape[:-1]) + [1, x1.shape[-1]]), swapaxes(x2, -1, -2))
