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
  reductions and scans: prod, any, all, ptp, var, std, average, cumsum, cumprod, diff, trapezoid
                                                      src/library/numpy.ts:358-500, 560-772, 3100-3140
  element-wise: logical / bitwise / shifts, signbit, copysign, fmin / fmax, division family (trueDivide, floorDivide,
  fmod, remainder, divmod, modf, trunc), rint / round, exp2 / log2 / log10 / expm1 / logaddexp, power / floatPower /
  cbrt, sinc, tan, acos, atan2, hypot, sinh ... arctanh, nanToNum and the float class predicates
                                                      src/library/numpy.ts:159-225, 2433-3100, 3194-3253
  creation (lazy constants): full / zeros / ones, eye, arange, tri / tril / triu, linspace / logspace / geomspace,
  bartlett / hann / blackman                          src/frontend/array.ts:1484-1790; numpy.ts:2524-2566
  shapes and joins: ravel, squeeze, expandDims, broadcastTo, repeat, tile, pad, split family, concatenate, stack
  family, unstack, append, flip / rot90 / roll, swapaxes, moveaxis
                                                      src/library/numpy.ts:253-275, 792-1330, 1474-1492
  selection and comparison: select, arrayEqual, arrayEquiv, isin, diag / diagflat / diagIndices / trace, meshgrid,
  indices, ediff1d                                    src/library/numpy.ts:774-790, 1350-1450, 1583-1727, 2312-2385, 3176-3192
  products and polynomials: dot, inner, outer, tensordot, vdot, vecdot, matvec, vecmat, cross, vander, polyval, polyadd,
  polysub, polymul, convolve, correlate, cov, corrcoef, unwrap
                                                      src/library/numpy.ts:1729-1815, 1988-2310, 2933-2980, 3141-3174
  activations: relu ... mish, glu, logSoftmax, logmeanexp, log1mexp, oneHot; lax.topK; scipySpecial.logit
                                                      src/library/nn.ts:47-380, 430-436; lax.ts:538-567; scipy-special.ts
  numpy.linalg: cholesky (symmetrised), det, slogdet, eigh / eigvalsh, inv, lstsq, matrixPower, multiDot, solve with
  broadcast batches, norm / vectorNorm / matrixNorm   src/library/numpy-linalg.ts:14-485
  numpy.fft over (real, imag) pairs: fft / ifft, fftn / fft2 and inverses, rfft / irfft and n-d forms, hfft / ihfft,
  fftfreq / rfftfreq, fftshift / ifftshift            src/library/numpy-fft.ts:105-384
  random: ball, bernoulli, categorical, cauchy, choice, doubleSidedMaxwell, geometric, gumbel, laplace, logistic,
  lognormal, maxwell, multivariateNormal, pareto, permutation, rademacher, randint, rayleigh, triangular, weibullMin
                                                      src/library/random.ts:146-700
Not restated: fromfunction and applyAlongAxis (they are built on vmap, a transformation this layer does not have).
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


def softmax(x, axis=-1):
    x = J._raise(x)
    if not J._normalize_axis(axis, x.ndim):
        return onesLike(x)  # no axes to normalise over (nn.ts:294-296)
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


def einsum(*args):
    """`einsum("ij,jk->ik", a, b, ...)` or `einsum(a, [0, 1], b, [1, 2], [0, 2])`: operands are contracted pairwise in
    the order the path search picks; before each contraction an operand's repeated indices are replaced by diagonals and
    indices nobody else needs are summed away; each pair goes through one general dot with the shared surviving indices as
    batch dimensions; a final transpose gives the requested order (numpy.ts:1851-1986)."""
    from .einsum import EinsumInput, computeEinsumPath, parseEinsumExpression
    if not args:
        raise ValueError("einsum: must provide at least one argument")
    if isinstance(args[0], str):
        operands = [J._raise(x) for x in args[1:]]
        inp = parseEinsumExpression(args[0], [list(x.shape) for x in operands])
    else:
        n = len(args) >> 1
        operands = [J._raise(args[2 * i]) for i in range(n)]
        lhs = [list(args[2 * i + 1]) for i in range(n)]
        if len(args) % 2 == 1:
            rhs = list(args[2 * n])
        else:
            count: dict = {}
            for i in [i for idx in lhs for i in idx]:
                count[i] = count.get(i, 0) + 1
            rhs = sorted(i for i, c in count.items() if c == 1)
        inp = EinsumInput([list(x.shape) for x in operands], lhs, rhs)
    path = computeEinsumPath(inp)
    usage: dict = {}
    for i in [i for idx in inp.lhsIndices for i in idx] + list(inp.rhsIndex):
        usage[i] = usage.get(i, 0) + 1
    indices = [list(i) for i in inp.lhsIndices]

    def single(ar: Tracer, index, keep=()):
        index = list(index)
        again = True
        while again:
            again = False
            for i, idx in enumerate(index):
                if idx in index[i + 1:]:
                    j = index.index(idx, i + 1)
                    ar = diagonal(ar, 0, i, j)
                    del index[j], index[i]
                    index.append(idx)
                    again = True
                    break
        for i in range(len(index) - 1, -1, -1):
            if usage.get(index[i], 0) == 0 and index[i] not in keep:
                ar = ar.sum(i)
                del index[i]
        return ar, index

    for i, j in path.path:
        reduced = []
        for idx in indices[i] + indices[j]:
            usage[idx] -= 1
            if usage[idx] == 0:
                reduced.append(idx)
        a, aidx = single(operands[i], indices[i], indices[j])
        b, bidx = single(operands[j], indices[j], indices[i])
        reduced = [idx for idx in dict.fromkeys(reduced) if idx in aidx]
        batch = [idx for idx in aidx if idx in bidx and idx not in reduced]
        operands.append(lax_dot(a, b, [aidx.index(x) for x in reduced], [bidx.index(x) for x in reduced],
                                [aidx.index(x) for x in batch], [bidx.index(x) for x in batch]))
        indices.append(batch + [x for x in aidx if x not in bidx] + [x for x in bidx if x not in aidx])
        for idx in indices[-1]:
            usage[idx] += 1
    for idx in indices[len(operands) - 1]:
        usage[idx] -= 1
    ar, index = single(operands[-1], indices[len(operands) - 1])
    perm = [index.index(x) for x in inp.rhsIndex]
    return ar.transpose(perm)


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


def _lower_conv_transpose_1d(lhs: Tracer, rhs: Tracer, strides, padding, ld, rd):
    """A 1-D transposed convolution (unit stride, input dilated by `stride`, non-negative padding) without dilating the
    input: every input sample times every kernel tap as one Dot giving [N, O, K, W]; the reversed kernel axis is cut into
    ceil(K / stride) contributions of `stride` phases each, contribution i is shifted by i input blocks (a Pad) and the
    contributions are added; the requested output range is then cut out of the full overlap-add signal
    (lax.ts:166-250).  None when the shape is outside that case (more than eight contributions included)."""
    from .convolution import ConvParams, checkConvShape
    if (lhs.ndim != 3 or rhs.ndim != 3 or len(strides) != 1 or strides[0] != 1 or len(ld) != 1 or ld[0] <= 1
            or len(rd) != 1 or rd[0] != 1 or len(padding) != 1 or padding[0][0] < 0 or padding[0][1] < 0
            or any(d <= 0 for d in lhs.shape) or any(d <= 0 for d in rhs.shape)):
        return None
    outShape = checkConvShape(list(lhs.shape), list(rhs.shape), ConvParams(0, list(strides), [tuple(p) for p in padding], list(ld), list(rd)))
    if any(d <= 0 for d in outShape):
        return None
    B, C, W = lhs.shape
    O, _, K = rhs.shape
    stride = ld[0]
    count = -(-K // stride)
    if count > 8:
        return None
    a = lhs.transpose([0, 2, 1]).reshape([B, 1, 1, W, C])
    b = rhs.transpose([0, 2, 1]).reshape([1, O, K, 1, C])
    cols = J.dot(a, b)  # [B, O, K, W]
    cols = J.flip(cols.transpose([0, 1, 3, 2]), [3])
    cols = J.pad(cols, [(0, 0), (0, 0), (0, 0), (0, count * stride - K)]).reshape([B, O, W, count, stride])
    terms = []
    for index, term in enumerate(J.split(cols, 3, [1] * count)):
        term = term.reshape([B, O, W, stride])
        terms.append(J.pad(term, [(0, 0), (0, 0), (index, count - 1 - index), (0, 0)]))
    out = terms[0]
    for t in terms[1:]:
        out = out.add(t)
    out = out.reshape([B, O, -1])
    full = (W - 1) * stride + K
    out = J.shrink(out, [(0, B), (0, O), (0, full)])
    outLen = outShape[2]
    offset = K - 1 - padding[0][0]
    padL, padR = max(0, -offset), max(0, offset + outLen - full)
    out = J.pad(out, [(0, 0), (0, 0), (padL, padR)])
    return J.shrink(out, [(0, B), (0, O), (offset + padL, offset + padL + outLen)])


def convGeneralDilated(lhs: Tracer, rhs: Tracer, windowStrides: Sequence[int], padding, lhsDilation=None, rhsDilation=None,
                       featureGroupCount: int = 1):
    """`lax.conv_general_dilated`: lhs `[N, C, *xs]`, rhs `[O, C / G, *ks]`.  One feature group goes to the Conv primitive
    (a 1-D transposed convolution through the overlap-add lowering above when it applies); G groups become a leading
    batch axis of the primitive: lhs -> [G, N, C/G, *xs], rhs -> [G, O/G, C/G, *ks], result moved back to [N, O, *ys]
    (lax.ts:252-343)."""
    lhs, rhs = J._raise(lhs), J._raise(rhs)
    if lhs.ndim < 2:
        raise ValueError("lhs must have at least 2 dimensions")
    if rhs.ndim < 2:
        raise ValueError("rhs must have at least 2 dimensions")
    n = lhs.ndim - 2
    rd = list(rhsDilation) if rhsDilation is not None else [1] * n
    ld = list(lhsDilation) if lhsDilation is not None else [1] * n
    if isinstance(padding, str):
        if any(d != 1 for d in ld):
            raise ValueError("String padding is not supported for transposed convolutions")
        padding = padtypeToPads(lhs.shape[2:], rhs.shape[2:], windowStrides, rd, padding)
    padding = [tuple(p) for p in padding]
    from .convolution import ConvParams
    if featureGroupCount == 1:
        lowered = _lower_conv_transpose_1d(lhs, rhs, list(windowStrides), padding, ld, rd)
        if lowered is not None:
            return lowered
        return J.conv(lhs, rhs, ConvParams(0, list(windowStrides), padding, ld, rd))
    G = featureGroupCount
    N, C_in, xs = lhs.shape[0], lhs.shape[1], list(lhs.shape[2:])
    C_out, C_per, ks = rhs.shape[0], rhs.shape[1], list(rhs.shape[2:])
    if C_in % G != 0:
        raise ValueError(f"featureGroupCount={G} must divide input channels={C_in}")
    if C_out % G != 0:
        raise ValueError(f"featureGroupCount={G} must divide output channels={C_out}")
    if C_in // G != C_per:
        raise ValueError(f"rhs input channels={C_per} must equal lhs input channels / groups={C_in // G}")
    lg = moveaxis(lhs.reshape([N, G, C_in // G] + xs), 1, 0)
    rg = rhs.reshape([G, C_out // G, C_per] + ks)
    result = J.conv(lg, rg, ConvParams(1, list(windowStrides), padding, ld, rd))
    return moveaxis(result, 0, 1).reshape([N, C_out] + list(result.shape[3:]))


def _conv_transpose_padding(k: int, s: int, padding):
    """Padding of the dilated input that makes a stride-s transposed convolution the gradient of the forward one
    (lax.ts:444-467)."""
    if padding == "SAME":
        padLen = k + s - 2
        pad1 = k - 1 if s > k - 1 else -(-padLen // 2)
    elif padding == "VALID":
        padLen = k + s - 2 + max(k - s, 0)
        pad1 = k - 1
    elif isinstance(padding, (list, tuple)):
        pad1 = k - 1 - padding[0]
        padLen = pad1 + k - 1 - padding[1]
    else:
        raise ValueError(f"convTranspose: Invalid padding type {padding}")
    return (pad1, padLen - pad1)


def convTranspose(lhs: Tracer, rhs: Tracer, strides: Sequence[int], padding, rhsDilation=None, transposeKernel: bool = False):
    """`lax.conv_transpose`: unit window strides over an input dilated by `strides` (lax.ts:407-442)."""
    lhs, rhs = J._raise(lhs), J._raise(rhs)
    ks = list(rhs.shape[2:])
    rd = list(rhsDilation) if rhsDilation is not None else [1] * len(ks)
    eff = [max(0, (k - 1) * d + 1) for k, d in zip(ks, rd)]
    pads = [_conv_transpose_padding(k, strides[i], padding if isinstance(padding, str) else padding[i]) for i, k in enumerate(eff)]
    if transposeKernel:
        rhs = moveaxis(J.flip(rhs, list(range(2, rhs.ndim))), 0, 1)
    return convGeneralDilated(lhs, rhs, [1] * (lhs.ndim - 2), pads, lhsDilation=list(strides), rhsDilation=rd)


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


def argmax(a: Tracer, axis: Optional[int] = None):
    """First index of the maximum: max over isMax * (length - i), then length - that (numpy.ts:533-556)."""
    a = J._raise(a)
    if axis is None:
        a, axis = a.reshape([-1]), 0  # the flattened array by default
    axis = axis + a.ndim if axis < 0 else axis
    n = a.shape[axis]
    isMax = J.equal(a, a.max(axis, keepdims=True))
    length = J.scalar(n, DType.Int32)
    rev = arange_const(n, 0, -1, DType.Int32, shape=[n] + [1] * (a.ndim - axis - 1))
    idx = isMax.astype(DType.Int32).mul(rev)
    return length.sub(idx.max(axis))


def argmin(a: Tracer, axis: Optional[int] = None):
    """First index of the minimum: the same construction on `a == min(a)` (numpy.ts:497-524)."""
    a = J._raise(a)
    if axis is None:
        a, axis = a.reshape([-1]), 0
    axis = axis + a.ndim if axis < 0 else axis
    n = a.shape[axis]
    isMin = J.equal(a, a.min(axis, keepdims=True))
    length = J.scalar(n, DType.Int32)
    rev = arange_const(n, 0, -1, DType.Int32, shape=[n] + [1] * (a.ndim - axis - 1))
    idx = isMin.astype(DType.Int32).mul(rev)
    return length.sub(idx.max(axis))


def logsumexp(x: Tracer, axis=None, keepdims: bool = False):
    """max + log(sum(exp(x - max))) (nn.ts:332-345)."""
    x = J._raise(x)
    if not J._normalize_axis(axis, x.ndim):
        return x
    xMax = J.stopGradient(x.max(axis, keepdims=True))
    shifted = x.sub(xMax)
    result = xMax.add(J.log(J.exp(shifted).sum(axis, keepdims=True)))
    if keepdims:
        return result
    ax = J._normalize_axis(axis, x.ndim)
    return result.reshape([n for i, n in enumerate(x.shape) if i not in ax])


def dotProductAttention(query: Tracer, key: Tracer, value: Tracer, isCausal: bool = False, scale: Optional[float] = None,
                        fused: bool = False):
    """[B,L,N,H] attention with equal query and key/value head counts (nn.ts:478-583).  `fused=True` hands the whole
    chain to the backend as one `Attention` routine when the operands fit its kernel (float16, head size 32, 64 or 128;
    any L and S) -- a front-end switch the reference does not have; otherwise the reference's composition is traced."""
    B, L, N, H = query.shape
    S = key.shape[1]
    if key.shape != value.shape or key.shape[0] != B or key.shape[3] != H or key.shape[2] != N:
        raise ValueError("dotProductAttention: shape mismatch")
    scale = 1 / math.sqrt(H) if scale is None else scale
    if fused and H in (32, 64, 128) and L >= 1 and S >= 1 and all(t.dtype == DType.Float16 for t in (query, key, value)):
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
    """`numpy.linalg.solve`: batch dimensions broadcast, LU with partial pivoting, the permutation applied as a 0/1
    matrix product, then a unit-lower and an upper triangular solve (numpy-linalg.ts:274-318)."""
    a, b = J._raise(a), J._raise(b)
    n = a.shape[-1] if a.ndim >= 1 else 0
    if a.ndim < 2 or a.shape[-2] != n:
        raise ValueError(f"solve: a must be a batch of square matrices, got {a.shape}")
    if b.ndim == 0:
        raise ValueError("solve: b cannot be scalar")
    b_is_1d = b.ndim == 1
    if b_is_1d:
        b = b.reshape(list(b.shape) + [1])
    if b.shape[-2] != n:
        raise ValueError(f"solve: leading dimension of b must match size of a, got a={a.shape}, b={b.shape}")
    m = b.shape[-1]
    batch = list(J.generalBroadcast(tuple(a.shape[:-2]), tuple(b.shape[:-2])))
    if list(a.shape[:-2]) != batch:
        a = J.broadcast(a, batch + [n, n], list(range(len(batch) + 2 - a.ndim)))
    if list(b.shape[:-2]) != batch:
        b = J.broadcast(b, batch + [n, m], list(range(len(batch) + 2 - b.ndim)))
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
    xs = [_as_array(x) for x in xs]
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
    """`(isnan | isinf) != true` (numpy.ts:3250-3253)."""
    x = J._raise(x)
    if x.dtype not in (DType.Float32, DType.Float16, DType.Float64):
        return J.equal(x, x)
    return J.notEqual(J.add(isnan(x), isinf(x)), True)


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


# ---- element-wise arithmetic, as the reference spells it (src/library/numpy.ts) -----------------------------------

_FLOATS = (DType.Float32, DType.Float16, DType.Float64)


def _floatish(x: Tracer) -> Tracer:
    return x if x.dtype in _FLOATS else x.astype(DType.Float32)


def logicalAnd(x, y):  # numpy.ts:159-162: bool `*` is AND
    return J.mul(J._raise(x).astype(DType.Bool), J._raise(y).astype(DType.Bool))


def logicalOr(x, y):  # numpy.ts:164-167: bool `+` is OR
    return J.add(J._raise(x).astype(DType.Bool), J._raise(y).astype(DType.Bool))


def logicalXor(x, y):  # numpy.ts:169-172
    return J.notEqual(J._raise(x).astype(DType.Bool), J._raise(y).astype(DType.Bool))


def logicalNot(x):  # numpy.ts:174-177
    return J.notEqual(J._raise(x).astype(DType.Bool), True)


def bitwiseAnd(x, y):
    return J.bitCombine(x, y, "and")


def bitwiseOr(x, y):
    return J.bitCombine(x, y, "or")


def bitwiseXor(x, y):
    return J.bitCombine(x, y, "xor")


def invert(x: Tracer):
    """XOR with all ones of the operand's own dtype (numpy.ts:194-211)."""
    x = J._raise(x)
    if x.dtype == DType.Bool:
        ones = True
    elif x.dtype == DType.Uint32:
        ones = J.scalar(0xFFFFFFFF, DType.Uint32)
    elif x.dtype == DType.Int32:
        ones = J.scalar(-1, DType.Int32)
    else:
        raise TypeError(f"invert: unsupported dtype {x.dtype}")
    return J.bitCombine(x, ones, "xor")


def leftShift(x, y):
    return J.bitShift(x, y, "shl")


def rightShift(x, y):
    return J.bitShift(x, y, "shr")


def signbit(x: Tracer):
    """Bool and uint32 have no sign; int32 compares with 0; floats read the top bit of their f32 image through a
    bitcast, which keeps -0 and the sign of a NaN (numpy.ts:2470-2485)."""
    x = J._raise(x)
    if x.dtype in (DType.Bool, DType.Uint32):
        return J.notEqual(x, x)  # all false, shaped like x
    if x.dtype == DType.Int32:
        return J.less(x, 0)
    return J.less(J.bitcast(x.astype(DType.Float32), DType.Int32), J.scalar(0, DType.Int32))


def copysign(x: Tracer, y: Tracer):  # numpy.ts:2490-2492 (so a zero y gives 0)
    return absolute(x).mul(sign(y))


def fmax(x1: Tracer, x2: Tracer):  # numpy.ts:2501-2503
    return J.where(J.add(J.greater(x1, x2), isnan(x2)), x1, x2)


def fmin(x1: Tracer, x2: Tracer):  # numpy.ts:2512-2514
    return J.where(logicalOr(J.less(x1, x2), isnan(x2)), x1, x2)


def heaviside(x1: Tracer, x2):  # numpy.ts:2574-2576
    return J.where(J.less(x1, 0), 0, J.where(J.equal(x1, 0), x2, 1))


def tan(x: Tracer):
    return J.sin(x).div(J.cos(x))


def sinc(x: Tracer):  # numpy.ts:2600-2604
    pix = x.mul(math.pi)
    return J.where(J.equal(x, 0), 1, J.sin(pix).div(pix))


def acos(x: Tracer):
    return J._raise(math.pi / 2).sub(J.asin(x))


def hypot(x1: Tracer, x2: Tracer):
    return J.sqrt(square(x1).add(square(x2)))


def atan2(y: Tracer, x: Tracer):
    """Half-angle form: 2*atan(y / (r + x)) for x >= 0 and 2*atan((r - x) / y) for x < 0 (numpy.ts:2636-2647)."""
    r = J.sqrt(square(x).add(square(y)))
    xNeg = J.less(x, 0)
    numer = J.where(xNeg, r.sub(x), y)
    denom = J.where(xNeg, y, r.add(x))
    return J.atan(numer.div(denom)).mul(2)


def trueDivide(x, y):  # numpy.ts:2669-2677
    x, y = J._raise(x), J._raise(y)
    if x.dtype not in _FLOATS and y.dtype not in _FLOATS:
        x, y = x.astype(DType.Float32), y.astype(DType.Float32)
    return x.div(y)


def fmod(x: Tracer, y: Tracer):  # numpy.ts:2700-2702
    x, y = J._raise(x), J._raise(y)
    return x.sub(J.mul(y, J.idiv(x, y)))


def remainder(x: Tracer, y: Tracer):
    """Sign of the divisor: `mod(mod(x, y) + y, y)` over the numerator-signed Mod primitive (numpy.ts:2708-2712)."""
    return J.mod(J.add(J.mod(x, y), y), y)


def floorDivide(x, y):  # numpy.ts:2684-2694
    x, y = J._raise(x), J._raise(y)
    if x.dtype in _FLOATS or y.dtype in _FLOATS:
        return J.floor(trueDivide(x, y))
    return J._raise(x).sub(remainder(x, y)).div(y)


def divmod_(x, y):
    return [floorDivide(x, y), remainder(x, y)]


def trunc(x):
    return J.idiv(x, 1)  # numpy.ts:2731-2733


def modf(x: Tracer):
    x = _floatish(J._raise(x))
    whole = trunc(x)
    return [x.sub(whole), whole]


def rint(x: Tracer):
    """Round half to even from floor(x + 0.5), stepping back when the fraction is exactly one half and the rounded
    value is odd (numpy.ts:2774-2781)."""
    rounded = J.floor(x.add(0.5))
    half = J.equal(x.sub(J.floor(x)), 0.5)
    odd = J.notEqual(remainder(rounded, 2), 0)
    return J.where(J.mul(half, odd), rounded.sub(1), rounded)


def round_(a: Tracer, decimals: int = 0):  # numpy.ts:2757-2766
    if decimals == 0:
        return rint(a)
    factor = 10 ** decimals
    return rint(a.mul(factor)).mul(1 / factor)


def exp2(p):
    return J.exp(J.mul(p, math.log(2)))


def log2(x):
    return J.log(x).mul(math.log2(math.e))


def log10(x):
    return J.log(x).mul(math.log10(math.e))


def ldexp(x1, x2):
    return J.mul(x1, exp2(x2))


def expm1(x: Tracer):
    """Series through x^7 (Horner) for |x| <= 0.1 (0.01 in f64), exp(x) - 1 elsewhere (numpy.ts:2827-2852)."""
    x = _floatish(J._raise(x))
    cutoff = 0.01 if x.dtype == DType.Float64 else 0.1
    useSeries = J.lessEqual(absolute(x), cutoff)
    sx = clip(x, -cutoff, cutoff)
    series = (sx.mul(1 / 5040).add(1 / 720).mul(sx).add(1 / 120).mul(sx).add(1 / 24).mul(sx).add(1 / 6).mul(sx)
              .add(1 / 2).mul(sx).add(1).mul(sx))
    return J.where(useSeries, series, J.exp(x).sub(1))


def logaddexp(x1: Tracer, x2: Tracer):  # numpy.ts:2890-2893
    xmax = J.maximum(x1, x2)
    return J.log(J.exp(J._raise(x1).sub(xmax)).add(J.exp(J._raise(x2).sub(xmax)))).add(xmax)


def logaddexp2(x1: Tracer, x2: Tracer):  # numpy.ts:2899-2902
    xmax = J.maximum(x1, x2)
    return log2(exp2(J._raise(x1).sub(xmax)).add(exp2(J._raise(x2).sub(xmax)))).add(xmax)


def deg2rad(x):
    return J.mul(x, math.pi / 180)


def rad2deg(x):
    return J.mul(x, 180 / math.pi)


def power(x1, x2):
    """exp(x2 * log|x1|) with the sign put back for odd integer exponents and NaN for a negative base with a
    non-integer exponent (numpy.ts:2982-2999)."""
    x1, x2 = J._raise(x1), J._raise(x2)
    x2i = trunc(x2)
    shouldBeNaN = J.mul(J.notEqual(x2, x2i), J.less(x1, 0))
    resultSign = J.where(J.notEqual(J.mod(x2i, 2), 0), J.where(J.less(x1, 0), -1, 1), 1)
    return J.where(shouldBeNaN, math.nan, J.exp(J.log(absolute(x1)).mul(x2)).mul(resultSign))


def resultType(*xs) -> DType:
    """The promoted dtype of the operands, shapes aside (numpy.ts:342-355)."""
    avals = [J.ShapedArray((), t.dtype, t.aval.weak) for t in (J._raise(x) for x in xs)]
    out = avals[0]
    for a in avals[1:]:
        out = J.promoteAvals(out, a)
    return out.dtype


def floatPower(x1, x2):  # numpy.ts:3007-3015
    x1, x2 = J._raise(x1), J._raise(x2)
    dt = J.promoteAvals(x1.aval, x2.aval).dtype
    if dt not in _FLOATS:
        dt = DType.Float32
    return power(x1.astype(dt), x2.astype(dt))


def cbrt(x: Tracer):  # numpy.ts:3018-3022
    sgn = J.where(J.less(x, 0), -1, 1)
    return sgn.mul(J.exp(J.log(x.mul(sgn)).mul(1 / 3)))


def sinh(x: Tracer):
    ex = J.exp(x)
    return ex.sub(J.reciprocal(ex)).mul(0.5)


def cosh(x: Tracer):
    ex = J.exp(x)
    return ex.add(J.reciprocal(ex)).mul(0.5)


def arcsinh(x: Tracer):
    return J.log(x.add(J.sqrt(square(x).add(1))))


def arccosh(x: Tracer):
    return J.log(x.add(J.sqrt(square(x).sub(1))))


def arctanh(x: Tracer):
    return J.log(J.add(1, x).div(J._raise(1).sub(x))).mul(0.5)


_FINFO_MAX = {DType.Float32: 3.4028234663852886e38, DType.Float16: 65504.0, DType.Float64: 1.7976931348623157e308}


def nanToNum(x: Tracer, nan=0.0, posinf=None, neginf=None):
    """NaN -> `nan`, +-Inf -> `posinf` / `neginf` (default: the dtype's largest finite values) (numpy.ts:3225-3244)."""
    x = J._raise(x)
    x = J.where(isnan(x), nan, x)
    if x.dtype in _FLOATS:
        hi, lo = _FINFO_MAX[x.dtype], -_FINFO_MAX[x.dtype]
    else:
        hi, lo = {DType.Int32: (2**31 - 1, -2**31), DType.Uint32: (2**32 - 1, 0), DType.Bool: (1, 0)}[x.dtype]
    x = J.where(isposinf(x), hi if posinf is None else posinf, x)
    return J.where(isneginf(x), lo if neginf is None else neginf, x)


# ---- array creation: lazy constants (src/frontend/array.ts:1484-1790) ---------------------------------------------

def full(shape: Sequence[int], value, dtype: Optional[DType] = None) -> ConstArray:
    if dtype is None:
        dtype = DType.Bool if isinstance(value, bool) else DType.Float32
    return ConstArray(tuple(shape), dtype, AluExp.const(dtype, value))


def zeros(shape: Sequence[int], dtype: DType = DType.Float32) -> ConstArray:
    return full(shape, 0, dtype)


def ones(shape: Sequence[int], dtype: DType = DType.Float32) -> ConstArray:
    return full(shape, 1, dtype)


def zerosLike(a: Tracer, dtype: Optional[DType] = None, shape: Optional[Sequence[int]] = None) -> ConstArray:
    return full(a.shape if shape is None else shape, 0, dtype or a.dtype)


def onesLike(a: Tracer, dtype: Optional[DType] = None, shape: Optional[Sequence[int]] = None) -> ConstArray:
    return full(a.shape if shape is None else shape, 1, dtype or a.dtype)


def eye(numRows: int, numCols: Optional[int] = None, dtype: DType = DType.Float32):
    """`idx % (cols + 1) < 1` cast to the dtype; with fewer columns than rows the transpose of the wide case, since that
    is no modular expression of the index any more (array.ts:1515-1547)."""
    numCols = numRows if numCols is None else numCols
    if numCols < numRows:
        return J.transpose(J._raise(eye(numCols, numRows, dtype)))
    if numRows == 0:
        return zeros([0, numCols], dtype)
    exp = AluExp.cmplt(AluExp.mod(AluVar.gidx, AluExp.i32(numCols + 1)), AluExp.i32(1))
    return ConstArray((numRows, numCols), dtype, AluExp.cast(dtype, exp))


def arange(start, stop=None, step=1, dtype: DType = DType.Int32) -> ConstArray:
    """`start + cast(idx) * step` in the result dtype, so a fractional step in int32 adds zeros (array.ts:1570-1612)."""
    if stop is None:
        start, stop = 0, start
    if step == 0:
        raise ValueError(f"Invalid step for arange: {step}. Step must be non-zero.")
    size = max(0, math.ceil((stop - start) / step))
    if size == 0:
        return zeros([0], dtype)
    exp = AluExp.add(AluExp.const(dtype, start), AluExp.mul(AluExp.cast(dtype, AluVar.gidx), AluExp.const(dtype, step)))
    return ConstArray((size,), dtype, exp)


def tri(n: int, m: Optional[int] = None, k: int = 0, dtype: DType = DType.Float32):
    """`arange(k, n + k)[:, None] >= arange(m)` (array.ts:1614-1635)."""
    m = n if m is None else m
    for name, v in (("n", n), ("m", m)):
        if not isinstance(v, int) or v < 0:
            raise ValueError(f"tri: {name} must be a non-negative integer, got {v}")
    if not isinstance(k, int):
        raise ValueError(f"tri: k must be an integer, got {k}")
    rows, cols = J._raise(arange(k, n + k, 1)), J._raise(arange(0, m, 1))
    return J.greaterEqual(rows.reshape([n, 1]), cols).astype(dtype)


def tril(a: Tracer, k: int = 0):
    a = J._raise(a)
    if a.ndim < 2:
        raise ValueError(f"tril: input array must be at least 2D, got {a.ndim}D")
    return J.where(tri(a.shape[-2], a.shape[-1], k, DType.Bool), a, zerosLike(a))


def triu(a: Tracer, k: int = 0):
    a = J._raise(a)
    if a.ndim < 2:
        raise ValueError(f"tril: input array must be at least 2D, got {a.ndim}D")
    return J.where(tri(a.shape[-2], a.shape[-1], k - 1, DType.Bool), zerosLike(a), a)


def linspace(start: float, stop: float, num: int = 50, endpoint: bool = True, dtype: DType = DType.Float32) -> ConstArray:
    """`cast(f32(start) + f32(delta / denom) * f32(idx))` (array.ts:1673-1729)."""
    if not isinstance(num, int) or num < 0:
        raise ValueError(f"Invalid num for linspace: {num}. Must be non-negative integer.")
    if num == 0:
        return zeros([0], dtype)
    if num == 1:
        return full([1], start, dtype)
    if start == stop:
        return full([num], start, dtype)
    denom = num - 1 if endpoint else num
    exp = AluExp.cast(dtype, AluExp.add(AluExp.f32(start), AluExp.mul(AluExp.f32((stop - start) / denom), AluExp.cast(DType.Float32, AluVar.gidx))))
    return ConstArray((num,), dtype, exp)


def logspace(start: float, stop: float, num: int = 50, endpoint: bool = True, base: float = 10, dtype: DType = DType.Float32):
    return J.exp(J.mul(linspace(start, stop, num, endpoint, dtype), math.log(base)))  # array.ts:1731-1743


def geomspace(start: float, stop: float, num: int = 50, endpoint: bool = True, dtype: DType = DType.Float32):
    if start == 0 or stop == 0 or (start > 0) != (stop > 0):
        raise ValueError(f"geomspace: start ({start}) and stop ({stop}) must be nonzero and have the same sign")
    comp = dtype if dtype in _FLOATS else DType.Float32
    y = logspace(math.log10(abs(start)), math.log10(abs(stop)), num, endpoint, 10, comp)
    result = y.mul(-1) if start < 0 else y
    return result.astype(dtype)


def _window_size(name: str, M):
    if not isinstance(M, int) or M < 0:
        raise ValueError(f"Invalid window size for {name}: {M}. Must be a non-negative integer.")


def bartlett(M: int):  # numpy.ts:2524-2532
    _window_size("bartlett", M)
    if M <= 1:
        return ones([M])
    return J._raise(1).sub(absolute(J._raise(linspace(-1, 1, M))))


def hann(M: int):
    return J.cos(linspace(0, 2 * math.pi, M)).mul(-0.5).add(0.5)


def blackman(M: int):  # numpy.ts:2552-2566
    _window_size("blackman", M)
    if M <= 1:
        return ones([M])
    return J.cos(linspace(0, 2 * math.pi, M)).mul(-0.5).add(J.cos(linspace(0, 4 * math.pi, M)).mul(0.08)).add(0.42)


# ---- shapes, joins and selections (src/library/numpy.ts:792-1500) --------------------------------------------------

def _as_array(x):
    """A Python number becomes a 0-d constant array (what the reference's fudgeArray makes of it) rather than a literal
    inlined into the expression: Pad and Concatenate act on views, and a bare literal has none."""
    if isinstance(x, bool):
        return J._raise(full([], x))
    if isinstance(x, (int, float)):
        return J._raise(full([], float(x)))
    return J._raise(x)


def ravel(a):
    return _as_array(a).reshape([-1])


def squeeze(a: Tracer, axis=None):
    a = J._raise(a)
    if axis is None:
        axis = [i for i, d in enumerate(a.shape) if d == 1]
    axis = J._normalize_axis(axis, a.ndim)
    if any(a.shape[i] != 1 for i in axis):
        raise ValueError("Cannot squeeze axis with size != 1")
    return a.reshape([d for i, d in enumerate(a.shape) if i not in axis])


def expandDims(a: Tracer, axis):
    a = J._raise(a)
    axis = [axis] if isinstance(axis, int) else list(axis)
    nd = a.ndim + len(axis)
    norm = [x + nd if x < 0 else x for x in axis]
    if any(x < 0 or x >= nd for x in norm):
        raise ValueError(f"expandDims: axis {axis} out of bounds for array of dimension {nd}")
    if len(set(norm)) != len(norm):
        raise ValueError("expandDims: repeated axis")
    src = iter(a.shape)
    return a.reshape([1 if i in norm else next(src) for i in range(nd)])


def broadcastTo(a, shape: Sequence[int]):
    a = J._raise(a)
    if len(shape) < a.ndim:
        raise ValueError(f"broadcastTo: target shape {list(shape)} has fewer dimensions than input array: {a.ndim}")
    return J.broadcast(a, list(shape), list(range(len(shape) - a.ndim)))


def broadcastArrays(*xs):
    xs = [J._raise(x) for x in xs]
    shape: Sequence[int] = ()
    for x in xs:
        shape = J.generalBroadcast(tuple(shape), tuple(x.shape))
    return [broadcastTo(x, shape) for x in xs]


def repeat(a: Tracer, repeats: int, axis: Optional[int] = None):
    """Each element `repeats` times in a row: broadcast a new axis after `axis`, then merge it (numpy.ts:1254-1276)."""
    if not isinstance(repeats, int) or repeats < 0:
        raise ValueError(f"repeat: repeats must be a non-negative integer, got {repeats}")
    a = J._raise(a)
    if axis is None:
        a, axis = ravel(a), 0
    (axis,) = J._normalize_axis(axis, a.ndim)
    if repeats == 1:
        return a
    wide = list(a.shape[:axis + 1]) + [repeats] + list(a.shape[axis + 1:])
    final = list(a.shape[:axis]) + [a.shape[axis] * repeats] + list(a.shape[axis + 1:])
    return J.broadcast(a, wide, [axis + 1]).reshape(final)


def tile(a: Tracer, reps):
    """Whole-array copies: a new leading axis per repeated dimension, then merged (numpy.ts:1283-1310)."""
    a = J._raise(a)
    reps = [reps] if isinstance(reps, int) else list(reps)
    if any(not isinstance(r, int) or r < 0 for r in reps):
        raise ValueError(f"tile: reps must be non-negative integers, got {reps}")
    ndiff = len(reps) - a.ndim
    if ndiff > 0:
        a = a.reshape([1] * ndiff + list(a.shape))
    if ndiff < 0:
        reps = [1] * (-ndiff) + reps
    wide, axes = [], []
    for i in range(a.ndim):
        if reps[i] > 1:
            wide.append(reps[i])
            axes.append(len(wide) - 1)
        wide.append(a.shape[i])
    final = [d * r for d, r in zip(a.shape, reps)]
    if any(r == 0 for r in reps):
        return zeros(final, a.dtype)
    return J.broadcast(a, wide, axes).reshape(final)


def pad(x: Tracer, width):
    """Width as one number, one pair (both for every axis), a pair per axis, or {axis: pair} (core.ts:500-527)."""
    x = J._raise(x)
    nd = x.ndim
    is_pair = lambda w: isinstance(w, (list, tuple)) and len(w) == 2 and all(isinstance(v, int) for v in w)
    if isinstance(width, int):
        w = [(width, width)]
    elif is_pair(width):
        w = [tuple(width)]
    elif isinstance(width, dict):
        w = [(0, 0)] * nd
        for k, v in width.items():
            w[J._normalize_axis(int(k), nd)[0]] = tuple(v)
    elif not all(is_pair(p) for p in width):
        raise TypeError(f"Invalid pad() type: {width}")
    else:
        w = [tuple(p) for p in width]
    if len(w) == 1:
        w = [w[0]] * nd
    elif len(w) != nd:
        raise ValueError(f"Invalid pad(): expected {nd} axes, got {len(w)}")
    return J.pad(x, w)


def _split_by_sizes(a: Tracer, sizes: List[int], axis: int):
    """Groups of at most eight outputs per Split (numpy.ts:912-935)."""
    results: List[Tracer] = []
    i = 0
    while i < len(sizes):
        if i + 8 >= len(sizes):
            results.extend(J.split(a, axis, sizes[i:]))
            break
        outs = J.split(a, axis, sizes[i:i + 7] + [sum(sizes[i + 7:])])
        results.extend(outs[:-1])
        a = outs[-1]
        i += 7
    return results


def split(a: Tracer, indicesOrSections, axis: int = 0):
    a = J._raise(a)
    (axis,) = J._normalize_axis(axis, a.ndim)
    size = a.shape[axis]
    if isinstance(indicesOrSections, int):
        if size % indicesOrSections != 0:
            raise ValueError(f"Array of size {size} cannot be split into {indicesOrSections} equal parts")
        sizes = [size // indicesOrSections] * indicesOrSections
    else:
        bounds = [0] + [i + size if i < 0 else i for i in indicesOrSections] + [size]
        sizes = [bounds[i + 1] - bounds[i] for i in range(len(bounds) - 1)]
    return _split_by_sizes(a, sizes, axis)


def arraySplit(a: Tracer, indicesOrSections, axis: int = 0):
    a = J._raise(a)
    (axis,) = J._normalize_axis(axis, a.ndim)
    if not isinstance(indicesOrSections, int):
        return split(a, indicesOrSections, axis)
    size = a.shape[axis]
    part, rem = divmod(size, indicesOrSections)
    return _split_by_sizes(a, [part + 1] * rem + [part] * (indicesOrSections - rem), axis)


def dsplit(a: Tracer, indicesOrSections):
    if J._raise(a).ndim < 3:
        raise ValueError("dsplit only works on arrays of 3 or more dimensions")
    return split(a, indicesOrSections, 2)


def hsplit(a: Tracer, indicesOrSections):
    a = J._raise(a)
    if a.ndim == 0:
        raise ValueError("hsplit only works on arrays of 1 or more dimensions")
    return split(a, indicesOrSections, 1 if a.ndim > 1 else 0)


def vsplit(a: Tracer, indicesOrSections):
    return split(a, indicesOrSections, 0)


def concatenate(xs: Sequence[Tracer], axis: int = 0):
    """In groups of eight operands per Concatenate (numpy.ts:937-962)."""
    xs = [J._raise(x) for x in xs]
    if not xs:
        raise ValueError("Need at least one array to concatenate")
    (axis,) = J._normalize_axis(axis, xs[0].ndim)
    for x in xs[1:]:
        if x.ndim != xs[0].ndim or any(j != axis and d != xs[0].shape[j] for j, d in enumerate(x.shape)):
            raise ValueError(f"Cannot concatenate arrays {list(xs[0].shape)} and {list(x.shape)} along axis {axis}")
    result = xs[0]
    for i in range(1, len(xs), 7):
        result = J.concatenate([result] + xs[i:i + 7], axis)
    return result


def unstack(x: Tracer, axis: int = 0):
    x = J._raise(x)
    if x.ndim == 0:
        raise ValueError("unstack requires arrays with rank > 0")
    (axis,) = J._normalize_axis(axis, x.ndim)
    if x.shape[axis] == 0:
        return []
    return [squeeze(p, axis) for p in split(x, x.shape[axis], axis)]


def _same_rank(xs, name):
    xs = [_as_array(x) for x in xs]
    if not xs:
        raise ValueError(f"Need at least one array to {name}")
    if any(x.ndim != xs[0].ndim for x in xs):
        raise ValueError(f"Cannot stack different ranks: {[x.ndim for x in xs]}")
    return xs, xs[0].ndim


def hstack(xs):
    xs, nd = _same_rank(xs, "hstack")
    return stack(xs) if nd == 0 else concatenate(xs, 0 if nd == 1 else 1)


def vstack(xs):
    xs, nd = _same_rank(xs, "vstack")
    if nd == 0:
        return stack(xs).reshape([-1, 1])
    return stack(xs) if nd == 1 else concatenate(xs, 0)


def dstack(xs):
    xs, nd = _same_rank(xs, "dstack")
    if nd == 0:
        return stack(xs).reshape([1, 1, -1])
    if nd == 1:
        r = stack(xs, -1)
        return r.reshape([1] + list(r.shape))
    return stack(xs, -1) if nd == 2 else concatenate(xs, 2)


def columnStack(xs):
    xs, nd = _same_rank(xs, "columnStack")
    if nd == 0:
        return stack(xs).reshape([1, -1])
    return stack(xs, -1) if nd == 1 else concatenate(xs, 1)


def append(arr, values, axis: Optional[int] = None):
    if axis is None:
        return concatenate([ravel(arr), ravel(values)], 0)
    return concatenate([_as_array(arr), _as_array(values)], axis)


def select(condlist, choicelist, defaultValue=0):
    """The first true condition picks: nested `where` from the last pair inwards (numpy.ts:1583-1603)."""
    if len(condlist) != len(choicelist):
        raise ValueError(f"select: condlist must have length equal to choicelist ({len(condlist)} vs {len(choicelist)})")
    if not condlist:
        raise ValueError("select: condlist must be non-empty")
    out = J._raise(defaultValue)
    for c, v in zip(reversed(condlist), reversed(choicelist)):
        out = J.where(J._raise(c).astype(DType.Bool), v, out)
    return out


def arrayEqual(a1, a2, equalNaN: bool = False):
    a1, a2 = J._raise(a1), J._raise(a2)
    if tuple(a1.shape) != tuple(a2.shape):
        return full([], False)
    if equalNaN:
        return all_(J.where(J.mul(isnan(a1), isnan(a2)), True, J.equal(a1, a2)))
    return all_(J.equal(a1, a2))


def arrayEquiv(a1, a2):
    try:
        b1, b2 = broadcastArrays(a1, a2)
    except (ValueError, TypeError):
        return full([], False)
    return all_(J.equal(b1, b2))


def isin(element, testElements, invert: bool = False):
    """any(element[:, None] == test[None, :], 1) over the raveled operands (numpy.ts:3176-3192)."""
    element = J._raise(element)
    outShape = list(element.shape)
    if _int_prod(outShape) == 0:
        return element.astype(DType.Bool)
    test = ravel(testElements)
    if test.shape[0] == 0:  # nothing to compare with: the reduction's identity
        result = full([_int_prod(outShape)], False)
    else:
        result = any_(J.equal(expandDims(ravel(element), 1), test), 1)
    return J._raise(logicalNot(result) if invert else result).reshape(outShape)


def ediff1d(ary, toEnd=None, toBegin=None):
    """Differences of the raveled array, with `toBegin` / `toEnd` cast to its dtype on either side (numpy.ts:774-790)."""
    arr = ravel(ary)
    n = arr.shape[0]
    d = J.shrink(arr, [(min(n, 1), n)]).sub(J.shrink(arr, [(0, max(n - 1, 0))]))
    parts = [d]
    if toBegin is not None:
        parts.insert(0, ravel(toBegin).astype(arr.dtype))
    if toEnd is not None:
        parts.append(ravel(toEnd).astype(arr.dtype))
    return parts[0] if len(parts) == 1 else concatenate(parts, 0)


def diag(v: Tracer, k: int = 0):
    """1-D: where(eye(n) == 1, v, 0) padded out to the k-th diagonal; 2-D: that diagonal (numpy.ts:1365-1393)."""
    a = J._raise(v)
    if not isinstance(k, int):
        raise ValueError(f"k must be an integer, got {k}")
    if a.ndim == 1:
        n = a.shape[0]
        ret = J.where(J.equal(eye(n), 1), a, zerosLike(a))
        if k > 0:
            return J.pad(ret, [(0, k), (k, 0)])
        if k < 0:
            return J.pad(ret, [(-k, 0), (0, -k)])
        return ret
    if a.ndim == 2:
        return diagonal(a, k)
    raise ValueError("numpy.diag only supports 1D and 2D arrays")


def diagflat(v: Tracer, k: int = 0):
    return diag(ravel(v), k)


def diagIndices(n: int, ndim: int = 2):
    if not isinstance(n, int) or n < 0:
        raise ValueError(f"n must be a nonnegative integer, got {n}")
    if not isinstance(ndim, int) or ndim < 0:
        raise ValueError(f"ndim must be a nonnegative integer, got {ndim}")
    index = arange(n)
    return [index] * ndim


def diagIndicesFrom(arr: Tracer):
    a = J._raise(arr)
    if a.ndim < 2:
        raise ValueError(f"diagIndicesFrom: input array must be at least 2D, got {a.ndim}D")
    if any(d != a.shape[0] for d in a.shape):
        raise ValueError(f"diagIndicesFrom: all dimensions of input must be equal, got shape {list(a.shape)}")
    return diagIndices(a.shape[0], a.ndim)


def trace(a: Tracer, offset: int = 0, axis1: int = 0, axis2: int = 1):
    return diagonal(a, offset, axis1, axis2).sum(-1)


def meshgrid(xs: Sequence[Tracer], indexing: str = "xy"):
    """Coordinate grids by broadcasting alone; "xy" swaps the first two (numpy.ts:2312-2345)."""
    xs = [J._raise(x) for x in xs]
    for x in xs:
        if x.ndim != 1:
            raise ValueError(f"meshgrid: all inputs must be 1D arrays, got {x.ndim}D array")
    if len(xs) <= 1:
        return xs
    if indexing == "xy":
        rb, ra, *rest = meshgrid([xs[1], xs[0]] + xs[2:], "ij")
        return [ra, rb] + rest
    shape = [x.shape[0] for x in xs]
    return [J.broadcast(x, shape, [j for j in range(len(xs)) if j != i]) for i, x in enumerate(xs)]


def indices(dimensions: Sequence[int], dtype: DType = DType.Int32, sparse: bool = False):
    if any(not isinstance(d, int) or d < 0 for d in dimensions):
        raise ValueError(f"indices: dimensions must be non-negative integers, got {list(dimensions)}")
    out = []
    for i, dim in enumerate(dimensions):
        shape = [1] * len(dimensions)
        shape[i] = dim
        x = J._raise(arange(0, dim, 1, dtype)).reshape(shape)
        out.append(x if sparse else broadcastTo(x, list(dimensions)))
    if sparse:
        return out
    return stack(out) if out else zeros([0], dtype)


def cumulativeProd(x: Tracer, axis: Optional[int] = None, includeInitial: bool = False):
    x = J._raise(x)
    if x.ndim == 0:
        x = x.reshape([1])
    if x.ndim > 1 and axis is None:
        raise ValueError("cumulativeProd: axis is required for arrays of ndim > 1")
    (axis,) = J._normalize_axis(axis or 0, x.ndim)
    if includeInitial:
        x = concatenate([onesLike(x, shape=[1 if i == axis else d for i, d in enumerate(x.shape)]), x], axis)
    return _cumulative(AluOp.Mul, x, axis)


def cumulativeSum(x: Tracer, axis: Optional[int] = None, includeInitial: bool = False):
    x = J._raise(x)
    if x.ndim == 0:
        x = x.reshape([1])
    if x.ndim > 1 and axis is None:
        raise ValueError("cumulativeSum: axis is required for arrays of ndim > 1")
    (axis,) = J._normalize_axis(axis or 0, x.ndim)
    if includeInitial:
        x = concatenate([zerosLike(x, shape=[1 if i == axis else d for i, d in enumerate(x.shape)]), x], axis)
    return _cumulative(AluOp.Add, x, axis)


def vander(x: Tracer, n: Optional[int] = None, increasing: bool = False):
    """Powers of x as a running product over n - 1 copies, highest power first unless `increasing` (numpy.ts:2014-2034)."""
    x = J._raise(x)
    if x.ndim != 1:
        raise ValueError(f"vander: input must be 1D, got {x.ndim}D")
    n = x.shape[0] if n is None else n
    if not isinstance(n, int) or n < 0:
        raise ValueError(f"vander: n must be a non-negative integer, got {n}")
    rows = x.shape[0]
    if n <= 1:
        return onesLike(x, shape=[rows, n])
    tiled = broadcastTo(x.reshape([rows, 1]), [rows, n - 1])
    result = cumulativeProd(tiled, axis=1, includeInitial=True)
    return result if increasing else J.flip(result, 1)


def polyval(p: Tracer, x: Tracer):
    p, x = J._raise(p), J._raise(x)
    if p.ndim == 0:
        raise ValueError(f"polyval: coefficients must have at least one dimension, got {p.ndim}D")
    n = p.shape[0]
    powers = J._raise(vander(ravel(x), n)).reshape(list(x.shape) + [n])
    return vecdot(moveaxis(p, 0, -1), powers)


def _poly_align(a1, a2, name):
    a1, a2 = J._raise(a1), J._raise(a2)
    if a1.ndim == 0 or a2.ndim == 0:
        raise ValueError(f"{name}: both inputs must be at least 1D arrays, got {a1.ndim}D and {a2.ndim}D")
    swapped = a2.shape[0] > a1.shape[0]
    base, update = (a2, a1) if swapped else (a1, a2)
    update = broadcastTo(update, [update.shape[0]] + list(base.shape[1:]))
    leading = base.shape[0] - update.shape[0]
    if leading > 0:
        update = pad(update, {0: (leading, 0)})
    return base, update, swapped


def polyadd(a1, a2):  # numpy.ts:2071-2102
    base, update, _ = _poly_align(a1, a2, "polyadd")
    return J.add(base, update)


def polysub(a1, a2):  # numpy.ts:2109-2137
    base, update, swapped = _poly_align(a1, a2, "polysub")
    return update.sub(base) if swapped else base.sub(update)


def _conv_impl(name: str, x: Tracer, y: Tracer, mode: str):
    """1-D convolution / correlation through the Conv primitive: the longer operand is the signal
    (numpy.ts:2255-2287)."""
    x, y = J._raise(x), J._raise(y)
    if x.ndim != 1 or y.ndim != 1:
        raise ValueError(f"{name}: both inputs must be 1D arrays, got {x.ndim}D and {y.ndim}D")
    flipOutput = False
    if x.shape[0] < y.shape[0]:
        x, y = y, x
        flipOutput = name == "correlate"
    if name == "convolve":
        y = J.flip(y, None)
    if mode == "valid":
        padding = "VALID"
    elif mode == "same":
        padding = "SAME_LOWER"
    elif mode == "full":
        padding = [(y.shape[0] - 1, y.shape[0] - 1)]
    else:
        raise ValueError(f'{name}: invalid mode {mode}, expected "full", "same", or "valid"')
    z = convGeneralDilated(x.reshape([1, 1, x.shape[0]]), y.reshape([1, 1, y.shape[0]]), [1], padding)
    z = z.reshape([z.shape[-1]])
    return J.flip(z, None) if flipOutput else z


def convolve(x, y, mode: str = "full"):
    return _conv_impl("convolve", x, y, mode)


def correlate(x, y, mode: str = "valid"):
    return _conv_impl("correlate", x, y, mode)


def polymul(a1, a2):  # numpy.ts:2144-2168
    a1, a2 = J._raise(a1), J._raise(a2)
    if a1.ndim != 1 or a2.ndim != 1:
        raise ValueError(f"polymul: both inputs must be 1D arrays, got {a1.ndim}D and {a2.ndim}D")
    dt = resultType(a1, a2)
    if dt not in _FLOATS:
        dt = DType.Float32
    a1, a2 = a1.astype(dt), a2.astype(dt)
    if a1.shape[0] == 0:
        a1 = J._raise(zeros([1], dt))
    if a2.shape[0] == 0:
        a2 = J._raise(zeros([1], dt))
    return convolve(a1, a2, "full")


def cross(a, b, axisa: int = -1, axisb: int = -1, axisc: int = -1, axis: Optional[int] = None):
    """2- and 3-component cross products along an axis; 2-component operands gain a zero third component
    (numpy.ts:2176-2229)."""
    a, b = J._raise(a), J._raise(b)
    if axis is not None:
        axisa = axisb = axisc = axis
    a, b = moveaxis(a, axisa, -1), moveaxis(b, axisb, -1)
    da, db = a.shape[-1], b.shape[-1]
    if da not in (2, 3) or db not in (2, 3):
        raise ValueError(f"cross: incompatible dimensions for cross product (got {da} and {db})")
    if da == 2 and db == 2:
        a0, a1 = split(a, 2, -1)
        b0, b1 = split(b, 2, -1)
        return squeeze(a0.mul(b1).sub(a1.mul(b0)), -1)
    if da == 2:
        a = concatenate([a, zeros(list(a.shape[:-1]) + [1])], -1)
    if db == 2:
        b = concatenate([b, zeros(list(b.shape[:-1]) + [1])], -1)
    a0, a1, a2 = split(a, 3, -1)
    b0, b1, b2 = split(b, 3, -1)
    c0 = a1.mul(b2).sub(a2.mul(b1))
    c1 = a2.mul(b0).sub(a0.mul(b2))
    c2 = a0.mul(b1).sub(a1.mul(b0))
    return moveaxis(concatenate([c0, c1, c2], -1), -1, axisc)


def dot(x, y):
    """Scalar operands multiply; a 1-D y contracts with x's last axis; otherwise x's last axis against y's second to
    last (numpy.ts:1764-1782)."""
    x, y = J._raise(x), J._raise(y)
    if x.ndim == 0 or y.ndim == 0:
        return J.mul(x, y)
    if y.ndim == 1:
        return J.dot(x, y)
    return lax_dot(x, y, [-1], [-2])


def cov(x, y=None, rowvar: bool = True):
    """Rows are variables, columns observations: centre each row, then `x @ x.T / (N - 1)` (numpy.ts:3141-3160)."""
    x = J._raise(x)
    if x.ndim == 1:
        x = x.reshape([1, x.shape[0]])
    if y is not None:
        y = J._raise(y)
        if y.ndim == 1:
            y = y.reshape([1, y.shape[0]])
        x = vstack([x, y])
    if not rowvar:
        x = x.transpose()
    N = x.shape[1]
    x = x.sub(x.mean(1, keepdims=True))
    return dot(x, x.transpose()).div(N - 1)


def corrcoef(x, y=None):
    c = cov(x, y)
    variances = diag(c)
    return c.div(J.sqrt(outer(variances, variances)))


def _round_to(dtype: DType, v: float) -> float:
    import numpy as _np
    if dtype == DType.Float64:
        return float(v)
    with _np.errstate(over="ignore"):  # beyond the dtype's range the rounded constant is an infinity, as Math.fround gives
        return float(_np.float16(v)) if dtype == DType.Float16 else float(_np.float32(v))


def unwrap(p, discont: Optional[float] = None, axis: int = -1, period: float = 2 * math.pi):
    """Jumps of more than `discont` between neighbours are replaced by their complement modulo `period`; the scalar
    constants are rounded to the array's dtype first so that a delta of exactly period / 2 falls the same way on every
    backend (numpy.ts:2933-2980)."""
    x = _floatish(J._raise(p))
    (axis,) = J._normalize_axis(axis, x.ndim)
    n = x.shape[axis]
    if n <= 1:
        return x
    T = _round_to(x.dtype, period)
    interval = _round_to(x.dtype, T / 2)
    disc = _round_to(x.dtype, T / 2 if discont is None else discont)
    head, tail = J.split(x, axis, [1, n - 1])
    dd = tail.sub(J.shrink(x, [(0, n - 1) if i == axis else (0, d) for i, d in enumerate(x.shape)]))
    r = J.mod(dd.add(interval), T)
    pymod = J.where(J.less(r, 0), r.add(T), r) if T >= 0 else J.where(J.greater(r, 0), r.add(T), r)
    ddmod = pymod.sub(interval)
    ddmod = J.where(logicalAnd(J.equal(ddmod, -interval), J.greater(dd, 0)), interval, ddmod)
    correction = J.where(J.less(absolute(dd), disc), 0, ddmod.sub(dd))
    return concatenate([head, tail.add(cumsum(correction, axis))], axis)


def applyOverAxes(func, a, axes: Sequence[int]):
    a = J._raise(a)
    for axis in axes:
        b = func(a, axis)
        if b.ndim == a.ndim:
            a = b
        elif b.ndim == a.ndim - 1:
            a = expandDims(b, axis)
        else:
            raise ValueError("function must return array of the correct shape")
    return a


# ---- activations and friends (src/library/nn.ts:47-380, 430-436), lax.topK, scipySpecial.logit ----------------------

def relu(x):
    return J.maximum(x, 0)


def relu6(x):
    return clip(J._raise(x), 0, 6)


def softplus(x):
    return J.log(J.exp(x).add(1))


def sparsePlus(x: Tracer):
    return J.where(J.lessEqual(x, -1), 0, J.where(J.less(x, 1), square(x.add(1)).mul(0.25), x))


def sparseSigmoid(x: Tracer):
    return clip(x.add(1).mul(0.5), 0, 1)


def softSign(x: Tracer):
    x = J._raise(x)
    return x.div(absolute(x).add(1))


def silu(x: Tracer):
    return x.mul(sigmoid(x))


def logSigmoid(x):
    return J.neg(softplus(J.neg(x)))


def leakyRelu(x: Tracer, negativeSlope=0.01):
    x = J._raise(x)
    return J.where(J.less(x, 0), x.mul(negativeSlope), x)


def hardSigmoid(x):
    return relu6(J.add(x, 3)).mul(1 / 6)


def hardSilu(x: Tracer):
    return J._raise(x).mul(hardSigmoid(x))


def hardTanh(x):
    return clip(J._raise(x), -1, 1)


def elu(x: Tracer, alpha=1.0):
    x = J._raise(x)
    return J.where(J.less(x, 0), J.exp(x).sub(1).mul(alpha), x)


def celu(x: Tracer, alpha=1.0):
    x = J._raise(x)
    return J.where(J.less(x, 0), J.exp(x.div(alpha)).sub(1).mul(alpha), x)


def selu(x: Tracer):
    return J.where(J.less(x, 0), expm1(x).mul(1.6732632423543772), x).mul(1.0507009873554805)


def glu(x: Tracer, axis: int = -1):
    x = J._raise(x)
    (axis,) = J._normalize_axis(axis, x.ndim)
    size = x.shape[axis]
    if size % 2 != 0:
        raise ValueError(f"glu: axis {axis} of shape ({list(x.shape)}) does not have even length")
    sl = lambda lo, hi: [(lo, hi) if i == axis else (0, d) for i, d in enumerate(x.shape)]
    return J.shrink(x, sl(0, size // 2)).mul(sigmoid(J.shrink(x, sl(size // 2, size))))


def squareplus(x: Tracer, b=4.0):
    x = J._raise(x)
    return x.add(J.sqrt(square(x).add(b))).mul(0.5)


def mish(x: Tracer):
    x = J._raise(x)
    return x.mul(tanh(softplus(x)))


def logSoftmax(x: Tracer, axis=-1):
    x = J._raise(x)
    ax = J._normalize_axis(axis, x.ndim)
    if not ax:
        return zerosLike(x)
    shifted = x.sub(J.stopGradient(x.max(ax, keepdims=True)))
    return shifted.sub(J.log(J.exp(shifted).sum(ax, keepdims=True)))


def logmeanexp(x: Tracer, axis=None, keepdims: bool = False):
    x = J._raise(x)
    ax = J._normalize_axis(axis, x.ndim)
    if not ax:
        return x
    return logsumexp(x, ax, keepdims).sub(math.log(_int_prod([x.shape[a] for a in ax])))


def log1mexp(x: Tracer):
    """log(1 - exp(-x)): through expm1 up to log 2, through log1p beyond (nn.ts:370-376)."""
    return J.where(J.lessEqual(x, math.log(2)), J.log(J.neg(expm1(J.neg(x)))), log1p(J.neg(J.exp(J.neg(x)))))


def oneHot(x: Tracer, numClasses: int):
    """Rows of the identity picked by the indices (nn.ts:430-435)."""
    if x.dtype in _FLOATS:
        raise TypeError(f"oneHot expects integers, got {x.dtype}")
    return J.gather(J._raise(eye(numClasses)), [x], [0], 0)


def logit(x: Tracer):
    return J.log(J._raise(x).div(J._raise(1).sub(x)))  # scipy-special.ts


def topK(x: Tracer, k: int, axis: int = -1):
    """The k largest along `axis`, largest first, ties by smaller index: a stable ascending argsort of the reversed
    axis, its last k entries reversed back, indices mirrored (lax.ts:538-567)."""
    x = J._raise(x)
    (axis,) = J._normalize_axis(axis, x.ndim)
    size = x.shape[axis]
    if k < 0 or k > size:
        raise ValueError(f"topK: k must be in the range [0, {size}], got {k}")
    if k == 0:
        shape = [0 if i == axis else d for i, d in enumerate(x.shape)]
        return [zerosLike(x, shape=shape), zerosLike(x, DType.Int32, shape)]
    y, yi = J.argsort(moveaxis(J.flip(x, [axis]), axis, -1))

    def extract(a):
        a = J.shrink(a, [(0, d) for d in a.shape[:-1]] + [(a.shape[-1] - k, a.shape[-1])])
        return J.flip(moveaxis(a, -1, axis), [axis])
    return [extract(y), extract(J.neg(yi).add(size - 1))]


# ---- numpy.linalg (src/library/numpy-linalg.ts) ----------------------------------------------------------------------

def _check_square(name: str, shape) -> int:
    if len(shape) < 2 or shape[-1] != shape[-2]:
        raise ValueError(f"{name}: input must be at least 2D square matrix, got {list(shape)}")
    return shape[-1]


def matrixTranspose(a: Tracer):
    a = J._raise(a)
    if a.ndim < 2:
        raise ValueError("matrixTranspose: input array must be at least 2D")
    return moveaxis(a, -1, -2)


def linalgCholesky(a: Tracer, upper: bool = False, symmetrizeInput: bool = True):
    """`numpy.linalg.cholesky`: the input is symmetrised as (a + a^T) / 2 first (numpy-linalg.ts:14-30)."""
    a = J._raise(a)
    _check_square("cholesky", a.shape)
    if symmetrizeInput:
        a = a.add(matrixTranspose(a)).mul(0.5)
    return cholesky(a, upper)


def det(a: Tracer):
    """Product of U's diagonal times (-1)^(number of row exchanges) (numpy-linalg.ts:53-62)."""
    a = J._raise(a)
    n = _check_square("det", a.shape)
    lu, pivots, _perm = J.lu(a)
    parity = J.mod(J.notEqual(pivots, arange(n)).astype(DType.Int32).sum(-1), 2)
    sign = parity.mul(-2).add(1)
    return prod(diagonal(lu, 0, -1, -2), -1).mul(sign)


def slogdet(a: Tracer):
    a = J._raise(a)
    n = _check_square("slogdet", a.shape)
    lu, pivots, _perm = J.lu(a)
    parity = J.notEqual(pivots, arange(n)).astype(DType.Int32).sum(-1)
    diag = diagonal(lu, 0, -1, -2)
    parity = J.mod(parity.add(J.less(diag, 0).astype(DType.Int32).sum(-1)), 2)
    return [parity.mul(-2).add(1), J.log(absolute(diag)).sum(-1)]


def linalgEigh(a: Tracer, symmetrizeInput: bool = True):
    """`numpy.linalg.eigh`: (eigenvalues ascending, eigenvectors) (numpy-linalg.ts:77-83)."""
    vectors, values = eigh(a, symmetrizeInput=symmetrizeInput)
    return [values, vectors]


def eigvalsh(a: Tracer, symmetrizeInput: bool = True):
    return eigh(a, symmetrizeInput=symmetrizeInput)[1]


def inv(a: Tracer):
    a = J._raise(a)
    n = _check_square("inv", a.shape)
    return solve(a, J._raise(eye(n, None, a.dtype)))


def lstsq(a: Tracer, b: Tracer):
    """Normal equations through a Cholesky factor: A^T (A A^T)^-1 B for wide or square A, (A^T A)^-1 A^T B for tall A
    (numpy-linalg.ts:145-181)."""
    a, b = J._raise(a), J._raise(b)
    if a.ndim != 2:
        raise ValueError(f"lstsq: 'a' must be a 2D array, got {list(a.shape)}")
    m, n = a.shape
    if b.ndim < 1 or b.shape[0] != m:
        raise ValueError(f"lstsq: leading dimension of 'b' must match number of rows of 'a', got {list(b.shape)}")
    at = matrixTranspose(a)
    if m <= n:
        l = linalgCholesky(matmul(a, at), symmetrizeInput=False)
        lb = triangularSolve(l, b, leftSide=True, lower=True)
        return matmul(at, triangularSolve(l, lb, leftSide=True, lower=True, transposeA=True))
    l = linalgCholesky(matmul(at, a), symmetrizeInput=False)
    lb = triangularSolve(l, matmul(at, b), leftSide=True, lower=True)
    return triangularSolve(l, lb, leftSide=True, lower=True, transposeA=True)


def matrixPower(a: Tracer, n: int):
    """Binary powering; a negative exponent powers the inverse (numpy-linalg.ts:185-209)."""
    if not isinstance(n, int):
        raise ValueError(f"matrixPower: exponent must be an integer, got {n}")
    a = J._raise(a)
    m = _check_square("matrixPower", a.shape)
    if n == 0:
        return broadcastTo(eye(m, None, a.dtype), list(a.shape))
    if n < 0:
        a, n = inv(a), -n
    result, a2k, k = None, a, 0
    while n:
        if k > 0:
            a2k = matmul(a2k, a2k)
        if n % 2 == 1:
            result = a2k if result is None else matmul(result, a2k)
        n //= 2
        k += 1
    return result


def multiDot(arrays: Sequence[Tracer]):
    """A chain of matrix products with 1-D ends as row / column vectors, handed to einsum in index-list form so that its
    path search picks the order of the products (numpy-linalg.ts:223-246)."""
    arrays = [J._raise(a) for a in arrays]
    if len(arrays) < 2:
        raise ValueError("Expected at least two arrays")
    if arrays[0].ndim == 1:
        r = multiDot([arrays[0].reshape([1, -1])] + arrays[1:])
        return r.reshape(list(r.shape[1:]))
    if arrays[-1].ndim == 1:
        r = multiDot(arrays[:-1] + [arrays[-1].reshape([-1, 1])])
        return r.reshape(list(r.shape[:-1]))
    args: list = []
    for i, a in enumerate(arrays):
        if a.ndim != 2:
            raise ValueError(f"multiDot: expected 2D, got {list(a.shape)} at index {i}")
        args += [a, [i, i + 1]]
    return einsum(*args)


def vectorNorm(x: Tracer, ord=2, axis=None, keepdims: bool = False):
    x = J._raise(x)
    if ord == math.inf:
        return absolute(x).max(axis, keepdims)
    if ord == -math.inf:
        return absolute(x).min(axis, keepdims)
    if ord == 0:
        return J.notEqual(x, 0).astype(x.dtype).sum(axis, keepdims)
    return power(power(absolute(x), ord).sum(axis, keepdims), 1 / ord)


def matrixNorm(x: Tracer, ord="fro", keepdims: bool = False):
    x = J._raise(x)
    if x.ndim < 2:
        raise ValueError(f"Input must be at least 2-dimensional. Recieved {x.ndim}-dimensional array")
    if ord == "fro":
        return J.sqrt(square(x).sum([-2, -1], keepdims))
    if ord in (1, -1):
        s = absolute(x).sum([-2], keepdims)
        return s.max([-1], keepdims) if ord == 1 else s.min([-1], keepdims)
    if ord in (math.inf, -math.inf):
        s = absolute(x).sum([-1], keepdims)
        ax = [-2 if keepdims else -1]
        return s.max(ax, keepdims) if ord == math.inf else s.min(ax, keepdims)
    raise ValueError(f"Order {ord} is not supported")


def norm(x: Tracer, ord=None, axis=None, keepdims: bool = False):
    """`numpy.linalg.norm`: the flattened 2-norm by default, vector norms over one axis, matrix norms (Frobenius, 1, inf,
    and the singular-value ones) over a pair of axes (numpy-linalg.ts:338-412)."""
    x = _floatish(J._raise(x))
    nd = x.ndim
    check = lambda a: J._normalize_axis(a, nd)[0] if -nd <= a < nd else (_ for _ in ()).throw(ValueError(f"norm: axis {a} out of bounds"))
    if axis is None:
        if ord is None:
            return J.sqrt(square(x).sum(None, keepdims))
        axes = list(range(nd))
    elif isinstance(axis, int):
        axes = [check(axis)]
    else:
        axes = [check(a) for a in axis]
    if len(axes) == 1:
        if isinstance(ord, str):
            raise ValueError(f"norm: invalid order '{ord}' for vector norm")
        return vectorNorm(x, 2 if ord is None else ord, axes[0], keepdims)
    if len(axes) != 2:
        raise ValueError(f"norm: axis must be null, an integer, or a pair of integers, got {axis}")
    rowAxis, colAxis = axes
    if rowAxis == colAxis:
        raise ValueError(f"norm: duplicate axes {axis}")
    if ord is None or ord in ("f", "fro"):
        return J.sqrt(square(x).sum(axes, keepdims))
    if ord in (1, -1):
        sums = absolute(x).sum(rowAxis, keepdims)
        if not keepdims and colAxis > rowAxis:
            colAxis -= 1
        return sums.max(colAxis, keepdims) if ord == 1 else sums.min(colAxis, keepdims)
    if ord in (math.inf, -math.inf):
        sums = absolute(x).sum(colAxis, keepdims)
        if not keepdims and rowAxis > colAxis:
            rowAxis -= 1
        return sums.max(rowAxis, keepdims) if ord == math.inf else sums.min(rowAxis, keepdims)
    if ord in (2, -2, "nuc"):
        y = moveaxis(x, rowAxis, -1)
        y = moveaxis(y, colAxis - 1 if colAxis > rowAxis else colAxis, -1)
        sv = svdvals(y)
        result = sv.max(-1) if ord == 2 else sv.min(-1) if ord == -2 else sv.sum(-1)
        return expandDims(result, axes) if keepdims else result
    raise ValueError(f"norm: invalid order '{ord}' for matrix norm")


# ---- numpy.fft over (real, imag) pairs (src/library/numpy-fft.ts) ------------------------------------------------------

def _check_pair(name: str, real: Tracer, imag: Tracer):
    full = f"jax.numpy.fft.{name}"
    if tuple(real.shape) != tuple(imag.shape):
        raise ValueError(f"{full}: real and imaginary parts must have the same shape, got {list(real.shape)} and {list(imag.shape)}")
    if real.dtype != imag.dtype:
        raise ValueError(f"{full}: real and imaginary parts must have the same dtype, got {real.dtype} and {imag.dtype}")
    if real.dtype not in _FLOATS:
        raise ValueError(f"{full}: input must have a float dtype, got {real.dtype}")


def _axes_in_order(axes, ndim: int) -> List[int]:
    """Given order kept, duplicates refused (utils.ts normalizeAxis with sort = false)."""
    if axes is None:
        return list(range(ndim))
    out: List[int] = []
    for a in ([axes] if isinstance(axes, int) else axes):
        if not -ndim <= a < ndim:
            raise ValueError(f"axis {a} out of bounds for array of dimension {ndim}")
        a = a + ndim if a < 0 else a
        if a in out:
            raise ValueError(f"Duplicate axis {a} passed to function")
        out.append(a)
    return out


def _fft_checked(name: str, real, imag, axis: int, inverse: bool):
    real, imag = J._raise(real), J._raise(imag)
    _check_pair(name, real, imag)
    (axis,) = _axes_in_order(axis, real.ndim)
    if real.shape[axis] < 1:
        raise ValueError(f"jax.numpy.fft.{name}: size must be a positive integer, got {real.shape[axis]}")
    return fft(real, imag, axis, inverse)


def fft1(real, imag, axis: int = -1):
    """`numpy.fft.fft` of a (real, imag) pair along one axis, with the reference's input checks."""
    return _fft_checked("fft", real, imag, axis, False)


def ifft(real, imag, axis: int = -1):
    return _fft_checked("ifft", real, imag, axis, True)


def _transform_n(name, real, imag, axes, transform):
    real, imag = J._raise(real), J._raise(imag)
    _check_pair(name, real, imag)
    for axis in _axes_in_order(axes, real.ndim):
        real, imag = transform(real, imag, axis)
    return real, imag


def fftn(real, imag, axes=None):
    return _transform_n("fftn", real, imag, axes, fft1)


def fft2(real, imag, axes=(-2, -1)):
    return fftn(real, imag, list(axes))


def ifftn(real, imag, axes=None):
    return _transform_n("ifftn", real, imag, axes, ifft)


def ifft2(real, imag, axes=(-2, -1)):
    return ifftn(real, imag, list(axes))


def _slice_axis(a: Tracer, axis: int, start: int, end: int):
    return J.shrink(a, [(start, end) if i == axis else (0, d) for i, d in enumerate(a.shape)])


def rfft(a: Tracer, axis: int = -1):
    """The non-negative half of the spectrum of a real signal: a full transform with a zero imaginary part, cut at
    n // 2 + 1 (numpy-fft.ts:218-229)."""
    a = J._raise(a)
    if a.dtype not in _FLOATS:
        raise ValueError(f"jax.numpy.fft.rfft: input must have a float dtype, got {a.dtype}")
    (axis,) = _axes_in_order(axis, a.ndim)
    re, im = fft1(a, zerosLike(a), axis)
    stop = a.shape[axis] // 2 + 1
    return _slice_axis(re, axis, 0, stop), _slice_axis(im, axis, 0, stop)


def irfft(real, imag, axis: int = -1):
    """Inverse of rfft for an even output length: the packed half is mirrored (conjugated) into the full Hermitian
    spectrum first (numpy-fft.ts:237-262)."""
    real, imag = J._raise(real), J._raise(imag)
    _check_pair("irfft", real, imag)
    (axis,) = _axes_in_order(axis, real.ndim)
    m = real.shape[axis]
    if m < 2:
        raise ValueError(f"jax.numpy.fft.irfft: packed input length must be at least 2, got {m}")
    mr = J.flip(_slice_axis(real, axis, 1, m - 1), [axis])
    mi = J.flip(_slice_axis(imag, axis, 1, m - 1), [axis]).mul(-1)
    return ifft(concatenate([real, mr], axis), concatenate([imag, mi], axis), axis)[0]


def rfftn(a: Tracer, axes=None):
    a = J._raise(a)
    if a.dtype not in _FLOATS:
        raise ValueError(f"jax.numpy.fft.rfftn: input must have a float dtype, got {a.dtype}")
    order = _axes_in_order(axes, a.ndim)
    if not order:
        return a, zerosLike(a)
    re, im = rfft(a, order[-1])
    for axis in order[:-1]:
        re, im = fft1(re, im, axis)
    return re, im


def rfft2(a: Tracer, axes=(-2, -1)):
    return rfftn(a, list(axes))


def irfftn(real, imag, axes=None):
    real, imag = J._raise(real), J._raise(imag)
    _check_pair("irfftn", real, imag)
    order = _axes_in_order(axes, real.ndim)
    if not order:
        return real
    for axis in order[:-1]:
        real, imag = ifft(real, imag, axis)
    return irfft(real, imag, order[-1])


def irfft2(real, imag, axes=(-2, -1)):
    return irfftn(real, imag, list(axes))


def hfft(real, imag, axis: int = -1):
    real, imag = J._raise(real), J._raise(imag)
    _check_pair("hfft", real, imag)
    (axis,) = _axes_in_order(axis, real.ndim)
    n = 2 * (real.shape[axis] - 1)
    return irfft(real, imag.mul(-1), axis).mul(n)


def ihfft(a: Tracer, axis: int = -1):
    a = J._raise(a)
    (axis,) = _axes_in_order(axis, a.ndim)
    n = a.shape[axis]
    re, im = rfft(a, axis)
    return re.div(n), im.mul(-1).div(n)


def _check_frequency_args(name: str, n, d):
    if not isinstance(n, int) or n < 1:
        raise ValueError(f"jax.numpy.fft.{name}: n must be a positive integer, got {n}")
    if not math.isfinite(d) or d == 0:
        raise ValueError(f"jax.numpy.fft.{name}: d must be a finite non-zero number, got {d}")


def fftfreq(n: int, d: float = 1.0):
    """Sample frequencies as host float32 data, computed in double and rounded once, the way the reference builds the
    array it uploads (numpy-fft.ts:347-356)."""
    import numpy as _np
    _check_frequency_args("fftfreq", n, d)
    scale = 1 / (n * d)
    vals = [i * scale for i in range((n - 1) // 2 + 1)] + [i * scale for i in range(-(n // 2), 0)]
    return _np.asarray(vals, dtype=_np.float32)


def rfftfreq(n: int, d: float = 1.0):
    import numpy as _np
    _check_frequency_args("rfftfreq", n, d)
    scale = 1 / (n * d)
    return _np.asarray([i * scale for i in range(n // 2 + 1)], dtype=_np.float32)


def fftshift(a: Tracer, axes=None):
    a = J._raise(a)
    order = _axes_in_order(axes, a.ndim)
    return roll(a, [a.shape[ax] // 2 for ax in order], order)


def ifftshift(a: Tracer, axes=None):
    a = J._raise(a)
    order = _axes_in_order(axes, a.ndim)
    return roll(a, [-(a.shape[ax] // 2) for ax in order], order)


# ---- further distributions (src/library/random.ts:146-700), all built on uniform / normal above ------------------------

def _split2(key: Tracer):
    ka, kb = J.split(random_split(key, 2), 0, [1, 1])
    return ka.reshape([2]), kb.reshape([2])


def random_ball(key: Tracer, d: int, p: float = 2, shape: Sequence[int] = ()):
    """Uniform in the unit d-ball: a normal direction scaled by u^(1/d) (random.ts:146-171)."""
    if not isinstance(d, int) or d <= 0:
        raise ValueError(f"ball: dimension must be a positive integer, got {d}")
    if p != 2:
        raise ValueError("ball: only the Euclidean p=2 case is supported")
    k1, k2 = _split2(key)
    z = random_normal(k1, list(shape) + [d])
    nrm = J.sqrt(z.mul(z).sum(-1, keepdims=True))
    radius = J.exp(J.log(random_uniform(k2, list(shape) + [1])).mul(1 / d))
    return z.div(nrm).mul(radius)


def random_bernoulli(key: Tracer, p=0.5, shape: Sequence[int] = ()):
    return J.less(random_uniform(key, shape), p)


def random_gumbel(key: Tracer, shape: Sequence[int] = ()):
    return J.neg(J.log(J.neg(log1p(J.neg(random_uniform(key, shape))))))  # -log(-log(1 - u))


def random_categorical(key: Tracer, logits: Tracer, axis: int = -1, shape: Optional[Sequence[int]] = None, replace: bool = True):
    """Gumbel-max (with replacement) or Gumbel top-k (without) over `axis` of the logits (random.ts:203-262)."""
    logits = J._raise(logits)
    (axis,) = J._normalize_axis(axis, logits.ndim)
    numCategories = logits.shape[axis]
    batchShape = [d for i, d in enumerate(logits.shape) if i != axis]
    if shape is None:
        shape = batchShape
    else:
        shape = list(shape)
        if list(J.generalBroadcast(tuple(shape), tuple(batchShape))) != shape:
            raise ValueError(f"Shape {shape} is not broadcast-compatible with batch shape {batchShape}.")
    prefix = shape[:len(shape) - len(batchShape)]
    if replace:
        noise = random_gumbel(key, prefix + list(logits.shape))
        return argmax(noise.add(logits), axis + len(prefix))
    k = _int_prod(prefix)
    if k > numCategories:
        raise ValueError(f"Number of samples without replacement ({k}) cannot exceed number of categories ({numCategories}).")
    _values, indices = topK(random_gumbel(key, list(logits.shape)).add(logits), k, axis)
    return J._raise(indices).reshape(shape)


def random_cauchy(key: Tracer, shape: Sequence[int] = ()):
    return tan(random_uniform(key, shape).sub(0.5).mul(math.pi))


def random_randint(key: Tracer, minval: int, maxval: int, shape: Sequence[int] = (), dtype: DType = DType.Int32):
    if not isinstance(minval, int) or not isinstance(maxval, int):
        raise ValueError("randint: minval and maxval must be integers")
    if minval >= maxval:
        raise ValueError(f"Invalid range: [{minval}, {maxval}).")
    if dtype not in (DType.Int32, DType.Uint32):
        raise ValueError(f"randint: dtype must be int32 or uint32, got {dtype}")
    if dtype == DType.Uint32 and minval < 0:
        raise ValueError("randint: uint32 dtype requires minval >= 0")
    return J.mod(random_bits(key, shape), maxval - minval).astype(dtype).add(minval)


def random_permutation(key: Tracer, x, axis: int = 0):
    """argsort of uniforms; an array is gathered along `axis` by that permutation (random.ts:542-566)."""
    if isinstance(x, int):
        if x < 0:
            raise ValueError(f"permutation: x must be a non-negative integer, got {x}")
        return argsort(random_uniform(key, [x])).astype(DType.Int32)
    arr = J._raise(x)
    (axis,) = J._normalize_axis(axis, arr.ndim)
    return J.gather(arr, [random_permutation(key, arr.shape[axis])], [axis], axis)


def random_choice(key: Tracer, a, shape: Sequence[int] = (), replace: bool = True, p=None, axis: int = 0):
    shape = list(shape)
    values = None
    if isinstance(a, int):
        if a < 0:
            raise ValueError(f"choice: a must be a non-negative integer, got {a}")
        n = a
    else:
        values = J._raise(a)
        (axis,) = J._normalize_axis(axis, values.ndim)
        n = values.shape[axis]
    if p is not None:
        idx = random_categorical(key, J.log(p), shape=shape, replace=replace)
    elif replace:
        idx = random_randint(key, 0, n, shape)
    else:
        k = _int_prod(shape)
        if k > n:
            raise ValueError(f"Number of samples without replacement ({k}) cannot exceed population size ({n}).")
        idx = J.shrink(random_permutation(key, n), [(0, k)]).reshape(shape)
    return idx if values is None else J.gather(values, [idx], [axis], axis)


def random_rademacher(key: Tracer, shape: Sequence[int] = (), dtype: DType = DType.Int32):
    if dtype in (DType.Uint32, DType.Bool):
        raise ValueError(f"rademacher: unsupported dtype {dtype}")
    return J.where(random_bernoulli(key, 0.5, shape), J.scalar(1, dtype), J.scalar(-1, dtype))


def random_maxwell(key: Tracer, shape: Sequence[int] = ()):
    z = random_normal(key, list(shape) + [3])
    return J.sqrt(z.mul(z).sum(-1))


def random_doubleSidedMaxwell(key: Tracer, loc, scale, shape: Sequence[int] = ()):
    k1, k2 = _split2(key)
    return random_rademacher(k1, shape, DType.Float32).mul(random_maxwell(k2, shape)).mul(scale).add(loc)


def random_geometric(key: Tracer, p, shape: Sequence[int] = (), dtype: DType = DType.Int32):
    return J.floor(log1p(J.neg(random_uniform(key, shape))).div(log1p(J.neg(J._raise(p))))).add(1).astype(dtype)


def random_laplace(key: Tracer, shape: Sequence[int] = ()):
    centered = random_uniform(key, shape).sub(0.5)
    return sign(centered).mul(log1p(absolute(centered).mul(-2)).mul(-1))


def random_logistic(key: Tracer, shape: Sequence[int] = ()):
    u = random_uniform(key, shape)
    return J.log(u).sub(log1p(J.neg(u)))


def random_lognormal(key: Tracer, sigma=1, shape: Sequence[int] = ()):
    return J.exp(random_normal(key, shape).mul(sigma))


def random_multivariateNormal(key: Tracer, mean: Tracer, cov: Tracer, shape: Sequence[int] = ()):
    """mean + L z with L the Cholesky factor of the covariance (random.ts:475-509)."""
    mean, cov = J._raise(mean), J._raise(cov)
    n = mean.shape[-1]
    if cov.ndim < 2 or cov.shape[-1] != n or cov.shape[-2] != n:
        raise ValueError(f"Invalid covariance shape: {list(cov.shape)}. Expected last two dimensions to be [{n}, {n}].")
    out: Sequence[int] = tuple(shape)
    for s in (tuple(mean.shape[:-1]), tuple(cov.shape[:-2])):
        out = J.generalBroadcast(tuple(out), s)
    Lc = linalgCholesky(cov)
    z = random_normal(key, list(out) + [n])
    return matvec(Lc, z).add(mean)


def random_pareto(key: Tracer, b, shape: Sequence[int] = ()):
    return J.exp(random_exponential(key, shape).div(b))


def random_rayleigh(key: Tracer, scale=1, shape: Sequence[int] = ()):
    return J.sqrt(random_exponential(key, shape).mul(2)).mul(scale)


def random_triangular(key: Tracer, left, mode, right, shape: Sequence[int] = ()):
    left, mode, right = _as_array(left), _as_array(mode), _as_array(right)
    u = random_uniform(key, shape)
    width, leftSpan, rightSpan = right.sub(left), mode.sub(left), right.sub(mode)
    cond = J.less(u, leftSpan.div(width))
    lower = left.add(J.sqrt(u.mul(width).mul(leftSpan)))
    upper = right.sub(J.sqrt(J.neg(u).add(1).mul(width).mul(rightSpan)))
    return J.where(cond, lower, upper)


def random_weibullMin(key: Tracer, scale, concentration, shape: Sequence[int] = ()):
    return J.mul(scale, J.exp(J.log(random_exponential(key, shape)).div(concentration)))


def frexp(x: Tracer):
    """Mantissa and exponent with x = m * 2^e, through floor(log2|x|) + 1 (numpy.ts:2799-2809)."""
    x = J._raise(x)
    exponent = J.where(J.equal(x, 0), 0, J.floor(log2(absolute(x))).add(1).astype(DType.Int32))
    return [x.div(exp2(exponent.astype(x.dtype))), exponent]


def flipud(x: Tracer):
    return J.flip(x, 0)


def fliplr(x: Tracer):
    return J.flip(x, 1)
