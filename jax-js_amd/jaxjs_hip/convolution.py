"""View algebra of convolution and pooling: how the `Conv` and `Pool` primitives become a broadcast
multiply under an Add reduction (or a windowed reduction) purely by re-viewing their inputs.

Restates src/frontend/convolution.ts: `checkConvShape` :58-122, `checkPoolShape` :124-146, `pool` :157-262,
`applyDilation` :374-395, `prepareConv` :403-442.  Shapes: lhs `[*vmap, batch, in_channels, *spatial]`,
rhs `[*vmap, out_channels, in_channels, *kernel]`.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

from .shape import ShapeTracker, prod

Pair = Tuple[int, int]


@dataclass
class ConvParams:
    vmapDims: int = 0
    strides: List[int] = field(default_factory=list)
    padding: List[Pair] = field(default_factory=list)
    lhsDilation: List[int] = field(default_factory=list)
    rhsDilation: List[int] = field(default_factory=list)


def _broadcast_shapes(a, b):
    out = []
    for i in range(max(len(a), len(b))):
        x = a[len(a) - 1 - i] if i < len(a) else 1
        y = b[len(b) - 1 - i] if i < len(b) else 1
        if x != y and x != 1 and y != 1:
            raise ValueError(f"incompatible shapes for broadcasting: {list(a)} and {list(b)}")
        out.append(max(x, y))
    return list(reversed(out))


def checkConvShape(lhsShape: Sequence[int], rhsShape: Sequence[int], p: ConvParams) -> List[int]:
    if len(lhsShape) != len(rhsShape):
        raise ValueError(f"conv() requires inputs with the same number of dimensions, got {len(lhsShape)} and {len(rhsShape)}")
    v = p.vmapDims
    n = len(lhsShape) - 2 - v
    if n < 0:
        raise ValueError("conv() requires at least 2D inputs")
    for name, val in (("strides", p.strides), ("padding", p.padding), ("lhsDilation", p.lhsDilation), ("rhsDilation", p.rhsDilation)):
        if len(val) != n:
            raise ValueError(f"conv() {name} != spatial dims")
    if lhsShape[v + 1] != rhsShape[v + 1]:
        raise ValueError(f"conv() input channels: {lhsShape[v + 1]} != {rhsShape[v + 1]}")
    out = _broadcast_shapes(lhsShape[:v], rhsShape[:v]) + [lhsShape[v], rhsShape[v]]
    for i in range(n):
        if p.strides[i] <= 0 or p.lhsDilation[i] <= 0 or p.rhsDilation[i] <= 0:
            raise ValueError("conv() strides and dilations must be positive integers")
        x, k = lhsShape[i + v + 2], rhsShape[i + v + 2]
        if k <= 0:
            raise ValueError("conv() kernel size must be positive")
        pl, pr = p.padding[i]
        if pl < -x or pr < -x or pl + pr < -x:
            raise ValueError(f"conv() padding[{i}]=({pl},{pr}) is too negative for input size {x}")
        kernel = (k - 1) * p.rhsDilation[i] + 1
        size = max((x - 1) * p.lhsDilation[i] + 1, 0) + pl + pr
        if kernel > size:
            raise ValueError(f"conv() kernel size {kernel} > input size {size} in dimension {i}")
        out.append(-(-(size - kernel + 1) // p.strides[i]))
    return out


def checkPoolShape(inShape: Sequence[int], window: Sequence[int], strides: Sequence[int]) -> List[int]:
    if len(strides) != len(window):
        raise ValueError("pool() strides != window dims")
    if len(window) > len(inShape):
        raise ValueError("pool() window has more dimensions than input")
    out = list(inShape[:len(inShape) - len(window)])
    for i, (k, s) in enumerate(zip(window, strides)):
        size = inShape[len(inShape) - len(window) + i]
        if k <= 0 or s <= 0:
            raise ValueError("pool() window and strides must be positive integers")
        if k > size:
            raise ValueError(f"pool() window[{i}]={k} > input size {size}")
        out.append(-(-(size - k + 1) // s))
    return out + list(window)


def pool(st: ShapeTracker, ks: Sequence[int], strides=1, dilation=1) -> ShapeTracker:
    """Re-view `[..., *spatial]` as `[..., *out, *ks]`: element (o, k) is input position o*s + k*d."""
    ks = list(ks)
    if not ks:
        return st
    if len(st.shape) < len(ks):
        raise ValueError("pool() called with too many dimensions")
    s_ = [strides] * len(ks) if isinstance(strides, int) else list(strides)
    d_ = [dilation] * len(ks) if isinstance(dilation, int) else list(dilation)
    if any(s <= 0 for s in s_) or any(d <= 0 for d in d_):
        raise ValueError("pool() strides and dilation must be positive integers")
    nk = len(ks)
    noop = list(st.shape[:-nk])
    i_ = list(st.shape[-nk:])
    o_ = [-(-(i - d * (k - 1)) // s) for i, d, k, s in zip(i_, d_, ks, s_)]
    nn = len(noop)

    if all(d == 1 for d in d_) and all(k <= s for k, s in zip(ks, s_)):
        # Non-overlapping windows (e.g. max pooling): pad/shrink to o*s, split, keep the first k of each s.
        st = st.padOrShrink([(0, 0)] * nn + [(0, o * s - i) for i, o, s in zip(i_, o_, s_)])
        st = st.reshape(noop + [x for o, s in zip(o_, s_) for x in (o, s)])
        st = st.shrink([(0, x) for x in noop] + [pr for o, k in zip(o_, ks) for pr in ((0, o), (0, k))])
        return st.permute(list(range(nn)) + [nn + 2 * j for j in range(nk)] + [nn + 2 * j + 1 for j in range(nk)])

    # General case: repeat each row so that consecutive repeats are shifted by the dilation, then stride.
    f_ = [1 + int(o * s > i - d * (k - 1)) for o, s, i, d, k in zip(o_, s_, i_, d_, ks)]
    kidf = list(zip(ks, i_, d_, f_))
    st = st.repeat([1] * nn + [-(-(k * (i * f + d)) // i) for k, i, d, f in kidf])
    st = st.shrink([(0, x) for x in noop] + [(0, k * (i * f + d)) for k, i, d, f in kidf])
    st = st.reshape(noop + [x for k, i, d, f in kidf for x in (k, i * f + d)])
    kos = list(zip(ks, o_, s_))
    st = st.shrink([(0, x) for x in noop] + [pr for k, o, s in kos for pr in ((0, k), (0, o * s))])
    st = st.reshape(noop + [x for k, o, s in kos for x in (k, o, s)])
    st = st.shrink([(0, x) for x in noop] + [pr for k, o, s in kos for pr in ((0, k), (0, o), (0, 1))])
    st = st.reshape(noop + [x for k, o, s in kos for x in (k, o)])
    return st.permute(list(range(nn)) + [nn + 2 * j + 1 for j in range(nk)] + [nn + 2 * j for j in range(nk)])


def poolTranspose(st: ShapeTracker, inShape: Sequence[int], ks: Sequence[int], strides=1, dilation=1) -> ShapeTracker:
    """The adjoint view of `pool` (src/frontend/convolution.ts:274-378): re-view a pooled array `[..., *out, *ks]` as
    `[*inShape, *repeats]` so that summing the trailing axes adds up, for every input position, the pooled elements
    that were read from it (masked where there is none).  This is the Kernel a transform emits for the cotangent of a
    window reduction or convolution input; nothing in the forward library traces it."""
    ks = list(ks)
    if not ks:
        return st
    nk = len(ks)
    s_ = [strides] * nk if isinstance(strides, int) else list(strides)
    d_ = [dilation] * nk if isinstance(dilation, int) else list(dilation)
    noop = list(inShape[:-nk])
    nn = len(noop)
    i_ = list(inShape[-nk:])
    o_ = [-(-(i - d * (k - 1)) // s) for i, d, k, s in zip(i_, d_, ks, s_)]

    if all(d == 1 for d in d_) and all(k <= s for k, s in zip(ks, s_)):
        # Non-overlapping windows: interleave (o, k) again, pad each k up to its stride, merge, fit to the input extent.
        st = st.permute(list(range(nn)) + [x for j in range(nk) for x in (nn + j, nn + nk + j)])
        st = st.pad([(0, 0)] * nn + [pr for s, k in zip(s_, ks) for pr in ((0, 0), (0, s - k))])
        st = st.reshape(noop + [o * s for o, s in zip(o_, s_)])
        st = st.padOrShrink([(0, 0)] * nn + [(0, i - o * s) for i, o, s in zip(i_, o_, s_)])
        return st.reshape(list(st.shape) + [1] * nk)  # the repeat axes the general form has, of extent 1

    if o_ != list(st.shape[nn:nn + nk]):
        raise ValueError("poolTranspose() called with mismatched output shape")
    f_ = [1 + int(o * s > i - d * (k - 1)) for o, s, i, d, k in zip(o_, s_, i_, d_, ks)]
    kidf = list(zip(ks, i_, d_, f_))
    kos = list(zip(ks, o_, s_))
    # every step of pool()'s general form, undone in reverse order
    st = st.permute(list(range(nn)) + [x for j in range(nk) for x in (nn + nk + j, nn + j)])
    st = st.reshape(noop + [x for k, o, s in kos for x in (k, o, 1)])
    st = st.pad([(0, 0)] * nn + [pr for s in s_ for pr in ((0, 0), (0, 0), (0, s - 1))])
    st = st.reshape(noop + [x for k, o, s in kos for x in (k, o * s)])
    st = st.pad([(0, 0)] * nn + [pr for (k, i, d, f), o, s in zip(kidf, o_, s_) for pr in ((0, 0), (0, i * f + d - o * s))])
    st = st.reshape(noop + [k * (i * f + d) for k, i, d, f in kidf])
    st = st.pad([(0, 0)] * nn + [(0, -(-(k * (i * f + d)) // i) * i - k * (i * f + d)) for k, i, d, f in kidf])
    st = st.reshape(noop + [x for k, i, d, f in kidf for x in (-(-(k * (i * f + d)) // i), i)])
    return st.permute(list(range(nn)) + [nn + 2 * j + 1 for j in range(nk)] + [nn + 2 * j for j in range(nk)])


def applyDilation(st: ShapeTracker, dilation: Sequence[int]) -> ShapeTracker:
    """Insert `s-1` zeros between the elements of the last axes (transposed convolution)."""
    if all(s == 1 for s in dilation):
        return st
    s_ = list(dilation)
    n = len(s_)
    prefix, k_ = list(st.shape[:-n]), list(st.shape[-n:])
    st = st.reshape(prefix + [x for k in k_ for x in (k, 1)])
    st = st.pad([(0, 0)] * len(prefix) + [pr for s in s_ for pr in ((0, 0), (0, s - 1))])
    st = st.reshape(prefix + [k * s for k, s in zip(k_, s_)])
    return st.shrink([(0, p) for p in prefix] + [(0, (k - 1) * s + 1) for k, s in zip(k_, s_)])


def prepareConv(stX: ShapeTracker, stY: ShapeTracker, p: ConvParams) -> Tuple[ShapeTracker, ShapeTracker]:
    """Views of lhs and rhs with shapes `[*vmap, batch, 1, *out, C*prod(ks)]` and `[*vmap, 1, O, 1.., C*prod(ks)]`."""
    v = p.vmapDims
    n = len(stX.shape) - 2 - v
    vmapShape = list(stX.shape[:v])
    stX = applyDilation(stX, p.lhsDilation)
    ks = list(stY.shape[v + 2:])
    stX = stX.padOrShrink([(0, 0)] * (v + 2) + [tuple(x) for x in p.padding])
    stX = pool(stX, ks, p.strides, p.rhsDilation)
    stX = stX.moveaxis(v + 1, v + n + 1)
    moved = list(stX.shape)
    # after the move: [*vmap, batch, *out, C, *ks]
    stX = stX.reshape(vmapShape + [moved[v], 1] + moved[v + 1:v + n + 1] + [moved[v + n + 1] * prod(ks)])
    stY = stY.reshape(vmapShape + [1, stY.shape[v]] + [1] * n + [stY.shape[v + 1] * prod(ks)])
    return stX, stY
