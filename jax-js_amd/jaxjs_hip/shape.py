"""Lazy shape tracking: `View` (shape/strides/offset/mask) and `ShapeTracker` (a chain of views).

Host-side mirror of the reference's shape module (reference: src/shape.ts).  A `GlobalView`
node in the IR carries a ShapeTracker; `toAluExp` turns N-d logical indices into a flat buffer
index plus a validity predicate (src/shape.ts:277-300, 690-700).  All values are Python ints;
views are immutable and hashable so that expressions holding them can be interned.
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

from .alu import AluExp

Pair = Tuple[int, int]


def prod(xs: Sequence[int]) -> int:
    out = 1
    for x in xs:
        out *= x
    return out


def _canonical_strides(shape: Sequence[int], strides: Sequence[int]) -> Tuple[int, ...]:
    # A size-1 axis never moves in memory, so its stride is normalised to 0.
    return tuple(0 if s == 1 else int(st) for s, st in zip(shape, strides))


def _row_major(shape: Sequence[int]) -> Tuple[int, ...]:
    strides = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        strides[i - 1] = strides[i] * shape[i]
    return _canonical_strides(shape, strides)


def _merge_dims(shape, strides, mask) -> List[Tuple[int, int, int]]:
    """Fuse neighbouring axes that walk memory like one axis.

    Returns `(merged_size, stride, real_size)` triples (same contract as `mergeDims` in
    src/shape.ts:60-101): `real_size` is how much of the merged extent really advances in
    memory; beyond it the data repeats (stride 0) or is masked to a single index.
    """
    if not shape:
        return []
    assert len(shape) == len(strides) and (mask is None or len(mask) == len(shape))
    out = [[shape[0], strides[0], shape[0] if strides[0] != 0 else 0]]
    # An axis whose mask admits exactly one index can be absorbed by the next one.
    absorbing = (mask[0][1] - mask[0][0] == 1) if mask else (shape[0] == 1)
    for i in range(1, len(shape)):
        s, st = shape[i], strides[i]
        if s == 1:
            continue
        last_s, last_st, last_real = out[-1]
        if absorbing or last_st == s * st:
            out[-1] = [last_s * s, st, s if absorbing else last_real * s]
        else:
            out.append([s, st, s])
        absorbing = (mask[i][1] - mask[i][0] == 1) if mask else False
    return [tuple(t) for t in out]


def _reshape_mask(mask: Sequence[Pair], old_shape: Sequence[int], new_shape: Sequence[int]) -> Optional[List[Pair]]:
    """Carry a mask through a reshape, or None when the masked box does not stay a box
    (same contract as `reshapeMask`, src/shape.ts:104-157).  Works right-to-left."""
    masks = list(mask)
    olds = list(old_shape)
    news = list(new_shape)

    def pop_mask():
        return masks.pop() if masks else (0, 1)

    def pop_old():
        return olds.pop() if olds else 1

    def pop_new():
        return news.pop() if news else 1

    out: List[Pair] = []
    stride = 1
    old_dim, new_dim, m = pop_old(), pop_new(), pop_mask()
    while len(out) < len(new_shape):
        lo, hi = m
        nxt = new_dim * stride
        if old_dim == nxt:
            out.append((lo // stride, (hi - 1) // stride + 1))
            stride = 1
            old_dim, new_dim, m = pop_old(), pop_new(), pop_mask()
        elif old_dim > nxt:
            if old_dim % nxt != 0:
                return None
            if (lo % nxt != 0 or hi % nxt != 0) and lo // nxt != (hi - 1) // nxt:
                return None
            out.append(((lo % nxt) // stride, ((hi - 1) % nxt) // stride + 1))
            stride, new_dim = nxt, pop_new()
        else:
            nm = pop_mask()
            if m != (0, old_dim) and lo != hi and nm[1] - nm[0] != 1:
                return None
            m = (nm[0] * old_dim + lo, (nm[1] - 1) * old_dim + hi)
            old_dim *= pop_old()
    out.reverse()
    return out


def unravel(shape: Sequence[int], offset: int) -> List[int]:
    """Row-major position of a flat offset (src/shape.ts:619-628); the top axis wraps."""
    idxs = []
    acc = 1
    for d in reversed(shape):
        idxs.append((offset // acc) % d if d else 0)
        acc *= d
    idxs.reverse()
    return idxs


def unravelAlu(shape: Sequence[int], offset: AluExp) -> List[AluExp]:
    """Expressions for `unravel` (src/shape.ts:631-640): `(offset / acc) % dim` per axis."""
    idxs = []
    acc = 1
    for d in reversed(shape):
        idxs.append(AluExp.mod(AluExp.idiv(offset, AluExp.i32(acc)), AluExp.i32(d)))
        acc *= d
    idxs.reverse()
    return idxs


class View:
    """One strided, optionally masked window onto a flat buffer (src/shape.ts:168-232).

    Element (i0..in) lives at `offset + sum(strides[k]*ik)` and reads as 0 where some index
    falls outside `mask[k] = (lo, hi)`.
    """

    __slots__ = ("shape", "strides", "offset", "mask", "_size", "_contig")

    def __init__(self, shape, strides, offset, mask):
        self.shape: Tuple[int, ...] = tuple(shape)
        self.strides: Tuple[int, ...] = tuple(strides)
        self.offset: int = int(offset)
        self.mask: Optional[Tuple[Pair, ...]] = None if mask is None else tuple((int(a), int(b)) for a, b in mask)
        self._size = None
        self._contig = None

    @staticmethod
    def create(shape: Sequence[int], strides: Optional[Sequence[int]] = None, offset: int = 0, mask=None) -> "View":
        shape = tuple(int(s) for s in shape)
        if any(s < 0 for s in shape):
            raise ValueError("View shape must be non-negative")
        strides = list(_canonical_strides(shape, strides) if strides is not None else _row_major(shape))
        if 0 in shape:
            return View(shape, [0] * len(shape), 0, None)
        if mask is not None:
            mask = [(int(a), int(b)) for a, b in mask]
            if all(m == (0, s) for m, s in zip(mask, shape)):
                mask = None
        if mask is not None:
            # Axes masked down to (at most) one index stop moving: fold them into the offset.
            single = [i for i, (b, e) in enumerate(mask) if b + 1 >= e]
            if single:
                if any(b >= e for b, e in mask):
                    strides = [0] * len(shape)
                    offset = 0
                    mask = [(0, 0)] * len(shape)
                for i in single:
                    offset += strides[i] * mask[i][0]
                    strides[i] = 0
        return View(shape, strides, offset, mask)

    def key(self):
        return (self.shape, self.strides, self.offset, self.mask)

    def __eq__(self, other):
        return isinstance(other, View) and self.key() == other.key()

    def __hash__(self):
        return hash(self.key())

    def __repr__(self):
        return f"View(shape={list(self.shape)}, strides={list(self.strides)}, offset={self.offset}, mask={self.mask})"

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def size(self) -> int:
        if self._size is None:
            self._size = prod(self.shape)
        return self._size

    @property
    def contiguous(self) -> bool:
        """Identity view: row-major, offset 0, unmasked (src/shape.ts:244-253)."""
        if self._contig is None:
            self._contig = self.size == 0 or (
                self.offset == 0 and self.mask is None and self.strides == _row_major(self.shape)
            )
        return self._contig

    def dataRange(self) -> Tuple[int, int]:
        """Half-open range of buffer elements this view can touch (src/shape.ts:256-274)."""
        if self.size == 0 or (self.mask and self.mask[0][0] == self.mask[0][1]):
            return (0, 0)
        lo = hi = self.offset
        for i in range(self.ndim):
            b, e = self.mask[i] if self.mask else (0, self.shape[i])
            e -= 1
            s = self.strides[i]
            if s > 0:
                lo += s * b
                hi += s * e
            elif s < 0:
                lo += s * e
                hi += s * b
        return (lo, hi + 1)

    def toAluExp(self, idxs: Sequence[AluExp]) -> Tuple[AluExp, AluExp]:
        """(flat index, validity) expressions for the given per-axis indices (src/shape.ts:277-300)."""
        iexpr = AluExp.i32(self.offset)
        vexpr = AluExp.bool(True)
        for i in range(self.ndim - 1, -1, -1):
            idx = idxs[i]
            if self.shape[i] != 1 and self.strides[i] != 0:
                iexpr = AluExp.add(AluExp.mul(idx, AluExp.i32(self.strides[i])), iexpr)
            if self.mask:
                lo, hi = self.mask[i]
                if lo != 0:
                    vexpr = AluExp.mul(AluExp.cmplt(idx, AluExp.i32(lo)).not_(), vexpr)
                if hi != self.shape[i]:
                    vexpr = AluExp.mul(AluExp.cmplt(idx, AluExp.i32(hi)), vexpr)
        return iexpr, vexpr

    # -- movement ops --------------------------------------------------------------------------
    def _resize(self, arg: Sequence[Pair], mask=None) -> "View":
        offset = sum(s * a[0] for s, a in zip(self.strides, arg))
        if self.mask:
            moved = [
                (max(0, min(mx - b, e - b)), max(0, min(my - b, e - b)))
                for (mx, my), (b, e) in zip(self.mask, arg)
            ]
            mask = [(max(a[0], m[0]), min(a[1], m[1])) for a, m in zip(mask, moved)] if mask else moved
        return View.create([e - b for b, e in arg], self.strides, self.offset + offset, mask)

    def pad(self, arg: Sequence[Pair]) -> "View":
        """Zero-pad each axis by (before, after) (src/shape.ts:457-465)."""
        if len(arg) != self.ndim or not all(b >= 0 and e >= 0 for b, e in arg):
            raise ValueError(f"invalid pad {list(arg)} for {list(self.shape)}")
        if all(b == 0 and e == 0 for b, e in arg):
            return self
        window = [(-b, s + e) for (b, e), s in zip(arg, self.shape)]
        mask = [(b, s + b) for (b, _), s in zip(arg, self.shape)]
        return self._resize(window, mask)

    def shrink(self, arg: Sequence[Pair]) -> "View":
        """Sub-box [b,e) per axis (src/shape.ts:468-476)."""
        if len(arg) != self.ndim or not all(0 <= b <= e <= s for (b, e), s in zip(arg, self.shape)):
            raise ValueError(f"invalid shrink {list(arg)} for {list(self.shape)}")
        return self._resize(arg)

    def expand(self, new_shape: Sequence[int]) -> "View":
        """Broadcast size-1 axes (src/shape.ts:505-530)."""
        new_shape = tuple(new_shape)
        if len(new_shape) != self.ndim or any(n != s and s != 1 for n, s in zip(new_shape, self.shape)):
            raise ValueError(f"Can't expand {list(self.shape)} into {list(new_shape)}")
        if self.size == 0:
            return View.create(new_shape)
        mask = None
        if self.mask:
            mask = [
                m if s == n else ((0, n) if m == (0, 1) else (0, 0))
                for m, s, n in zip(self.mask, self.shape, new_shape)
            ]
        return View.create(new_shape, self.strides, self.offset, mask)

    def permute(self, axis: Sequence[int]) -> "View":
        if sorted(axis) != list(range(self.ndim)):
            raise ValueError(f"Invalid permutation {list(axis)} of len {self.ndim}")
        return View.create(
            [self.shape[a] for a in axis],
            [self.strides[a] for a in axis],
            self.offset,
            [self.mask[a] for a in axis] if self.mask else None,
        )

    def flip(self, arg: Sequence[bool]) -> "View":
        if len(arg) != self.ndim:
            raise ValueError(f"Invalid flip {list(arg)} for {list(self.shape)}")
        strides = list(self.strides)
        offset = self.offset
        mask = list(self.mask) if self.mask else None
        for i, f in enumerate(arg):
            if f:
                s = self.shape[i]
                strides[i] = -strides[i]
                offset += (s - 1) * self.strides[i]
                if mask:
                    mask[i] = (s - mask[i][1], s - mask[i][0])
        return View.create(self.shape, strides, offset, mask)

    def reshape(self, new_shape: Sequence[int]) -> Optional["View"]:
        """Reinterpret with a new shape if one view can express it, else None (src/shape.ts:561-612)."""
        new_shape = tuple(int(s) for s in new_shape)
        if new_shape == self.shape:
            return self
        if any(s < 0 for s in new_shape):
            raise ValueError(f"Reshape cannot have negative numbers {list(new_shape)}")
        if self.size != prod(new_shape):
            raise ValueError(f"Reshape size {list(self.shape)} -> {list(new_shape)}")
        if self.size == 0:
            return View.create(new_shape)
        if len(new_shape) == 0 and self.mask and any(b == e for b, e in self.mask):
            return None
        if self.contiguous:
            return View.create(new_shape)

        # Walk merged memory runs from the innermost outwards and carve the new axes from them.
        rstrides: List[int] = []
        cursor = len(new_shape)
        for merged, stride, real in reversed(_merge_dims(self.shape, self.strides, self.mask)):
            acc = 1
            while acc < merged and cursor > 0:
                cursor -= 1
                rstrides.append(stride * acc)
                acc *= new_shape[cursor]
                if acc >= real:
                    stride = 0
            if acc != merged:
                return None
        new_strides = [0] * (len(new_shape) - len(rstrides)) + rstrides[::-1]
        if not self.mask:
            return View.create(new_shape, new_strides, self.offset)
        new_mask = _reshape_mask(self.mask, self.shape, new_shape)
        if new_mask is None:
            return None
        offset = self.offset
        offset += sum(s * m[0] for s, m in zip(self.strides, self.mask))
        offset -= sum(s * m[0] for s, m in zip(new_strides, new_mask))
        return View.create(new_shape, new_strides, offset, new_mask)

    def minify(self) -> "View":
        """Collapse to the fewest axes that describe the same walk (src/shape.ts:448-454)."""
        nv = self.reshape([m[0] for m in _merge_dims(self.shape, self.strides, self.mask)])
        return nv if nv is not None else self

    def compose(self, v1: "View") -> Optional["View"]:
        """Single view equal to "self, then v1", or None when two views are needed.

        `v1` indexes the row-major space of `self.shape` (src/shape.ts:312-445).  Each stride of
        v1 is decomposed into per-axis steps of self; the composition is affine exactly when
        walking v1's whole extent never carries across an axis of self.  This implementation is
        conservative: a masked `self` composes only when v1 stays inside the mask.
        """
        v2 = self
        if v2.contiguous:
            return v1
        if v1.contiguous:
            if v1.shape == v2.shape:
                return v2
            if v1.size == v2.size:
                r = v2.reshape(v1.shape)
                if r is not None:
                    return r
        if v1.mask is not None:
            inner = v2.compose(v1.shrink(v1.mask))
            if inner is None:
                return None
            return inner.pad([(m[0], s - m[1]) for m, s in zip(v1.mask, v1.shape)])
        if v1.size == 0:
            return View.create(v1.shape)
        lo, hi = v1.dataRange()
        if lo < 0 or hi > v2.size:
            return None

        origin = unravel(v2.shape, v1.offset)
        steps: List[List[Tuple[int, int]]] = [[] for _ in range(v2.ndim)]  # per v2 axis: (v1 axis, step)
        strides = [0] * v1.ndim
        for d1, st in enumerate(v1.strides):
            if st == 0 or v1.shape[d1] == 1:
                continue
            moved = unravel(v2.shape, v1.offset + st)
            for d2 in range(v2.ndim):
                diff = moved[d2] - origin[d2]
                if diff:
                    steps[d2].append((d1, diff))
                    strides[d1] += diff * v2.strides[d2]

        # Check for carries, merging adjacent axes of self where the walk spills over.
        groups: List[Tuple[int, int, int]] = []
        msize, mlo, mhi = 1, 0, 0
        for d2 in range(v2.ndim - 1, -1, -1):
            tmin = tmax = origin[d2]
            for d1, s1 in steps[d2]:
                if s1 > 0:
                    tmax += (v1.shape[d1] - 1) * s1
                else:
                    tmin += (v1.shape[d1] - 1) * s1
            mlo += tmin * msize
            mhi += tmax * msize
            msize *= v2.shape[d2]
            if mlo >= 0 and mhi < msize:
                groups.append((msize, mlo, mhi))
                msize, mlo, mhi = 1, 0, 0
        if mlo != 0 or mhi != 0:
            return None
        groups.reverse()
        merged_shape = tuple(g[0] for g in groups)
        if merged_shape != v2.shape:
            r = v2.reshape(merged_shape)
            if r is None or r.shape == v2.shape:
                return None
            return r.compose(v1)

        if v2.mask is not None:
            for (b, e), (_, tmin, tmax) in zip(v2.mask, groups):
                if not (b <= tmin and tmax < e):
                    return None

        offset = v2.offset + sum(o * s for o, s in zip(origin, v2.strides))
        return View.create(v1.shape, strides, offset, None)


class ShapeTracker:
    """A chain of views, each indexing the row-major space of the previous one (src/shape.ts:648-806)."""

    __slots__ = ("views",)

    def __init__(self, views: Sequence[View]):
        self.views: Tuple[View, ...] = tuple(views)

    def key(self):
        return tuple(v.key() for v in self.views)

    def __eq__(self, other):
        return isinstance(other, ShapeTracker) and self.views == other.views

    def __hash__(self):
        return hash(self.key())

    def __repr__(self):
        return f"ShapeTracker({list(self.views)})"

    @staticmethod
    def fromShape(shape: Sequence[int]) -> "ShapeTracker":
        return ShapeTracker([View.create(shape)])

    @property
    def contiguous(self) -> bool:
        return len(self.views) == 1 and self.views[0].contiguous

    @property
    def consecutive(self) -> bool:
        v = self.views[0]
        return len(self.views) == 1 and v.mask is None and v.strides == _row_major(v.shape)

    @property
    def lastStrides(self) -> List[int]:
        return list(self.views[-1].strides)

    @property
    def shape(self) -> List[int]:
        return list(self.views[-1].shape)

    @property
    def size(self) -> int:
        return self.views[-1].size

    def toAluExp(self, idxs: Sequence[AluExp]) -> Tuple[AluExp, AluExp]:
        """Chain the views innermost-last (src/shape.ts:690-700)."""
        iexpr, vexpr = self.views[-1].toAluExp(idxs)
        for view in reversed(self.views[:-1]):
            view = view.minify()
            i2, v2 = view.toAluExp(unravelAlu(view.shape, iexpr))
            iexpr = i2
            vexpr = AluExp.mul(vexpr, v2)
        return iexpr.simplify(), vexpr.simplify()

    def simplify(self) -> "ShapeTracker":
        views = list(self.views)
        while len(views) >= 2:
            merged = views[-2].compose(views[-1])
            if merged is None:
                break
            views[-2:] = [merged]
        return ShapeTracker(views)

    def compose(self, other: "ShapeTracker") -> "ShapeTracker":
        """Apply `other` after this tracker (src/shape.ts:652-659)."""
        if self.contiguous:
            return other
        ret = self
        for v in other.views:
            ret = ShapeTracker(ret.views + (v,)).simplify()
        return ret

    def _last(self, f) -> "ShapeTracker":
        return ShapeTracker(self.views[:-1] + (f(self.views[-1]),))

    def pad(self, arg):
        return self._last(lambda v: v.pad(arg))

    def shrink(self, arg):
        return self._last(lambda v: v.shrink(arg))

    def expand(self, new_shape):
        return self._last(lambda v: v.expand(new_shape))

    def permute(self, axis):
        return self._last(lambda v: v.permute(axis))

    def flip(self, arg):
        return self._last(lambda v: v.flip(arg))

    def reshape(self, new_shape) -> "ShapeTracker":
        nv = self.views[-1].reshape(new_shape)
        if nv is None:
            return ShapeTracker(self.views + (View.create(new_shape),))
        return ShapeTracker(self.views[:-1] + (nv,))

    # -- composite movement ops (src/shape.ts:737-805) -----------------------------------------
    def broadcast(self, new_shape: Sequence[int], axis: Sequence[int]) -> "ShapeTracker":
        st = self
        if axis:
            unsq = list(st.shape)
            for i in sorted(axis):
                unsq.insert(i, 1)
            st = st.reshape(unsq)
        return st.expand(new_shape)

    def repeat(self, reps: Sequence[int], tile: bool = True) -> "ShapeTracker":
        if len(reps) > len(self.shape):
            raise ValueError(f"Too many repeats {list(reps)} for shape {self.shape}")
        if any(c <= 0 for c in reps):
            raise ValueError(f"Invalid repeats {list(reps)}")
        if not reps:
            return self
        n = len(reps)
        noop, shape = self.shape[:-n], self.shape[-n:]
        wide: List[int] = list(noop)
        for s, r in zip(shape, reps):
            wide += [r, s] if tile else [s, r]
        axes = [len(noop) + 2 * i + (0 if tile else 1) for i in range(n)]
        return self.broadcast(wide, axes).reshape(list(noop) + [s * r for s, r in zip(shape, reps)])

    def moveaxis(self, i: int, j: int) -> "ShapeTracker":
        perm = list(range(len(self.shape)))
        perm.pop(i)
        perm.insert(j, i)
        return self.permute(perm)

    def padOrShrink(self, arg: Sequence[Pair]) -> "ShapeTracker":
        pads, shrinks = [], []
        for (b, e), s in zip(arg, self.shape):
            if b < -s or e < -s or b + e < -s:
                raise ValueError(f"Invalid padOrShrink {list(arg)} for {self.shape}")
            pads.append((max(0, b), max(0, e)))
            shrinks.append((max(0, -b), s - max(0, -e)))
        return self.shrink(shrinks).pad(pads)
