"""Einsum front half: expression parsing and contraction-order search, restating src/library/numpy/einsum.ts.

Index letters are numbered in Unicode order; an ellipsis stands for the trailing numbers.  The implicit form keeps the
letters used exactly once, sorted, behind the ellipsis.  The path is a list of operand pairs; every contraction appends
its result as a new operand.  Up to five operands every order is tried and the cheapest by the reference's flop estimate
wins (first found on ties); beyond that operands are folded left to right."""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, Iterator, List, Optional, Sequence, Tuple

_COMPONENT = re.compile(r"\.\.\.|[^\W\d_]")  # an ellipsis or one letter (the reference matches \p{ID_Start})


@dataclass
class EinsumInput:
    shapes: List[List[int]]
    lhsIndices: List[List[int]]
    rhsIndex: List[int]


def parseEinsumExpression(expr: str, shapes: Sequence[Sequence[int]]) -> EinsumInput:
    """einsum.ts:17-102."""
    lhs_text = expr.split("->")[0]
    idents = [c for c in _COMPONENT.findall(lhs_text) if c != "..."]
    if "->" not in expr:
        counts: Dict[str, int] = {}
        for c in idents:
            counts[c] = counts.get(c, 0) + 1
        out = sorted(c for c, n in counts.items() if n == 1)
        if "..." in expr:
            out.insert(0, "...")
        expr += "->" + "".join(out)
    identToIndex = {c: i for i, c in enumerate(sorted(set(idents)))}
    lhs, rhs = expr.split("->")
    lhsComponents = [_COMPONENT.findall(part) for part in lhs.split(",")]
    rhsComponents = _COMPONENT.findall(rhs)
    ellipsisRank = 0
    for i, comps in enumerate(lhsComponents):
        if "..." in comps:
            if comps.count("...") > 1:
                raise ValueError("Multiple ellipses in one einsum operand is not allowed")
            explicit = len(comps) - 1
            if len(shapes[i]) < explicit:
                raise ValueError(f'Einsum operand {i} has shape {list(shapes[i])} but indexed with "{"".join(comps)}"')
            ellipsisRank = max(ellipsisRank, len(shapes[i]) - explicit)

    def to_indices(comps: List[str], rank: Optional[int] = None) -> List[int]:
        out: List[int] = []
        for c in comps:
            if c == "...":
                start = len(comps) - 1 + ellipsisRank - rank if rank is not None else 0
                out.extend(range(len(identToIndex) + start, len(identToIndex) + ellipsisRank))
            else:
                out.append(identToIndex[c])
        return out

    return EinsumInput([list(s) for s in shapes], [to_indices(c, len(shapes[i])) for i, c in enumerate(lhsComponents)], to_indices(rhsComponents))


def computeSizeMap(inp: EinsumInput) -> Dict[int, int]:
    """einsum.ts:188-259: one size per index, a 1 giving way to any other size."""
    if not inp.shapes:
        raise ValueError("Einsum must have at least one input tensor")
    if len(inp.lhsIndices) != len(inp.shapes):
        raise ValueError(f"Mismatched number of lhs operands ({len(inp.lhsIndices)}) and shapes ({len(inp.shapes)})")
    for i, (idx, shape) in enumerate(zip(inp.lhsIndices, inp.shapes)):
        if len(idx) != len(shape):
            raise ValueError(f"Mismatched number of indices ({len(idx)}) and shape ({list(shape)}) for operand {i}")
    if len(set(inp.rhsIndex)) != len(inp.rhsIndex):
        raise ValueError("Repeated index in einsum output")
    sizeMap: Dict[int, int] = {}
    for idx, shape in zip(inp.lhsIndices, inp.shapes):
        for i, dim in zip(idx, shape):
            have = sizeMap.get(i)
            if have is None or have == 1:
                sizeMap[i] = dim
            elif have != dim and dim != 1:
                raise ValueError(f"Inconsistent size for index {i} in einsum: {have} vs {dim}")
    for i in inp.rhsIndex:
        if i not in sizeMap:
            raise ValueError(f"Output index {i} not present in einsum inputs")
    return sizeMap


def _prod(xs) -> int:
    out = 1
    for x in xs:
        out *= x
    return out


def approximatePathFlops(inp: EinsumInput, sizeMap: Dict[int, int], path: Sequence[Tuple[int, int]]) -> int:
    """einsum.ts:124-186: elements of the index group times (terms - 1 + 1 if anything is summed) per step."""
    if not path:
        return _prod(sizeMap[i] for i in dict.fromkeys(inp.lhsIndices[0]))
    usage: Dict[int, int] = {}
    for i in [i for idx in inp.lhsIndices for i in idx] + list(inp.rhsIndex):
        usage[i] = usage.get(i, 0) + 1
    indices = [list(i) for i in inp.lhsIndices]
    total = 0
    for group in path:
        reduced: List[int] = []
        members: List[int] = []
        for t in group:
            for i in indices[t]:
                if i not in members:
                    members.append(i)
                usage[i] -= 1
                if usage[i] == 0:
                    reduced.append(i)
        total += _prod(sizeMap[i] for i in members) * (len(group) - 1 + (1 if reduced else 0))
        new = [i for i in members if i not in reduced]
        for i in new:
            usage[i] += 1
        indices.append(new)
    return total


@dataclass
class EinsumPath:
    input: EinsumInput
    sizeMap: Dict[int, int]
    path: List[Tuple[int, int]]

    @property
    def outputShape(self) -> List[int]:
        return [self.sizeMap[i] for i in self.input.rhsIndex]

    @property
    def approximateFlops(self) -> int:
        return approximatePathFlops(self.input, self.sizeMap, self.path)


def _all_paths(tensors: List[int], nxt: int) -> Iterator[List[Tuple[int, int]]]:
    if len(tensors) == 2:
        yield [(tensors[0], tensors[1])]
        return
    for i in range(len(tensors)):
        for j in range(i + 1, len(tensors)):
            pair = (tensors[i], tensors[j])
            rest = [t for t in tensors if t not in pair] + [nxt]
            for sub in _all_paths(rest, nxt + 1):
                yield [pair] + sub


def computeEinsumPath(inp: EinsumInput, method: Optional[str] = None) -> EinsumPath:
    """einsum.ts:263-330."""
    if method is None:
        method = "optimal" if len(inp.shapes) <= 5 else "naive"
    sizeMap = computeSizeMap(inp)
    n = len(inp.shapes)
    if n == 1:
        return EinsumPath(inp, sizeMap, [])
    if method == "naive":
        path, last = [], 0
        for i in range(1, n):
            path.append((last, i))
            last = n + i - 1
        return EinsumPath(inp, sizeMap, path)
    if method != "optimal":
        raise ValueError(f"Unknown computePath method: {method}")
    best, bestFlops = None, None
    for path in _all_paths(list(range(n)), n):
        flops = approximatePathFlops(inp, sizeMap, path)
        if bestFlops is None or flops < bestFlops:
            best, bestFlops = path, flops
    return EinsumPath(inp, sizeMap, best)
