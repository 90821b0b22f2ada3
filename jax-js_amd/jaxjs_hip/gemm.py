"""Source generation for kernel class (d): MFMA GEMM (templates `gemm_f16.hip.inc`, `gemm_f32.hip.inc`).

The tuner's `match_gemm` has already reduced the Kernel to strides of a batched `C = A . B^T`-style
contraction; this module chooses the block tile, renders the fused epilogue as a device function
and fills the template.
"""

from __future__ import annotations

import math

from typing import Dict, List

from .alu import AluExp, AluOp, DType, Kernel, byteWidth
from .codegen import CTYPE, STORAGE_CTYPE, HipExpCodegen, strip_parens
from .kernelgen import KernelSource, LaunchStep, _Body, _min_bytes, _prelude, _used_args, epilogue_compile_options, fill, template
from . import tuner
from .tuner import TuneResult, classify_loads


def choose_tile(g: dict) -> Dict[str, int]:
    """Block tile (and wave arrangement) for one GEMM: f16 by a small cost model, f32 128x128 down to 64x64."""
    nb = 1
    for b in g["batch"]:
        nb *= b[0]

    def tiles(bm, bn):
        return -(-g["M"] // bm) * -(-g["N"] // bn) * nb

    CU = tuner.CU_COUNT
    # Slices of the k axis at most: 8, or 64 when the axis is very long (k = batch x positions of a filter cotangent:
    # 100352 against 9 output tiles), where the partial sums stay tiny next to the operands.
    plain_k = not (g.get("a_gather") or g.get("b_gather")) and g["a_k0"] == g["K"] and g["b_k0"] == g["K"]
    max_split = 64 if g["K"] >= (16384 if plain_k else 8192) else 8
    # A k axis that may be cut over workgroups: one stride per plain operand (a slice is a pointer offset), any gather
    # operand (a slice is an offset on the k its loader is asked for).
    # With exactly one gather operand and a short k axis the kernel is a forward convolution, whose stride-1 form has
    # its own template (image patch in LDS) that takes the whole k axis: those keep one slice.
    # A plain operand whose k axis has two strides (runs of k0 elements) can be cut where a slice is whole runs.
    two_level = [g[t + "_k0"] for t in ("a", "b") if g[t + "_k0"] != g["K"]]

    def runs_ok(slices):  # whole runs, or a whole fraction of one
        return all((g["K"] // slices) % k0 == 0 or k0 % (g["K"] // slices) == 0 for k0 in two_level)

    # (float32 has no such template: its forward convolutions are cut like any other gather GEMM.  Nor is that template
    # any use to a float16 convolution with a handful of tiles -- one small image, many channels: [1,512,7,7] * [512,512,3,3]
    # is 8 tiles whatever the template -- which is cut as well and then runs on the gather loaders.)
    one_gather = bool(g.get("a_gather")) != bool(g.get("b_gather"))
    few_tiles = (one_gather and 1024 <= g["K"] < 8192 and g["M"] >= 64 and tiles(64, 128) * 4 <= CU
                 and g["M"] * g["N"] * nb * g["K"] >= (1 << 26))  # (smaller than that, a launch is a launch)
    cut_k = (all(g["K"] % k0 == 0 for k0 in two_level)
             and (not one_gather or g["K"] >= 8192 or g["dtype"] == DType.Float32 or few_tiles))
    repack = _repack_operand(g)  # that operand is read from an aligned copy (rows padded to whole groups)
    loose_ops = bool(g.get("a_loose") or g.get("b_loose")) and repack is None

    def edge_ok(bm, bn):
        return (("a" in (repack or "") or _edge_ok(g["M"], bm, g["a_sk"] == 1))
                and ("b" in (repack or "") or _edge_ok(g["N"], bn, g["b_sk"] == 1)))

    if g["dtype"] == DType.Float32:
        # The f32 matrix pipe is 16x slower than the f16 one, so LDS traffic matters little and filling
        # every CU matters most: take the largest tile that still yields two workgroups per CU (the
        # second one hides the first one's staging latency).  Slabs are 32 deep (measured 3-6 % over 16 on
        # 2048^3 and 4096^3: half the barriers); gather operands keep the 16-deep slabs they were tuned with.
        bk = 32 if plain_k else 16
        # Among the shapes that do, the cheapest by (rounds of two workgroups per CU) x (tile area) / (rate of the
        # shape relative to 128x128: 0.97, 0.80): a last round that is nearly empty costs a whole one (products of
        # attention weights and values over 577 positions, 640 tiles of 128x64: 85.1 us, 66.1 us in 1280 of 64x64; the
        # scores of the same, 3200 tiles of 128x128: 84.9 us, 77.1 us in 6400 of 128x64; 512 x 11008 x 4096, 688 tiles of
        # 128x64: 600 -> 488 us in 1376 of 64x64; 2048 x 2304 x 768: 106 -> 91 us; 2048 x 3072 x 768 pays 4-7 % for it).
        # (16-deep slabs measured faster on some of these short k axes and slower on others: not taken.)
        best = None
        for bm, bn, rate in ((128, 128, 1.0), (128, 64, 0.97), (64, 64, 0.80)):
            if g["M"] >= bm and g["N"] >= bn and tiles(bm, bn) >= 2 * CU:
                cost = -(-tiles(bm, bn) // (2 * CU)) * bm * bn / rate
                if best is None or cost < best[0]:
                    best = (cost, dict(BM=bm, BN=bn, BK=bk))
        if best is not None:
            return best[1]
        # A handful of tiles (512^3 and smaller): the launch is as long as one workgroup's walk along k.  64x64 tiles and
        # up to 8 slices of at least 64 k, until every CU has a workgroup, folded inside the launch
        # (128^3 8.2 -> 5.4 us, 256^3 15.2 -> 6.3 us, 512^3 17.2 -> 9.1 us; the launch floor is 4.7 us).
        if plain_k and g["M"] >= 64 and g["N"] >= 64 and tiles(128, 64) * 4 <= CU:
            split = 1
            while tiles(64, 64) * split < CU and split < 8 and g["K"] % (split * 2 * bk) == 0 and g["K"] // (split * 2) >= 64:
                split *= 2
            return dict(BM=64, BN=64, BK=bk, **(dict(SPLITK=split, FUSEK=1) if split > 1 else {}))
        # Fewer tiles than that: 128x64 tiles with the k axis cut over blockIdx.y until the launch has at least 1.5
        # workgroups per CU (1024^3: 128 tiles x 4 slices, 37.9 -> 31.1 us; 128x14336x4096: 224 x 2, 222 -> 172 us).
        if plain_k and g["M"] >= 128 and g["N"] >= 64:
            split = 1
            while tiles(128, 64) * split < 1.5 * CU and split < 8 and g["K"] % (split * 2 * bk) == 0 and g["K"] // (split * 2) >= 256:
                split *= 2
            # The slices are folded inside the launch (1024^3: 30.2 -> 27.8 us, 128x14336x4096: 169 -> 166, same bits);
            # four waves stacked along m then measure another 1 % better than 2x2.
            return dict(BM=128, BN=64, BK=bk, SPLITK=split, **(dict(FUSEK=1, WM=4, WN=1) if split > 1 else {}))
        # Fewer than 128 rows or 64 columns: 64x64 tiles, the k axis cut the same way when they are few.  Gather operands
        # keep gaining up to four workgroups per CU (filter cotangents: [32,128,28,28] 143 us in 16 slices = 576
        # workgroups, 115 us in 32; [8,64,56,56] 54 -> 49 us; [16,128,28,28] 78 -> 67 us; [32,256,14,14] 183 -> 162 us).
        fill = 4.0 if not plain_k and g["K"] >= 8192 else 1.5
        split = 1
        while cut_k and tiles(64, 64) * split < fill * CU and split < max_split and g["K"] % (split * 2 * bk) == 0 and g["K"] // (split * 2) >= 256 and runs_ok(split * 2):
            split *= 2
        return dict(BM=64, BN=64, BK=bk, **(dict(SPLITK=split, FUSEK=1 if plain_k else 0) if split > 1 else {}))
    # f16: estimated time = (tiles the busiest CU runs) x (tile area) x (K + fixed per-tile overhead) / efficiency.
    # Efficiencies are measured rates of each tile shape relative to 256x256 on large problems (MI355X):
    # 128x256 0.84, 256x128 0.79, 128x128 0.62 with two workgroups resident per CU (8000^3: 0.63; 4100 x 4100 x 4096:
    # 218 us against 180 us with 128x256), 0.64 alone with its deeper slabs.  The fixed
    # overhead (pipeline fill + epilogue) is about 100 k-steps.  This picks big tiles for big problems and
    # smaller ones when 256x256 would leave the last round of CUs nearly empty (e.g. 288 tiles on 256 CUs).
    def k_split(count, fill=1.5):
        # Fewer workgroups than `fill` per CU: cut the k axis (partial sums in scratch, fold kernel) while slices stay >= 512 deep.
        split = 1
        gran = 64 if plain_k else 8  # whole slabs for the direct loads; the gather loaders take a ragged last slab
        while cut_k and count * split < fill * CU and split < max_split and g["K"] % (split * 2 * gran) == 0 and g["K"] // (split * 2) >= 512 and runs_ok(split * 2):
            split *= 2
        return dict(SPLITK=split) if split > 1 else {}

    if g["M"] <= 64 and g["N"] >= 128:
        # Few rows.  Many tiles (64 output channels of a convolution against thousands of positions): 64 x 256.
        if g["N"] >= 256 and tiles(64, 256) >= CU:
            return dict(BM=64, BN=256, WM=1, WN=4)
        # Few tiles (a linear layer on 2..64 tokens): bound by streaming B once, so what matters is enough workgroups
        # in flight -- 64 x 128 tiles and a k split (64 x 14336 x 4096: 65.7 us with 56 tiles of 64 x 256, 26.6 us with
        # 112 x 4 slices; 16 rows 24.6 us, 4 rows 23.5 us; B alone takes 15 us at the HBM rate).
        # When the direct-to-LDS template can take the shape (its A loads clamp to the last row that exists) its
        # 128x128 tiles in two or four slices stream B faster than the register-staged loaders, the empty rows of the
        # tile costing nothing that matters here: 4 / 16 / 64 x 14336 x 4096 25.2 / 25.9 / 28.2 -> 20.7 / 21.2 / 23.5 us,
        # 31 x 4096 x 4096 15.5 -> 13.0 us.  Those fall through to the plan below.
        # (Likewise a small B, whatever its k: the launch is all there is to it, and that template's is the shorter one --
        # 32 x 3072 x 768: 12.1 us on the register-staged loaders, 7.2 us for 128 rows on this one.)
        if not (edge_ok(128, 128) and plain_k and not loose_ops and repack is None and g["K"] % 128 == 0
                and (g["K"] >= 2048 or g["N"] * g["K"] <= (1 << 22)) and tiles(128, 128) * 2 <= CU):
            return dict(BM=64, BN=128, WM=1, WN=4, **k_split(tiles(64, 128)))
    elif g["N"] <= 64 and g["M"] >= 128:
        # A 128-wide tile would compute and store a half-empty block (attention's probabilities x V, N = head
        # size 64): measured 30 % faster with 128x64 tiles, which is then bound by reading A.
        return dict(BM=128, BN=64, WM=2, WN=2, **k_split(tiles(128, 64)))
    if (g["K"] <= 128 and g["K"] % 32 == 0 and plain_k and edge_ok(128, 128) and tiles(128, 128) >= 4 * CU
            and not loose_ops and repack is None):
        # A k axis of one to four slabs (attention scores: q.k^T over a head size of 64): the launch is bound by writing
        # C, and a workgroup spends its life in prologue and epilogue.  128x128 tiles with two shallow stages leave
        # room for four workgroups per CU, so that one's stores overlap another's loads and MFMAs
        # (96 x 1024 x 1024 x 64: 47.5 us with 256x256 tiles in the deep pipeline, 41.3 us = 5.5 TB/s this way).
        # Ragged lengths take it through clamped edge loads (scores of 128 heads over 577 positions: 48.9 us on the
        # 128x256 tiles the estimate below picked, 26.1 us here; 384 heads over 197: 17.2 -> 15.1 us).
        return dict(BM=128, BN=128, BK=32, STAGES=2, PIPE=0)
    if (g["K"] <= 1024 and g["K"] % 32 == 0 and plain_k and g["M"] % 128 == 0 and g["N"] % 256 == 0 and tiles(128, 256) >= 2 * CU
            and not loose_ops and repack is None and not (g["a_sk"] == 1 and g["b_sk"] == 1)):
        # A short k axis under many tiles (the projections of a transformer block: 8192 x 2304 x 768, 8192 x 3072 x 768):
        # a workgroup's prologue and its C stores weigh as much as its MFMAs.  128x256 tiles in two shallow stages
        # (48 KiB, 164 registers) put three workgroups on a CU, whose phases overlap: 39.5 -> 36.3 us and 43.4 -> 40.7 us;
        # the same as the deep pipeline at 4096 x 4096 x 1024 and 2048 x 8192 x 512; slower from k = 3072 (65.9 against
        # 41.9 us) and with fewer than two tiles per CU (8192 x 768 x 768: 17.0 against 14.9 us).
        return dict(BM=128, BN=256, WM=1, WN=4, BK=32, STAGES=2, PIPE=0)
    if not plain_k and cut_k and g["K"] >= 8192 and tiles(128, 128) * 8 <= CU:
        # A handful of tiles over a very long k axis read through gather loaders (the filter cotangent of a convolution:
        # 9 taps x 64 x 64 or 128 x 128 outputs, k = batch x positions): 64x64 tiles waste no half-empty MFMA tile and
        # give the k slices four times as many workgroups ([32,64,56,56] 93 -> 72 us, [32,128,28,28] 187 -> 64 us).  With a
        # gather loader on one side only, one workgroup per CU is where more slices stop paying ([32,64,56,56]: 48 us in
        # 32 slices = 288 workgroups, 53 us in 64; [8,64,56,56]: 25 / 30 us); with one on both sides the loads are slower
        # and 1.5 per CU still gain ([32,128,28,28]: 61 us in 8 slices = 288 workgroups, 51 in 16, 53 in 32).
        both = bool(g.get("a_gather")) and bool(g.get("b_gather"))
        return dict(BM=64, BN=64, **k_split(tiles(64, 64), 1.5 if both else 1.0))
    if few_tiles and cut_k:
        # [1,512,7,7] * [512,512,3,3] f16: 47.9 us as 8 tiles of the patch template; [1,256,28,28] stride 2: 37.9 us.
        return dict(BM=64, BN=64, **k_split(tiles(64, 64)))
    if (bool(g.get("a_gather")) != bool(g.get("b_gather")) and g["K"] < 8192 and g["M"] >= 128 and g["N"] >= 128
            and g["a_k0"] == g["K"] and g["b_k0"] == g["K"] and tiles(128, 128) < CU):
        # One gather operand, fewer 128x128 tiles than CUs (the convolutions of audio models: a few hundred channels
        # against one long row of a few thousand positions): smaller tiles until the launch covers the chip.
        # [1,512,1500] * [512,512,3]: 48 tiles, 40.5 us; 192 of 64x64, 33.5 us.  [1,384,3000] stride 2: 36 tiles, 46.5 us;
        # 144 of 64x64, 24.3 us.  [1,256,8000] * [256,256,7]: 126 tiles, 50.5 us; 250 of 128x64, 42.3 us (64x64: 49.6).
        return dict(BM=64, BN=64) if tiles(128, 128) * 4 <= 1.5 * CU else dict(BM=128, BN=64)
    best = None
    for bm, bn, eff, extra in ((256, 256, 1.00, dict()), (128, 256, 0.84, dict(WM=1, WN=4)), (256, 128, 0.79, dict()),
                                (128, 128, 0.62, dict())):
        if (bm > 128 and g["M"] < bm) or (bn > 128 and g["N"] < bn):
            continue
        per_cu = -(-tiles(bm, bn) // tuner.CU_COUNT)
        if (bm, bn) == (128, 128) and per_cu < 2:
            eff = 0.64
        whole = edge_ok(bm, bn) and (g["K"] % 32 == 0 or repack is not None) and plain_k and not loose_ops
        if not whole:
            # A ragged k axis, operands off the 16-byte grid or an edge the direct loads cannot clamp run the general
            # template, whose small tiles lose more
            # (8000^3: 838 / 597 / 691 / 512 TFLOP/s for the four shapes, against 1340 for whole 256x256 tiles).
            eff = {(256, 256): 0.63, (128, 256): 0.45, (256, 128): 0.52, (128, 128): 0.38}[(bm, bn)]
        cost = per_cu * bm * bn * (g["K"] + 100) / eff
        if best is None or cost < best[0]:
            best = (cost, dict(BM=bm, BN=bn, **extra), per_cu)
    tile, per_cu = dict(best[1]), best[2]
    both_k = g["a_sk"] == 1 and g["b_sk"] == 1
    if (tile["BM"], tile["BN"]) == (128, 128) and per_cu == 1 and plain_k and g["K"] % 64 == 0:
        # One 128x128 workgroup per CU (or fewer): nothing shares the CU's LDS, so the slabs can be 64 deep in four
        # stages (128 KiB: twice the bytes in flight per workgroup; 2048^3 20.7 -> 19.6 us, 128x14336x4096 35.2 -> 27.4 us).
        if not both_k:
            tile.update(BK=64, STAGES=4)
        # Half the CUs or fewer would get a workgroup: cut the k axis in two, four when a quarter or fewer would, the
        # slices folded inside the launch by the last one to arrive (128x14336x4096: 27.4 -> 26.0 us with a fold
        # launch, 24.7 folded in the launch; 128x4096x4096: 16.1 us in two slices, 13.9 in four; with 112 tiles four
        # slices cost more in partial sums than they gain).
        if tiles(128, 128) * 2 <= CU and g["K"] >= 2048 and g["K"] % 128 == 0:
            tile.update(SPLITK=4 if tiles(128, 128) * 4 <= CU and g["K"] >= 4096 and g["K"] % 256 == 0 else 2)
            # The slices take 32-deep slabs in four stages (64 KiB, so two workgroups fit a CU): as fast as the 64-deep
            # ones at their best and steady, where those swing between 21 and 28 us from launch to launch
            # (16 x 14336 x 4096: 20.2-20.7 us against 24-27; 128 rows: 26.0-26.6 against 29.6-32.9).
            tile.update(BK=32, STAGES=4)
            # Folding inside the launch is the direct-to-LDS template's: operands on the 16-byte grid, edges it can clamp.
            # Other shapes keep the split and fold in a second launch.
            # Two slices only: with four, the last workgroup's read-back of four slices behind the acknowledged stores
            # costs more than a fold launch (128x4096x4096: 16.0 us folded in the launch, 14.4 us with the fold kernel).
            # Edge tiles fold the same way (100 x 14336 x 4096: 31.1 us in four slices with a fold launch, 25.5 us in two).
            # Up to 64 rows the fold launch is the cheaper one: it touches the rows that exist, the fold inside the launch
            # whole tiles of partial sums (64 x 14336 x 4096: 23.5 against 23.7 us, 4 rows: 20.7 against 22.4 us).
            if edge_ok(128, 128) and not (g.get("a_loose") or g.get("b_loose")):  # (a repacked operand takes no k split)
                if tile["SPLITK"] == 2 and g["M"] > 64:
                    tile.update(FUSEK=1)
            else:  # the general template gains from more slices (100 x 14336 x 4096: 41.1 us in two, 34.6 us in four)
                tile.update(k_split(tiles(128, 128)) or dict(SPLITK=tile["SPLITK"]))
    elif not plain_k and cut_k and per_cu == 1 and tiles(tile["BM"], tile["BN"]) * 2 <= CU:
        # Gather operands on both sides and a handful of tiles over a long k axis (the filter cotangent of a
        # convolution: 9 taps x one tile, k = batch x positions): slices over workgroups, folded by a second launch.
        tile.update(k_split(tiles(tile["BM"], tile["BN"])))
    return tile


def _repack_operand(g: dict):
    """The operands ("a", "b" or "ab") that a pre-pass copies into scratch before the direct-to-LDS template reads them,
    or None.  That template loads whole 16-byte groups from the 16-byte grid and walks k in whole 32-deep slabs; an
    f16 operand off the grid (np.matmul against a [K, N] matrix with N = 50257: every row starts at an odd element) or a
    k axis that is not whole slabs (k = 50257, 4100, 1000) would otherwise send the whole GEMM to the general template
    (8192 x 50257 x 768: 1.19 ms against 0.80 ms).  The copy keeps the operand's orientation -- [rows][k] or [k][rows] --
    with rows rounded up to 8 and k to 32, zeros in the padding (2 x 2 bytes of traffic per element); a ragged k axis
    takes both operands.  Worth it when the other operand has enough rows to amortise the copy."""
    if g["dtype"] != DType.Float16 or g["batch"] or g.get("a_gather") or g.get("b_gather"):
        return None
    if g["a_k0"] != g["K"] or g["b_k0"] != g["K"] or g["K"] < 64:
        return None
    ragged_k = g["K"] % 32 != 0
    tags = "".join(t for t in ("a", "b") if g.get(t + "_loose") or ragged_k)
    if not tags:
        return None
    for t in tags:
        rows, other = (g["M"], g["N"]) if t == "a" else (g["N"], g["M"])
        srow, sk = (g["a_sm"], g["a_sk"]) if t == "a" else (g["b_sn"], g["b_sk"])
        if (srow != 1 and sk != 1) or rows < 128 or other < 512:
            return None
    if sum((g["M"] if t == "a" else g["N"]) for t in tags) * (g["K"] + 32) * 2 > (1 << 30):
        return None  # more than 1 GiB of copies: not at the price of that much scratch
    return tags


def _edge_ok(extent: int, tile: int, k_contiguous: bool) -> bool:
    """Whether the direct-to-LDS template can take an operand whose row count is `extent` in tiles of `tile` rows: whole
    tiles, or an edge tile whose loads can be clamped -- to the last row when the operand runs along k in memory, to
    the last whole 16-byte group of rows when it runs along its rows (the count must then be whole groups)."""
    return extent % tile == 0 or k_contiguous or (extent % 8 == 0 and extent >= 8)


def _strip_casts(e: AluExp) -> AluExp:
    """Drop float<->float casts around an operand (the MFMA consumes the storage type)."""
    while e.op == AluOp.Cast and e.dtype in (DType.Float16, DType.Float32, DType.Float64) and \
            e.src[0].dtype in (DType.Float16, DType.Float32):
        e = e.src[0]
    return e



# ---- row-vector gather: eight consecutive rows of a gather operand in one 128-bit load ------------------------------
#
# For an operand whose memory runs along its tile-row axis (the pixels of a stride-1 convolution's image operand),
# element (row0 + e, k) for an aligned row0 (row0 % 8 == 0) and e in 0..7 sits at index(row0, k) + e, and its mask is
# a conjunction of comparisons that are linear in e.  `_lin` proves that shape on the operand's own simplified
# expression: it splits an expression f(row) evaluated at row0 + e into rest(row0) + coef * e, pushing e out of
# `% D` and `/ D` when the rest is a multiple of 8 * coef that divides D.

def _has_row(e: AluExp) -> bool:
    return bool(e.collect(lambda x: x.op == AluOp.Special and x.arg[0] == "row"))


def _multiple_of(e: AluExp, m: int, group: int) -> bool:
    if m == 1:
        return True
    if e.op == AluOp.Const:
        return int(e.arg) % m == 0
    if e.op == AluOp.Special and e.arg[0] == "row":
        return group % m == 0
    if e.op in (AluOp.Add, AluOp.Sub):
        return _multiple_of(e.src[0], m, group) and _multiple_of(e.src[1], m, group)
    if e.op == AluOp.Mul:
        for x, y in ((e.src[0], e.src[1]), (e.src[1], e.src[0])):
            if y.op == AluOp.Const:
                c = abs(int(y.arg))
                if c % m == 0:
                    return True
                return c != 0 and _multiple_of(x, m // math.gcd(m, c), group)
        return False
    if e.op == AluOp.Mod and e.src[1].op == AluOp.Const and int(e.src[1].arg) % m == 0:
        return _multiple_of(e.src[0], m, group)
    return False


def _lin(e: AluExp, group: int = 8):
    """(coef, rest) with e(row0 + t) == rest(row0) + coef * t for every aligned row0 and t in [0, group), or None."""
    if not _has_row(e):
        return 0, e
    if e.dtype != DType.Int32:
        return None
    if e.op == AluOp.Special:
        return 1, e
    if e.op in (AluOp.Add, AluOp.Sub):
        a, b = _lin(e.src[0], group), _lin(e.src[1], group)
        if a is None or b is None:
            return None
        if e.op == AluOp.Add:
            return a[0] + b[0], AluExp.add(a[1], b[1])
        return a[0] - b[0], AluExp.sub(a[1], b[1])
    if e.op == AluOp.Mul:
        for x, y in ((e.src[0], e.src[1]), (e.src[1], e.src[0])):
            if y.op == AluOp.Const:
                a = _lin(x, group)
                if a is None:
                    return None
                return a[0] * int(y.arg), AluExp.mul(a[1], y)
        return None
    if e.op in (AluOp.Mod, AluOp.Idiv) and e.src[1].op == AluOp.Const:
        D = int(e.src[1].arg)
        a = _lin(e.src[0], group)
        if a is None or D <= 0:
            return None
        coef, rest = a
        if coef == 0:
            return 0, AluExp(e.op, e.dtype, (rest, e.src[1]))
        step = coef * group
        if coef < 0 or rest.min < 0 or D % step != 0 or not _multiple_of(rest, step, group):
            return None
        return (coef, AluExp.mod(rest, e.src[1])) if e.op == AluOp.Mod else (0, AluExp.idiv(rest, e.src[1]))
    return None


def rows8_form(oexp: AluExp, extent: int, group: int = 8):
    """For a gather operand's expression in (row, k, batch coordinates): (index at the group's first row, mask as a
    function of the extra variable `e` or None when unmasked, the GlobalIndex node) if `group` consecutive rows of
    every aligned group load `group` consecutive elements; else None."""
    cond = None
    node = oexp
    if node.op == AluOp.Where:
        zero = node.src[2]
        if zero.op != AluOp.Const or float(zero.arg) != 0.0:
            return None
        cond, node = node.src[0], node.src[1]
    if node.op != AluOp.GlobalIndex:
        return None
    a = _lin(node.src[0], group)
    if a is None or (group > 1 and a[0] != 1):
        return None
    idx0 = a[1].simplify()
    evar = AluExp.special(DType.Int32, "e", group)
    cond_e = None
    if cond is not None:
        atoms = []
        for atom in cond.splitOp(AluOp.Mul):
            neg = False
            inner = atom
            if inner.op == AluOp.Cmpne and inner.src[1].op == AluOp.Const and inner.src[0].dtype == DType.Bool and bool(inner.src[1].arg) is True:
                neg, inner = True, inner.src[0]
            if inner.op != AluOp.Cmplt:
                if _has_row(inner):
                    return None
                atoms.append(atom)
                continue
            sides = []
            for side in inner.src:
                la = _lin(side, group)
                if la is None:
                    return None
                coef, rest = la
                sides.append(AluExp.add(rest, AluExp.mul(evar, AluExp.i32(coef))) if coef else rest)
            lt = AluExp.cmplt(sides[0], sides[1])
            atoms.append(AluExp.cmpne(lt, AluExp.bool(True)) if neg else lt)
        cond_e = atoms[0]
        for x in atoms[1:]:
            cond_e = AluExp.mul(cond_e, x)
        cond_e = cond_e.simplify()
    return idx0, cond_e, node



def _swap_row_k(e: AluExp) -> AluExp:
    """The same expression with the roles of the Specials `row` and `k` exchanged."""
    def sw(n):
        if n.op == AluOp.Special and n.arg[0] == "row":
            return AluExp.special(n.dtype, "k", n.arg[1])
        if n.op == AluOp.Special and n.arg[0] == "k":
            return AluExp.special(n.dtype, "row", n.arg[1])
        return None
    return e.rewrite(sw)


def kvec_form(oexp: AluExp, K: int, group: int = 8):
    """`rows8_form` along the other axis: (index at the group's first k, mask as a function of `e`, the GlobalIndex node) if
    `group` consecutive k of every aligned group read `group` consecutive elements of one row (the image operand of a
    filter cotangent: k runs over batch x positions, and consecutive positions are consecutive pixels); else None."""
    form = rows8_form(_swap_row_k(oexp), K, group)
    if form is None:
        return None
    idx0, cond_e, node = form
    return _swap_row_k(idx0).simplify(), (None if cond_e is None else _swap_row_k(cond_e).simplify()), node


# ---- tap-major k order for convolution-like gather operands -----------------------------------------------------------
#
# The patch operand of a convolution reads element k = c * T + tap (T filter taps, tap fastest) of channel plane c:
# its index is `plane(c) + window(row, tap)` and its padding mask does not depend on c at all.  Walking k in the order
# k' = tap * C + c instead (a permutation of the reduction, applied to both operands alike) makes a slab of consecutive
# k' one tap over consecutive channels: the index/mask arithmetic is done once per (rows, tap) and each further channel
# costs one add and one load.

def _has_special(e: AluExp, name: str) -> bool:
    return bool(e.collect(lambda x: x.op == AluOp.Special and x.arg[0] == name))


def _affine_in(e: AluExp, name: str):
    """(coef, rest) with e == rest + coef * name, `name` reached only through +, - and * const; else None."""
    if not _has_special(e, name):
        return 0, e
    if e.op == AluOp.Special:
        return 1, AluExp.i32(0)
    if e.dtype != DType.Int32:
        return None
    if e.op in (AluOp.Add, AluOp.Sub):
        a, b = _affine_in(e.src[0], name), _affine_in(e.src[1], name)
        if a is None or b is None:
            return None
        return (a[0] + b[0], AluExp.add(a[1], b[1])) if e.op == AluOp.Add else (a[0] - b[0], AluExp.sub(a[1], b[1]))
    if e.op == AluOp.Mul:
        for x, y in ((e.src[0], e.src[1]), (e.src[1], e.src[0])):
            if y.op == AluOp.Const:
                a = _affine_in(x, name)
                return None if a is None else (a[0] * int(y.arg), AluExp.mul(a[1], y))
    return None


def _conj_terms(c: AluExp):
    """The terms of a conjunction (booleans multiply)."""
    if c.op == AluOp.Mul and c.dtype == DType.Bool:
        return _conj_terms(c.src[0]) + _conj_terms(c.src[1])
    return [c]


def interval_mask_form(cond: AluExp, name: str = "e"):
    """`cond` as (terms without `name`, lower bounds, upper bounds): cond == all(terms) and lo <= name < hi for every
    lower bound lo and upper bound hi (integer expressions without `name`); None when some term is not a comparison
    that is affine in `name` with coefficient +-1.  The padding masks of window views have this form: along a run of
    consecutive elements the elements inside the image are one interval."""
    inv, lows, highs = [], [], []
    for t in _conj_terms(cond):
        if not _has_special(t, name):
            inv.append(t)
            continue
        negated = False
        while t.op == AluOp.Cmpne and t.src[0].dtype == DType.Bool and any(x.op == AluOp.Const for x in t.src):
            c, x = (t.src[0], t.src[1]) if t.src[0].op == AluOp.Const else (t.src[1], t.src[0])
            if bool(c.arg):
                negated = not negated
            t = x
        if t.op != AluOp.Cmplt or t.src[0].dtype != DType.Int32:
            return None
        fa, fb = _affine_in(t.src[0], name), _affine_in(t.src[1], name)
        if fa is None or fb is None:
            return None
        coef, rest = fa[0] - fb[0], AluExp.sub(fa[1], fb[1])  # the term reads coef * name + rest < 0
        if coef == 1:  # name < -rest; negated: name >= -rest
            (lows if negated else highs).append(AluExp.sub(AluExp.i32(0), rest).simplify())
        elif coef == -1:  # name > rest, i.e. name >= rest + 1; negated: name <= rest, i.e. name < rest + 1
            (highs if negated else lows).append(AluExp.add(rest, AluExp.i32(1)).simplify())
        else:
            return None
    return inv, lows, highs


def mask_bits_fn(cond_e, tag: str, G: int, names, numerics: str) -> str:
    """C function `jh_mbits_<tag>(row, k, b0, b1, b2)`: bit e set when element e of the group of `G` that starts at
    (row, k) is inside the operand's mask.  From the interval form where the mask has one (two bounds and a few compares
    per group instead of a compare chain per element: the loaders of gather GEMMs are bound by such arithmetic), element
    by element otherwise."""
    head = f"static __device__ __forceinline__ unsigned jh_mbits_{tag}(int row, int k, int b0, int b1, int b2) {{\n"
    if cond_e is None:
        return head + f"  return {(1 << G) - 1}u;\n}}"
    vnames = {"row": "row", "e": "e", "k": "k", "b0": "b0", "b1": "b1", "b2": "b2"}
    form = interval_mask_form(cond_e)
    cg = HipExpCodegen(names, vnames, "  ", prefix=f"mb{tag}", numerics=numerics)
    if form is None:
        cg.indent = "    "
        cg.countReferences(cond_e)
        val = strip_parens(cg.run(cond_e))
        return (head + f"  unsigned bits = 0u;\n#pragma unroll\n  for (int e = 0; e < {G}; ++e) {{\n" + "\n".join(cg.take_lines())
                + f"\n    bits |= (({val}) ? 1u : 0u) << e;\n  }}\n  return bits;\n}}")
    inv, lows, highs = form
    for x in inv + lows + highs:
        cg.countReferences(x)
    inv_c = [strip_parens(cg.run(x)) for x in inv]
    lo_c = [strip_parens(cg.run(x)) for x in lows]
    hi_c = [strip_parens(cg.run(x)) for x in highs]
    body = "\n".join(cg.take_lines())
    lo_s = "".join(f"  lo = lo > ({x}) ? lo : ({x});\n" for x in lo_c)
    hi_s = "".join(f"  hi = hi < ({x}) ? hi : ({x});\n" for x in hi_c)
    ok = " && ".join(["lo < hi"] + [f"({x})" for x in inv_c])
    return (head + (body + "\n" if body else "") + f"  int lo = 0, hi = {G};\n{lo_s}{hi_s}"
            f"  return ({ok}) ? (((1u << hi) - 1u) & ~((1u << lo) - 1u)) : 0u;\n}}")


def tap_major_form(oexp: AluExp, K: int):
    """For a gather operand's expression in (row, k, batch coordinates): try k = c * T + tap for every T that the
    expression divides k by.  Returns dict(T, C, cs, exp) where `exp` is the operand re-expressed in (row, tap, batch
    coordinates) at c = 0, the element of channel c sitting `c * cs` further on and the mask not involving c; or None."""
    kvars = oexp.collect(lambda x: x.op == AluOp.Idiv and x.src[0].op == AluOp.Special and x.src[0].arg[0] == "k" and x.src[1].op == AluOp.Const)
    cands = sorted({int(x.src[1].arg) for x in kvars}, reverse=True)
    for T in cands:
        if T <= 1 or K % T != 0 or (K // T) % 8 != 0:
            continue
        C = K // T
        cvar, tvar = AluExp.special(DType.Int32, "c", C), AluExp.special(DType.Int32, "tap", T)
        kexp = AluExp.add(AluExp.mul(cvar, AluExp.i32(T)), tvar)
        e = oexp.rewrite(lambda n: kexp if (n.op == AluOp.Special and n.arg[0] == "k") else None).simplify()
        node, cond = e, None
        if node.op == AluOp.Where:
            if node.src[2].op != AluOp.Const or float(node.src[2].arg) != 0.0:
                continue
            cond, node = node.src[0], node.src[1]
        if node.op != AluOp.GlobalIndex or (cond is not None and _has_special(cond, "c")):
            continue
        a = _affine_in(node.src[0], "c")
        if a is None or a[0] <= 0:
            continue
        base = AluExp.globalIndex(node.dtype, node.arg[0], node.arg[1], a[1].simplify())
        exp0 = base if cond is None else AluExp.where(cond, base, e.src[2])
        return dict(T=T, C=C, cs=a[0], exp=exp0)
    return None


def gen_gemm(kernel: Kernel, t: TuneResult, numerics: str, name: str) -> KernelSource:
    g = t.gemm
    re = kernel.reduction
    assert g is not None and re is not None and t.epilogue is not None
    override = dict(t.params.get("gemm_tile") or {})
    tile = dict() if ("BM" in override or "BN" in override) else choose_tile(g)
    tile.update(override)
    if "BM" not in tile or "BN" not in tile:
        raise ValueError("a tile override must give both BM and BN")
    BM, BN = tile["BM"], tile["BN"]
    WM, WN = tile.get("WM", 2), tile.get("WN", 2)
    if BM % (32 * WM) or BN % (32 * WN):
        raise ValueError(f"tile {BM}x{BN} does not divide into {WM}x{WN} waves of 32x32 MFMA tiles")
    nthreads = 64 * WM * WN
    out_t = STORAGE_CTYPE[kernel.dtype]
    in_t = STORAGE_CTYPE[g["dtype"]]

    # Split of the k axis over blockIdx.y: every slice is the same kernel on K / split, its f32 accumulators go to a
    # scratch buffer [slice][output] and a generated fold Kernel adds the slices in order and applies the epilogue
    # (deterministic: no float atomics).  For launches that would otherwise leave most CUs without a workgroup.
    split = int(tile.get("SPLITK", 1))
    K_full = g["K"]
    two_stride = dict(a=g["a_k0"] != K_full, b=g["b_k0"] != K_full)  # of the whole k axis, before any slicing
    if split > 1:
        vec_k = 8 if g["dtype"] == DType.Float16 else 4
        # a two-stride k axis is cut into whole runs, or a run into whole slices
        if (K_full % split or (K_full // split) % vec_k
                or any(g[t + "_k0"] != K_full and (K_full // split) % g[t + "_k0"] and g[t + "_k0"] % (K_full // split) for t in ("a", "b"))):
            split = 1
    # ... or, with FUSEK (f32 template), folded inside the same launch by the slice that arrives last at the tile's
    # counter: one launch instead of two.
    fusek = 0
    if split > 1:
        KS = K_full // split
        run_full = dict(a=g["a_k0"], b=g["b_k0"])
        # (a slice inside one run has a single stride, like a slice of a single-stride axis)
        g = dict(g, K=KS, a_k0=KS if g["a_k0"] == K_full or g["a_k0"] > KS else g["a_k0"],
                 b_k0=KS if g["b_k0"] == K_full or g["b_k0"] > KS else g["b_k0"])
        fusek = split if tile.get("FUSEK", 0) else 0
        if not fusek:
            out_t = "float"

    # An operand off the 16-byte grid that a pre-pass copies into scratch (see `_repack_operand`): from here on it is a
    # dense [K][rows_pad] operand named `jh_repack`.
    repack = _repack_operand(g) if split == 1 and tile.get("REPACK", 1) else None
    load_rows = dict(a=g["M"], b=g["N"])
    repack_src = {}
    if repack:
        k_pad = -(-g["K"] // 32) * 32
        for tg in repack:
            rows = load_rows[tg]
            srow = g["a_sm"] if tg == "a" else g["b_sn"]
            rkey = "a_sm" if tg == "a" else "b_sn"
            kc = g[tg + "_sk"] == 1  # runs along k: copied as [rows][k_pad]; else along its rows: [k_pad][rows_pad]
            rows_pad = rows if kc else -(-rows // 8) * 8
            repack_src[tg] = dict(gid=g["gid_" + tg], off=g[tg + "_off"], sk=g[tg + "_sk"], srow=srow, rows=rows, rows_pad=rows_pad,
                                  k=g["K"], k_pad=k_pad, kc=kc)
            load_rows[tg] = rows_pad
            g = dict(g, **{tg + "_off": 0, tg + "_sk": 1 if kc else rows_pad, rkey: k_pad if kc else 1, tg + "_loose": False})
        g = dict(g, K=k_pad, a_k0=k_pad, b_k0=k_pad)

    used = _used_args(kernel.nargs, t.epilogue)
    used[g["gid_a"]] = g["dtype"]
    used[g["gid_b"]] = g["dtype"]
    names = [f"in{i}" for i in range(kernel.nargs)]
    params = ", ".join(
        [f"const {STORAGE_CTYPE[d or DType.Float32]}* __restrict__ {n}" for d, n in zip(used, names)]
        + [f"{out_t}* __restrict__ out"] + (["float* __restrict__ jh_part", "unsigned* __restrict__ jh_count"] if fusek else [])
        + [f"const jh_f16* __restrict__ jh_repack_{tg}" for tg in (repack or "")])

    # Fused epilogue as a device function of (acc, row, col, batch coordinates, buffers...).  The kernel's
    # epilogue is written over the flat output index; here that index is re-expressed through the tile's own
    # coordinates and simplified, so `gidx % N` becomes `col` and a bias load no longer depends on the row
    # (the compiler then hoists it out of the per-row loop instead of doing a division per element).
    if len(g["batch"]) > 3:
        raise ValueError("at most 3 batch axes")
    I32 = DType.Int32
    gexp = AluExp.add(AluExp.mul(AluExp.special(I32, "row", max(g["M"], 1)), AluExp.i32(g["c_sm"])),
                      AluExp.mul(AluExp.special(I32, "col", max(g["N"], 1)), AluExp.i32(g["c_sn"])))
    for k, (size, _sa, _sb, sc) in enumerate(g["batch"]):
        gexp = AluExp.add(AluExp.mul(AluExp.special(I32, f"b{k}", size), AluExp.i32(sc)), gexp)

    def _retarget(node):
        if node.op == AluOp.Special and node.arg[0] == "gidx":
            return gexp
        return None
    epilogue = t.epilogue.rewrite(_retarget).simplify()
    cg = HipExpCodegen(names, {"acc": "acc", "row": "row", "col": "col", "b0": "b0", "b1": "b1", "b2": "b2"}, "  ",
                       prefix="e", numerics=numerics)
    cg.countReferences(epilogue)
    value = strip_parens(cg.run(epilogue))
    epi_params = "".join(f", const {STORAGE_CTYPE[d or DType.Float32]}* __restrict__ {n}" for d, n in zip(used, names))
    epi_fn = (f"static __device__ __forceinline__ {out_t} jh_epilogue(float acc, int row, int col, int b0, int b1, int b2{epi_params}) {{\n"
              + "\n".join(cg.take_lines()) + f"\n  return ({out_t})({value});\n}}")
    src_options = epilogue_compile_options(epilogue)
    if split > 1 and not fusek:  # the fold kernel applies the epilogue; a slice stores its raw accumulator
        src_options = ""
        epi_fn = f"static __device__ __forceinline__ float jh_epilogue(float acc, int row, int col, int b0, int b1, int b2{epi_params}) {{\n  return acc;\n}}"
    epi_args = "".join(f", {n}" for n in names)

    # Element loaders for gather operands: the operand's lowered expression (masked load through its view
    # chain) with the flat output index rebuilt from (tile row, batch coordinates) and ridx = k.
    gather_fns, gather_calls, gather_flags, gather_group, gather_oexp, gather_slow, element_fn = [], {}, {}, {}, {}, {}, {}
    lowered = _strip_casts(t.exp)
    operand_exps = {g["gid_a"]: None, g["gid_b"]: None}
    if g.get("a_gather") or g.get("b_gather"):
        assert lowered.op == AluOp.Mul
        for side in lowered.src:
            gids = {n.arg[0] for n in side.collect(lambda x: x.op == AluOp.GlobalIndex)}
            if len(gids) != 1:
                raise ValueError("gather operand must read exactly one buffer")
            operand_exps[gids.pop()] = _strip_casts(side)
    for tag, gid, is_gather, extent, c_stride in (("a", g["gid_a"], g.get("a_gather"), g["M"], g["c_sm"]),
                                                  ("b", g["gid_b"], g.get("b_gather"), g["N"], g["c_sn"])):
        gather_flags[tag] = 1 if is_gather else 0
        if not is_gather:
            gather_calls[tag] = f"({in_t})0"
            continue
        flat = AluExp.mul(AluExp.special(I32, "row", max(extent, 1)), AluExp.i32(c_stride))
        for k, (size, _sa, _sb, sc) in enumerate(g["batch"]):
            flat = AluExp.add(AluExp.mul(AluExp.special(I32, f"b{k}", size), AluExp.i32(sc)), flat)
        kvar = AluExp.special(I32, "k", max(K_full, 1))  # the whole axis: a slice's loader is asked for k + its offset

        def _retarget_operand(node, flat=flat, kvar=kvar):
            if node.op == AluOp.Special and node.arg[0] == "gidx":
                return flat
            if node.op == AluOp.Special and node.arg[0] == "ridx":
                return kvar
            return None
        oexp = operand_exps[gid].rewrite(_retarget_operand).reduceExactIndex().simplify()
        gather_oexp[tag] = oexp
        if tag == "b" and g["dtype"] == DType.Float16 and split == 1 and tile.get("CONV", 1) and not tile.get("TAPMAJOR", 0):
            # A stride-1 window walk over an image (verified on the operand's own index expression): the patch-in-LDS
            # convolution template instead of an im2col tile built element by element.  The other operand -- the filter --
            # may itself be a gather operand (the flipped, transposed filter of the cotangent towards the activations): the
            # template's weight pre-pass then reads it through its element loader.
            from .convgen import gen_conv

            conv_need = _min_bytes(t.epilogue)
            if g.get("a_gather"):
                for gid_, b_ in _min_bytes(t.exp).items():
                    conv_need[gid_] = max(conv_need.get(gid_, 0), b_)
            conv = gen_conv(kernel, g, oexp, numerics, name, params, names, epi_fn, epi_args, conv_need, tile,
                            a_gather_fns=element_fn["a"] if g.get("a_gather") else None)
            if conv is not None:
                conv.sources[0] = src_options + conv.sources[0]
                return conv
        gcg = HipExpCodegen(names, {"row": "row", "k": "k", "b0": "b0", "b1": "b1", "b2": "b2"}, "  ", prefix=f"g{tag}", numerics=numerics)
        gcg.countReferences(oexp)
        gval = strip_parens(gcg.run(oexp))
        element_fn[tag] = (f"static __device__ __forceinline__ {in_t} jh_gather_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                           + "\n".join(gcg.take_lines()) + f"\n  return ({in_t})({gval});\n}}")
        gather_fns.append(element_fn[tag])
        gather_calls[tag] = f"jh_gather_{tag}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
        # Row-vector loader: when G = 8 or 4 consecutive rows of an aligned group read G consecutive elements, one
        # unaligned G-element load replaces G element loads and their index arithmetic; masked lanes are zeroed
        # afterwards (pairs measured slower than the element loader and are not used).  A group whose bytes would leave the buffer (first/last rows of the whole array, where the
        # out-of-range part is masked anyway) takes the element loader through an out-of-line call.
        r8, G = None, 0
        if g["dtype"] == DType.Float16 and tile.get("ROWS8", 1):
            for G in (8, 4):
                r8 = rows8_form(oexp, extent, G)
                if r8 is not None:
                    break
        if r8 is not None:
            idx0, cond_e, gnode = r8
            vnames = {"row": "row", "e": "e", "k": "k", "b0": "b0", "b1": "b1", "b2": "b2"}
            icg = HipExpCodegen(names, vnames, "  ", prefix=f"i{tag}", numerics=numerics)
            icg.countReferences(idx0)
            ival = strip_parens(icg.run(idx0))
            ilines = "\n".join(icg.take_lines())
            gather_fns.append(f"static __device__ __forceinline__ int jh_gindex_{tag}(int row, int k, int b0, int b1, int b2) {{\n"
                              f"{ilines}\n  return {ival};\n}}")
            gather_fns.append(mask_bits_fn(cond_e, tag, G, names, numerics))
            buf = names[gnode.arg[0]]
            # The loader only forms addresses and mask bits and issues the loads (no use of the loaded data, no
            # branches): the stager applies the mask when it writes the slab to LDS, one slab later, so the eight
            # loads of a block are in flight together.  A group that would leave the buffer loads from a clamped
            # address and is flagged; the stager replaces it through the out-of-line element loader afterwards.
            gather_fns.append(
                f"typedef jh_f16 jh_part_{tag} __attribute__((ext_vector_type({G})));\n"
                f"struct __attribute__((packed, aligned(2))) jh_part_u_{tag} {{ jh_part_{tag} v; }};\n"
                f"static __device__ __attribute__((noinline)) jh_half8 jh_gather8_slow_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                f"  jh_half8 v;\n#pragma unroll\n  for (int e = 0; e < 8; ++e) v[e] = jh_gather_{tag}(row + e, k, b0, b1, b2{epi_args});\n  return v;\n}}\n"
                f"static __device__ __forceinline__ jh_g8 jh_gather8_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                f"  jh_g8 out;\n  out.keep = 0u;\n#pragma unroll\n  for (int j = 0; j < {8 // G}; ++j) {{\n"
                f"    const int r = row + j * {G};\n    const int i0 = jh_gindex_{tag}(r, k, b0, b1, b2);\n"
                f"    const bool inside = (unsigned)i0 <= (unsigned)({gnode.arg[1]} - {G});\n"
                f"    if (!inside) out.keep |= 0x100u;\n"
                f"    const jh_part_{tag} part = reinterpret_cast<const jh_part_u_{tag}*>({buf} + (inside ? i0 : 0))->v;\n"
                f"#pragma unroll\n    for (int e = 0; e < {G}; ++e) out.v[j * {G} + e] = part[e];\n"
                f"    out.keep |= jh_mbits_{tag}(r, k, b0, b1, b2) << (j * {G});\n  }}\n"
                f"  return out;\n}}")
            gather_slow[tag] = f"jh_gather8_slow_{tag}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
            gather_calls[tag] = f"jh_gather8_{tag}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
            gather_flags[tag] = 2
            gather_group[tag] = G

        # float32: four consecutive rows of an aligned group as one 128-bit load (the image of a stride-1 convolution),
        # the operand staged like one that runs along its rows.  Groups whose bytes would leave the buffer take the
        # element loader, which applies the mask itself.
        if g["dtype"] == DType.Float32 and tile.get("ROWS4", 1) and extent % 4 == 0 and g["K"] % 8 == 0:
            r4 = rows8_form(oexp, extent, 4)
            if r4 is not None:
                idx0, cond_e, gnode = r4
                vnames = {"row": "row", "e": "e", "k": "k", "b0": "b0", "b1": "b1", "b2": "b2"}
                icg = HipExpCodegen(names, vnames, "  ", prefix=f"i{tag}", numerics=numerics)
                icg.countReferences(idx0)
                ival = strip_parens(icg.run(idx0))
                gather_fns.append(f"static __device__ __forceinline__ int jh_gindex_{tag}(int row, int k, int b0, int b1, int b2) {{\n"
                                  + "\n".join(icg.take_lines()) + f"\n  return {ival};\n}}")
                gather_fns.append(mask_bits_fn(cond_e, tag, 4, names, numerics))
                buf = names[gnode.arg[0]]
                # (raw data + mask bits, the load unconditional: see the k-vector loader below)
                gather_fns.append(
                    f"static __device__ __forceinline__ jh_g4 jh_gather4_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                    f"  const int i0 = jh_gindex_{tag}(row, k, b0, b1, b2);\n  jh_g4 out;\n  out.keep = 0u;\n"
                    f"  const bool inb = (unsigned)i0 <= (unsigned)({gnode.arg[1]} - 4);\n  __builtin_memcpy(&out.v, {buf} + (inb ? i0 : 0), 16);\n"
                    f"  out.keep = inb ? jh_mbits_{tag}(row, k, b0, b1, b2) : 0u;\n"
                    f"  if (__builtin_amdgcn_ballot_w64(!inb) != 0) {{\n    if (!inb) {{\n"
                    f"#pragma unroll\n      for (int e = 0; e < 4; ++e) out.v[e] = jh_gather_{tag}(row + e, k, b0, b1, b2{epi_args});\n      out.keep = 15u;\n    }}\n  }}\n  return out;\n}}")
                gather_calls[tag] = f"jh_gather4_{tag}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
                gather_flags[tag], gather_group[tag] = 5, 4

        # k-vector loader: when neither row form applies but G consecutive k of an aligned group read G consecutive elements
        # of one row (the activations under a filter cotangent: k = batch x positions), one G-element load per group feeds
        # the k-contiguous staging path; masked lanes are zeroed, groups that would leave the buffer go element by element.
        if gather_flags[tag] == 1 and tile.get("KVEC", 1) and g["K"] % 8 == 0:
            kv, G = None, 0
            for G in ((8, 4) if g["dtype"] == DType.Float16 else (4,)):
                kv = kvec_form(oexp, K_full, G)
                if kv is not None:
                    break
            if kv is not None:
                idx0, cond_e, gnode = kv
                vnames = {"row": "row", "e": "e", "k": "k", "b0": "b0", "b1": "b1", "b2": "b2"}
                icg = HipExpCodegen(names, vnames, "  ", prefix=f"ki{tag}", numerics=numerics)
                icg.countReferences(idx0)
                ival = strip_parens(icg.run(idx0))
                gather_fns.append(f"static __device__ __forceinline__ int jh_kindex_{tag}(int row, int k, int b0, int b1, int b2) {{\n"
                                  + "\n".join(icg.take_lines()) + f"\n  return {ival};\n}}")
                gather_fns.append(mask_bits_fn(cond_e, tag, G, names, numerics))
                buf = names[gnode.arg[0]]
                W = 8 if g["dtype"] == DType.Float16 else 4  # elements per chunk of the staging path
                part_t = (f"typedef {in_t} jh_kpart_{tag} __attribute__((ext_vector_type({G})));\n"
                          f"struct __attribute__((packed, aligned({2 if g['dtype'] == DType.Float16 else 4}))) jh_kpart_u_{tag} {{ jh_kpart_{tag} v; }};\n")
                if g["dtype"] == DType.Float16:
                    # The f16 loader hands back the raw vector and the mask as bits (`jh_g8`), to be applied when the staged
                    # registers are written to LDS, and its vector load is unconditional (a group that would leave the buffer
                    # loads from the buffer's start instead).  A select right behind the load would wait for the data inside
                    # the fetch, and a load under a branch makes the wait before the commit of the previous slab a wait for
                    # everything (the counter of loads in flight is not known at the join): either way one slab's loads are
                    # in flight instead of two.  Groups off the buffer are redone element by element under one wave-uniform
                    # branch, which consumes its own loads before it ends.
                    gather_fns.append(
                        part_t + f"static __device__ __forceinline__ jh_g8 jh_gatherk_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                        f"  jh_g8 out;\n  out.keep = 0u;\n  unsigned off = 0u;\n#pragma unroll\n  for (int j = 0; j < {W // G}; ++j) {{\n    const int kk = k + j * {G};\n"
                        f"    const int i0 = jh_kindex_{tag}(row, kk, b0, b1, b2);\n"
                        f"    const bool inb = (unsigned)i0 <= (unsigned)({gnode.arg[1]} - {G});\n"
                        f"    const jh_kpart_{tag} part = reinterpret_cast<const jh_kpart_u_{tag}*>({buf} + (inb ? i0 : 0))->v;\n"
                        f"#pragma unroll\n    for (int e = 0; e < {G}; ++e) out.v[j * {G} + e] = part[e];\n"
                        f"    if (inb) out.keep |= jh_mbits_{tag}(row, kk, b0, b1, b2) << (j * {G});\n"
                        f"    off |= (inb ? 0u : 1u) << j;\n  }}\n"
                        f"  if (__builtin_amdgcn_ballot_w64(off != 0u) != 0) {{\n#pragma unroll\n    for (int j = 0; j < {W // G}; ++j)\n      if ((off >> j) & 1u) {{\n"
                        f"#pragma unroll\n        for (int e = 0; e < {G}; ++e) out.v[j * {G} + e] = jh_gather_{tag}(row, k + j * {G} + e, b0, b1, b2{epi_args});\n"
                        f"        out.keep |= {(1 << G) - 1}u << (j * {G});\n      }}\n  }}\n"
                        f"  return out;\n}}")
                else:
                    gather_fns.append(
                        part_t + f"static __device__ __forceinline__ jh_g4 jh_gatherk_{tag}(int row, int k, int b0, int b1, int b2{epi_params}) {{\n"
                        f"  jh_g4 out;\n  out.keep = 0u;\n  const int i0 = jh_kindex_{tag}(row, k, b0, b1, b2);\n"
                        f"  const bool inb = (unsigned)i0 <= (unsigned)({gnode.arg[1]} - 4);\n"
                        f"  const jh_kpart_{tag} part = reinterpret_cast<const jh_kpart_u_{tag}*>({buf} + (inb ? i0 : 0))->v;\n"
                        f"#pragma unroll\n  for (int e = 0; e < 4; ++e) out.v[e] = part[e];\n"
                        f"  out.keep = inb ? jh_mbits_{tag}(row, k, b0, b1, b2) : 0u;\n"
                        f"  if (__builtin_amdgcn_ballot_w64(!inb) != 0) {{\n    if (!inb) {{\n"
                        f"#pragma unroll\n      for (int e = 0; e < 4; ++e) out.v[e] = jh_gather_{tag}(row, k + e, b0, b1, b2{epi_args});\n      out.keep = 15u;\n    }}\n  }}\n"
                        f"  return out;\n}}")
                gather_calls[tag] = f"jh_gatherk_{tag}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
                gather_flags[tag] = 7 if g["dtype"] == DType.Float16 else 6
                gather_group[tag] = G

    # Tap-major k order (see `tap_major_form`): one gather operand whose k splits into (channel, tap), the other a plain
    # strided operand.  Both are then loaded through block/chunk loaders that take the first k' of eight consecutive
    # ones: k' = tap * C + c, original k = c * T + tap.
    tap_major = None
    gtags = [tg for tg in ("a", "b") if gather_flags[tg]]
    if g["dtype"] == DType.Float16 and tile.get("TAPMAJOR", 0) and len(gtags) == 1 and g["K"] % 8 == 0:
        gt = gtags[0]
        pt = "b" if gt == "a" else "a"
        tm = tap_major_form(gather_oexp[gt], g["K"])
        plain_ok = g[f"{pt}_k0"] == g["K"] and not g.get(f"{pt}_gather")
        if tm is not None and plain_ok:
            form, G = None, 0
            for G in (8, 4, 1):
                form = rows8_form(tm["exp"], 0, G)
                if form is not None:
                    break
            if form is not None:
                idx0, cond_e, gnode = form
                T, C, CS = tm["T"], tm["C"], tm["cs"]
                vnames = {"row": "row", "e": "e", "tap": "tap", "b0": "b0", "b1": "b1", "b2": "b2"}
                icg = HipExpCodegen(names, vnames, "  ", prefix=f"ti{gt}", numerics=numerics)
                icg.countReferences(idx0)
                ival = strip_parens(icg.run(idx0))
                gather_fns.append(f"static __device__ __forceinline__ int jh_tindex_{gt}(int row, int tap, int b0, int b1, int b2) {{\n"
                                  + "\n".join(icg.take_lines()) + f"\n  return {ival};\n}}")
                if cond_e is not None:
                    mcg = HipExpCodegen(names, vnames, "  ", prefix=f"tm{gt}", numerics=numerics)
                    mcg.countReferences(cond_e)
                    mval = strip_parens(mcg.run(cond_e))
                    gather_fns.append(f"static __device__ __forceinline__ bool jh_tmask_{gt}(int row, int e, int tap, int b0, int b1, int b2) {{\n"
                                      + "\n".join(mcg.take_lines()) + f"\n  return {mval};\n}}")
                    mask_bits = f"jh_tmask_{gt}(r, e, tap, b0, b1, b2)"
                else:
                    mask_bits = "true"
                buf, LEN, NG = names[gnode.arg[0]], gnode.arg[1], 8 // G
                gather_fns.append(
                    f"typedef jh_f16 jh_tpart_{gt} __attribute__((ext_vector_type({G})));\n"
                    f"struct __attribute__((packed, aligned(2))) jh_tpart_u_{gt} {{ jh_tpart_{gt} v; }};\n"
                    f"static __device__ __attribute__((noinline)) jh_half8 jh_gather8_tslow_{gt}(int row, int kp, int b0, int b1, int b2{epi_params}) {{\n"
                    f"  const int tap = kp / {C};\n  const int k = (kp - tap * {C}) * {T} + tap;\n"
                    f"  jh_half8 v;\n#pragma unroll\n  for (int e = 0; e < 8; ++e) v[e] = jh_gather_{gt}(row + e, k, b0, b1, b2{epi_args});\n  return v;\n}}\n"
                    f"// Eight consecutive k' (one tap, channels c0 .. c0+7) of eight consecutive rows: loads only; the mask (one\n"
                    f"// per block, it does not depend on the channel) is applied when the block is written to LDS.\n"
                    f"static __device__ __forceinline__ jh_gblock jh_gather_block_{gt}(int row, int kbase, int b0, int b1, int b2{epi_params}) {{\n"
                    f"  jh_gblock out;\n  out.keep = 0u;\n  const int tap = kbase / {C};\n  const int c0 = kbase - tap * {C};\n"
                    f"#pragma unroll\n  for (int j = 0; j < {NG}; ++j) {{\n    const int r = row + j * {G};\n"
                    f"    const int i0 = jh_tindex_{gt}(r, tap, b0, b1, b2) + c0 * {CS};\n"
                    f"    const bool inside = i0 >= 0 && (long long)i0 + 7ll * {CS} <= {LEN}ll - {G};\n"
                    f"    if (!inside) out.keep |= 0x100u;\n"
                    f"#pragma unroll\n    for (int e = 0; e < {G}; ++e) if ({mask_bits}) out.keep |= 1u << (j * {G} + e);\n"
                    f"    const jh_f16* const src = {buf} + (inside ? i0 : 0);\n"
                    f"#pragma unroll\n    for (int i = 0; i < 8; ++i) {{\n"
                    f"      const jh_tpart_{gt} part = reinterpret_cast<const jh_tpart_u_{gt}*>(src + (inside ? i * {CS} : 0))->v;\n"
                    f"#pragma unroll\n      for (int e = 0; e < {G}; ++e) out.v[i][j * {G} + e] = part[e];\n    }}\n  }}\n  return out;\n}}")
                gather_slow[gt] = f"jh_gather8_tslow_{gt}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
                gather_calls[gt] = f"jh_gather_block_{gt}(row, k, jh_b0, jh_b1, jh_b2{epi_args})"
                gather_flags[gt], gather_group[gt] = 3, G
                # the plain operand, eight consecutive k' at a time: elements T * stride apart
                srow, sk = (g["a_sm"], g["a_sk"]) if pt == "a" else (g["b_sn"], g["b_sk"])
                gather_fns.append(
                    f"static __device__ __forceinline__ jh_half8 jh_gather_chunk_{pt}(const jh_f16* __restrict__ base, int row, int kbase) {{\n"
                    f"  const int tap = kbase / {C};\n  const int c0 = kbase - tap * {C};\n"
                    f"  const jh_f16* p = base + (long long)row * {srow}ll + ((long long)c0 * {T} + tap) * {sk}ll;\n  jh_half8 v;\n"
                    f"#pragma unroll\n  for (int e = 0; e < 8; ++e) v[e] = p[(long long)e * {T * sk}ll];\n  return v;\n}}")
                gather_calls[pt] = f"jh_gather_chunk_{pt}({'Ap' if pt == 'a' else 'Bp'}, row, k)"
                gather_flags[pt] = 4
                tap_major = dict(T=T, C=C, group=G)

    # Batch index decode, innermost batch axis last in g["batch"].
    lines = ["  {", "    int rem = batch;"]
    for k, (size, sa, sb, sc) in reversed(list(enumerate(g["batch"]))):
        lines.append(f"    jh_b{k} = rem % {size}; rem /= {size};")
        lines.append(f"    a_base += (long long)jh_b{k} * {sa}ll; b_base += (long long)jh_b{k} * {sb}ll; c_base += (long long)jh_b{k} * {sc}ll;")
    lines.append("  }")
    nbatch = 1
    for b in g["batch"]:
        nbatch *= b[0]
    pitch = -(-kernel.size // 8) * 8  # elements between two slices' partial outputs
    if split > 1:
        # a slice starts K elements further along k: K * sk for one stride, (K / k0) runs of sk1 for two
        # (whether the axis has two strides is the whole axis's property: a slice of exactly one run has k0 == K too)
        # and for runs cut into r slices each, slice z is piece z % r of run z / r
        def slice_offset(tag):
            if not two_stride[tag]:
                return f"(long long)blockIdx.y * {g['K'] * g[tag + '_sk']}ll"
            if g["K"] % run_full[tag] == 0:
                return f"(long long)blockIdx.y * {(g['K'] // run_full[tag]) * g[tag + '_sk1']}ll"
            r = run_full[tag] // g["K"]
            return f"((long long)(blockIdx.y / {r}) * {g[tag + '_sk1']}ll + (long long)(blockIdx.y % {r}) * {g['K'] * g[tag + '_sk']}ll)"

        lines.append(f"  a_base += {slice_offset('a')}; b_base += {slice_offset('b')};"
                     + ("" if fusek else f" c_base += (long long)blockIdx.y * {pitch}ll;"))
        lines.append(f"  const int jh_k_off = (int)blockIdx.y * {g['K']};  // a gather loader is asked for k of the whole axis")
        for d in (gather_calls, gather_slow):
            for tag in list(d):
                d[tag] = d[tag].replace("(row, k, ", "(row, k + jh_k_off, ")

    tmpl = "gemm_f16.hip.inc" if g["dtype"] == DType.Float16 else "gemm_f32.hip.inc"
    fBK = int(tile.get("BK", 16)) if g["dtype"] == DType.Float32 else 0  # slab depth of the f32 template
    if g["dtype"] == DType.Float32 and (fBK not in (16, 32, 64) or 2 * (BM + BN) * (fBK + 4) * 4 > 160 * 1024):
        raise ValueError(f"f32 slab depth {fBK} is not 16, 32 or 64, or two {BM}+{BN}-row slabs of it do not fit the LDS")
    # Fast path: direct global->LDS loads need whole tiles (no bounds predicates) and 32-deep slabs.
    # Slab depth.  When both operands run along k in memory, 64-deep slabs make every row of a slab one whole
    # 128-byte line (a 32-deep slab asks for the two halves of each line about a microsecond apart, as two requests):
    # measured +7..21 % on every tile shape.  An operand that runs along m or n is fetched in whole lines either way,
    # and the shorter pipeline that 64-deep slabs leave room for then costs more than it gains.
    both_k = g["a_sk"] == 1 and g["b_sk"] == 1 and g["K"] % 64 == 0 and g["K"] >= 128
    dBK = tile.get("BK", 64 if both_k and tile.get("PIPE", 1) else 32) if g["dtype"] == DType.Float16 else 32
    if dBK not in (32, 64):
        raise ValueError(f"direct-to-LDS slab depth must be 32 or 64, got {dBK}")
    a_kc, b_kc = g["a_sk"] == 1 or g["K"] == 1, g["b_sk"] == 1 or g["K"] == 1
    full = (_edge_ok(load_rows["a"], BM, a_kc) and _edge_ok(load_rows["b"], BN, b_kc) and g["K"] % dBK == 0 and BM >= 128 and BN >= 128
            and tile.get("EDGE", 1) | (g["M"] % BM == 0 and g["N"] % BN == 0))
    any_gather = bool(g.get("a_gather") or g.get("b_gather"))
    loose = {tag: 1 if g.get(tag + "_loose") and not g.get(tag + "_gather") else 0 for tag in ("a", "b")}
    dlds = g["dtype"] == DType.Float16 and full and tile.get("DLDS", 1) and not any_gather and not (loose["a"] or loose["b"])
    if repack and not dlds:  # the copy only serves the direct loads: plan again without it
        import copy

        t2 = copy.copy(t)
        t2.params = dict(t.params, gemm_tile=tuple(sorted(dict(override, REPACK=0).items())))
        return gen_gemm(kernel, t2, numerics, name)
    if dlds:
        tmpl = "gemm_f16_dlds.hip.inc"
    if dlds:
        # Stages that fit the 160 KiB of LDS: four of a 32-deep slab; of a 64-deep slab four (128x128), three
        # (128x256, 256x128), or the five-unit ring (256x256: 2.5 slabs).
        ring_default = 5 if dBK == 64 and (BM, BN) == (256, 256) and "STAGES" not in tile and tile.get("PIPE", 1) else 0
        stages_default = 4 if dBK == 32 else min(4, (160 * 1024) // ((BM + BN) * dBK * 2))
        sched = dict(BK=dBK, STAGES=tile.get("STAGES", stages_default), PIPE=tile.get("PIPE", 1), SGB=tile.get("SGB", 1), ASM_LOAD=tile.get("ASM", 1))
        # Scalar-base addressing needs every lane offset inside one slab of a tile to fit 32 bits.
        span = 2 * max((BM - 1) * abs(g["a_sm"]) + dBK * abs(g["a_sk"]), (BN - 1) * abs(g["b_sn"]) + dBK * abs(g["b_sk"]))
        sched["SADDR"] = 1 if tile.get("SADDR", 1) and span < 2 ** 31 and g["a_sm"] >= 0 and g["a_sk"] >= 0 and g["b_sn"] >= 0 and g["b_sk"] >= 0 else 0
        sched.update(PIN=tile.get("PIN", 1), BAR_AT=tile.get("BAR_AT", 2), READ_AHEAD=tile.get("RA", 1), LOADS_LATE=tile.get("LATE", 1))
        # Tile walk: groups of 4 tile rows (8192^3: 865 -> 853 us against groups of 8, 873 with 16; one group spanning
        # all rows loses a third).  Nontemporal C stores only for the f32 partials of a k split, where a wave's store
        # covers whole 128-byte lines (128x14336x4096: 26.1 -> 25.3 us): with 2-byte outputs they gain nothing once the
        # walk is in groups of 4 and the half-line writes cost a third more HBM write traffic (WRITE_SIZE 132 -> 176 MiB).
        sched.update(GROUP_M=int(tile.get("GM", 4)), NT_STORE=int(tile.get("NTS", 1 if split > 1 and not fusek else 0)), FUSEK=fusek)
        sched["RING"] = ring = tile.get("RING", ring_default)
        if ring and (ring != 5 or BM != BN or not sched["PIPE"]):
            raise ValueError("the unit ring is five units of a square block tile under the phase-pipelined loop")
        if (ring * BM * dBK * 2 if ring else sched["STAGES"] * (BM + BN) * dBK * 2) > 160 * 1024:
            raise ValueError(f"{ring or sched['STAGES']} {'units' if ring else 'stages'} of a {BM}x{BN}x{dBK} slab do not fit the 160 KiB of LDS")
        # Vector epilogue: needs unit column stride and 8-element alignment of every row / batch start of C.
        # It pays when the epilogue itself reads buffers (bias, residual): those become 128-bit loads.  A plain
        # cast-and-store epilogue measures the same either way and keeps the simpler path.
        has_loads = bool(epilogue.collect(lambda x: x.op == AluOp.GlobalIndex)) and split == 1
        vec = (split == 1 and tile.get("VEPI", 1 if has_loads else 0) and g["c_sn"] == 1 and g["c_sm"] % 8 == 0 and all(b[3] % 8 == 0 for b in g["batch"])
               and kernel.dtype != DType.Bool and (g["N"] % BN == 0 or g["N"] % 8 == 0))  # an edge tile ends on a whole group of 8
        if vec:
            vnames = {"acc": "acc", "row": "row", "col": "col", "b0": "b0", "b1": "b1", "b2": "b2"}
            body = _Body(epilogue, names, vnames, "col", "c0", 8, classify_loads(epilogue, "col", 8), numerics, "      ", "e")
            vhoist, vloads = body.hoisted()
            vbody, vvalue = body.lanes(vloads)
            sched.update(VEC_EPI=1, VEPI_LOADS=vhoist, VEPI_BODY=vbody, VEPI_VALUE=vvalue, OUT_T=out_t)
        else:
            sched.update(VEC_EPI=0, VEPI_LOADS="", VEPI_BODY="", VEPI_VALUE="0", OUT_T=out_t)
    elif g["dtype"] == DType.Float16:
        sched = dict(COMMIT_A=tile.get("CA", 2), COMMIT_B=tile.get("CB", 3), FETCH_A=tile.get("FA", 0),
                     FETCH_B=tile.get("FB", 1), IGLP=tile.get("IGLP", -1), SCHED_FENCE=tile.get("FENCE", 0),
                     A_LOOSE=loose["a"], B_LOOSE=loose["b"])
    else:
        sched = dict(BK=fBK, FRAG_FENCE=int(tile.get("FENCE", 1)), FUSEK=fusek, A_LOOSE=loose["a"], B_LOOSE=loose["b"])
    if not dlds:
        sched.update(GATHER_FNS="\n".join(gather_fns), A_GATHER=gather_flags["a"], B_GATHER=gather_flags["b"],
                     GATHER_A_CALL=gather_calls["a"], GATHER_B_CALL=gather_calls["b"],
                     GATHER_A_SLOW=gather_slow.get("a", "jh_half8{0, 0, 0, 0, 0, 0, 0, 0}"), GATHER_B_SLOW=gather_slow.get("b", "jh_half8{0, 0, 0, 0, 0, 0, 0, 0}"))
    src = src_options + _prelude(numerics) + fill(template(tmpl), dict(sched, 
        M=g["M"], N=g["N"], K=g["K"], M_LOAD=load_rows["a"], N_LOAD=load_rows["b"], BM=BM, BN=BN, WM=WM, WN=WN,
        A_KCONTIG=0 if gather_flags["a"] in (2, 3, 5) else (1 if g["a_sk"] == 1 or g["K"] == 1 or gather_flags["a"] in (1, 4, 6, 7) else 0),
        B_KCONTIG=0 if gather_flags["b"] in (2, 3, 5) else (1 if g["b_sk"] == 1 or g["K"] == 1 or gather_flags["b"] in (1, 4, 6, 7) else 0),
        NBATCH=nbatch, EPILOGUE_FN=epi_fn, NAME=name, PARAMS=params,
        A_OFF=g["a_off"], B_OFF=g["b_off"], BATCH_DECODE="\n".join(lines),
        A_PTR="jh_repack_a" if "a" in (repack or "") else names[g["gid_a"]], B_PTR="jh_repack_b" if "b" in (repack or "") else names[g["gid_b"]],
        A_SM=g["a_sm"], A_SK=g["a_sk"], B_SN=g["b_sn"], B_SK=g["b_sk"],
        A_K0=g["a_k0"], A_SK1=g["a_sk1"], B_K0=g["b_k0"], B_SK1=g["b_sk1"],
        C_SM=g["c_sm"], C_SN=g["c_sn"], EPILOGUE_ARGS=epi_args))
    tiles = -(-g["M"] // BM) * -(-g["N"] // BN) * nbatch
    if fusek and g["dtype"] == DType.Float16 and not dlds:
        raise ValueError("an in-launch fold of a k split needs the direct-to-LDS f16 template or the f32 template")
    out_args = [("out", 0), ("scratch", 0), ("scratch", 1)] if fusek else [("scratch", 0) if split > 1 else ("out", 0)]
    step = LaunchStep(name, (tiles, split, 1), (nthreads, 1, 1), 0, [("in", i) for i in range(kernel.nargs)] + out_args)
    need = _min_bytes(t.epilogue)
    if any_gather:
        for gid_, b_ in _min_bytes(t.exp).items():
            need[gid_] = max(need.get(gid_, 0), b_)
    eb = byteWidth(g["dtype"])
    need[g["gid_a"]] = max(need.get(g["gid_a"], 0), g["a_len"] * eb)
    need[g["gid_b"]] = max(need.get(g["gid_b"], 0), g["b_len"] * eb)
    info = dict(BM=BM, BN=BN, WM=WM, WN=WN, BK=dBK if dlds else (64 if g["dtype"] == DType.Float16 else fBK), direct_lds=bool(dlds), tiles=tiles, a_kcontig=g["a_sk"] == 1, b_kcontig=g["b_sk"] == 1,
                M=g["M"], N=g["N"], K=K_full, nbatch=nbatch, splitk=split)
    if dlds:
        info.update(stages=sched["STAGES"], ring=sched["RING"])
    if any_gather:
        info["gather"] = {tag: {0: "none", 1: "element", 2: f"rows{gather_group.get(tag, 8)}", 3: f"tap-major rows{gather_group.get(tag, 8)}",
                                4: "tap-major strided" if tap_major is not None else f"k{gather_group.get(tag, 8)}", 5: "rows4", 6: "k4", 7: f"k{gather_group.get(tag, 8)}"}[gather_flags[tag]] for tag in ("a", "b")}
        if tap_major is not None:
            info["tap_major"] = tap_major
    if repack:
        src += "\nstruct __attribute__((packed, aligned(2))) jh_half8_u { jh_half8 v; };\n"
        preps, scratch = [], []
        for si, tg in enumerate(repack):
            rs = repack_src[tg]
            if rs["kc"]:
                groups, outer, total = rs["k_pad"] // 8, rs["rows"], rs["rows"] * (rs["k_pad"] // 8)
                body = (f"  const int r = (int)(i / {groups}), k0 = (int)(i % {groups}) * 8;\n"
                        f"  const jh_f16* __restrict__ p = src + {rs['off']}ll + (long long)r * {rs['srow']}ll + k0;\n"
                        f"  const int valid = {rs['k']} - k0;\n"
                        f"  jh_f16* const q = dst + (long long)r * {rs['k_pad']} + k0;\n")
                what = f"[{rs['rows']} rows][{rs['k']} k] (row stride {rs['srow']}) -> [{rs['rows']}][{rs['k_pad']}]"
            else:
                groups, total = rs["rows_pad"] // 8, rs["k_pad"] * (rs["rows_pad"] // 8)
                body = (f"  const int k = (int)(i / {groups}), r0 = (int)(i % {groups}) * 8;\n"
                        f"  const jh_f16* __restrict__ p = src + {rs['off']}ll + (long long)k * {rs['sk']}ll + r0;\n"
                        f"  const int valid = k < {rs['k']} ? {rs['rows']} - r0 : 0;\n"
                        f"  jh_f16* const q = dst + (long long)k * {rs['rows_pad']} + r0;\n")
                what = f"[{rs['k']} k][{rs['rows']} rows] (k stride {rs['sk']}) -> [{rs['k_pad']}][{rs['rows_pad']}]"
            src += (f"""
// Operand {tg.upper()} {what}, first element {rs['off']}: eight elements per thread, one under-aligned 16-byte load and one
// aligned store; what lies past the operand's extents is zeros.
extern "C" __global__ __launch_bounds__(256) void {name}_repack_{tg}(const jh_f16* __restrict__ src, jh_f16* __restrict__ dst) {{
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= {total}ll) return;
{body}  jh_half8 v;
  if (valid >= 8) {{
    v = reinterpret_cast<const jh_half8_u*>(p)->v;
  }} else {{
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = e < valid ? p[e] : (jh_f16)0.0f;
  }}
  *reinterpret_cast<jh_half8*>(q) = v;
}}
""")
            preps.append(LaunchStep(f"{name}_repack_{tg}", (-(-total // 256), 1, 1), (256, 1, 1), 0, [("in", rs["gid"]), ("scratch", si)]))
            step.args.append(("scratch", si))
            scratch.append(rs["k_pad"] * rs["rows_pad"] * 2)
        info["repack"] = repack
        return KernelSource([src], preps + [step], scratch, "gemm", need, info)
    if split == 1:
        return KernelSource([src], [step], [], "gemm", need, info)
    if fusek:
        info["fused_fold"] = True
        return KernelSource([src], [step], [split * tiles * BM * BN * 4, tiles * 4], "gemm", need, info, zeroed_scratch=[1])
    from .kernelgen import fold_stage

    ks2, steps2, partial_len = fold_stage(kernel, numerics, name, split, pitch, slice_major=True)
    info["stage2"] = ks2.info
    need.update({gid_: b_ for gid_, b_ in ks2.min_input_bytes.items() if gid_ != kernel.nargs})
    return KernelSource([src] + ks2.sources, [step] + steps2, [partial_len * 4], "gemm+fold", need, info)
