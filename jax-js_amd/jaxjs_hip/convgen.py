"""Stride-1 convolution as an implicit GEMM with the image patch resident in LDS (template `conv_f16.hip.inc`).

The front-end lowers `convGeneralDilated` to one reduce Kernel whose image operand is read through a chain of
padded / windowed views (src/frontend/convolution.ts:410-442, src/frontend/jit.ts:622-635); the GEMM matcher sees it as
a *gather* operand.  Nothing here looks at the op that produced the kernel: `match_conv` takes the operand's lowered index
expression, proposes the geometry of a stride-1, undilated window walk (image width and height, window size, padding,
channel and batch strides) from a few probes, and then *evaluates the expression itself* on every (output position, tap)
pair -- index and padding mask -- against that model.  Only an exact match takes the specialised kernel; everything
else stays on the generic gather loaders of `gemm.py`.
"""

from __future__ import annotations

from typing import Dict, Optional

import numpy as np

from .alu import AluExp, AluOp, DType


def np_eval(e: AluExp, env: Dict[str, np.ndarray], memo: Optional[dict] = None):
    """Vectorised evaluation of an integer / boolean index expression over numpy int64 arrays bound to its Specials.
    Raises NotImplementedError for anything that is not index arithmetic."""
    memo = {} if memo is None else memo
    key = id(e)
    if key in memo:
        return memo[key]
    op = e.op
    if op == AluOp.Const:
        r = np.int64(int(e.arg)) if e.dtype != DType.Bool else np.bool_(bool(e.arg))
    elif op == AluOp.Special:
        r = env[e.arg[0]]
    elif op in (AluOp.Add, AluOp.Sub, AluOp.Mul, AluOp.Idiv, AluOp.Mod, AluOp.Cmplt, AluOp.Cmpne):
        a, b = np_eval(e.src[0], env, memo), np_eval(e.src[1], env, memo)
        if op == AluOp.Cmplt:
            r = a < b
        elif op == AluOp.Cmpne:
            r = a != b
        elif e.dtype == DType.Bool:
            r = {AluOp.Add: np.logical_or, AluOp.Mul: np.logical_and, AluOp.Sub: np.not_equal}[op](a, b)
        elif e.dtype != DType.Int32:
            raise NotImplementedError(f"{op} on {e.dtype}")
        elif op == AluOp.Add:
            r = a + b
        elif op == AluOp.Sub:
            r = a - b
        elif op == AluOp.Mul:
            r = a * b
        else:
            if np.any(np.asarray(b) <= 0) or np.any(np.asarray(a) < 0):
                raise NotImplementedError("division with a negative operand")
            r = a // b if op == AluOp.Idiv else a % b
    elif op == AluOp.Where:
        c = np_eval(e.src[0], env, memo)
        r = np.where(c, np_eval(e.src[1], env, memo), np_eval(e.src[2], env, memo))
    elif op == AluOp.Cast and e.dtype == DType.Int32 and e.src[0].dtype in (DType.Int32, DType.Bool):
        r = np.asarray(np_eval(e.src[0], env, memo)).astype(np.int64)
    else:
        raise NotImplementedError(str(op))
    memo[key] = r
    return r


def match_conv(oexp: AluExp, extent: int, K: int, batch: list) -> Optional[dict]:
    """Geometry of a stride-1 window walk, or None.  `oexp` is the gather operand in (row, k, b0..) coordinates: `row`
    the output position inside one image (0 .. extent-1), `k` = channel * taps + tap."""
    from .gemm import tap_major_form

    if len(batch) > 1:
        return None
    tm = tap_major_form(oexp, K)
    if tm is None:
        return None
    T, C, cs = tm["T"], tm["C"], tm["cs"]
    e = tm["exp"]
    cond, node = None, e
    if node.op == AluOp.Where:
        cond, node = node.src[0], node.src[1]
    if node.op != AluOp.GlobalIndex or node.dtype != DType.Float16:
        return None
    nb = batch[0][0] if batch else 1
    rows = np.arange(extent, dtype=np.int64)[:, None]
    taps = np.arange(T, dtype=np.int64)[None, :]

    def at(b):
        env = {"row": rows, "tap": taps, "b0": np.int64(b), "b1": np.int64(0), "b2": np.int64(0)}
        try:
            idx = np.broadcast_to(np_eval(node.src[0], env), (extent, T))
            ok = np.ones((extent, T), bool) if cond is None else np.broadcast_to(np_eval(cond, env), (extent, T))
        except (NotImplementedError, KeyError):
            return None
        return idx, ok

    first = at(0)
    if first is None:
        return None
    idx, ok = first
    # Probes.  The window width is where consecutive taps stop being consecutive elements, and what the next window
    # row advances by is the image width (a window of one row says nothing about it: every divisor of the plane is
    # tried); the output width is where consecutive positions stop being consecutive -- or, when output and image are
    # equally wide (the index is then linear in the position), whichever divisor of the position count makes the
    # padding mask come out right.  Every candidate is checked against the whole table.
    d_tap = np.diff(idx[0, :])
    tbreaks = np.nonzero(d_tap != 1)[0]
    KW = int(tbreaks[0]) + 1 if len(tbreaks) else T
    if T % KW:
        return None
    KH = T // KW
    # consecutive output positions advance by the column stride; the first break ends an output row
    d_row = np.diff(idx[:, 0])
    SX = int(d_row[0]) if len(d_row) else 1
    if SX < 1:
        return None
    breaks = np.nonzero(d_row != SX)[0]
    base = int(idx[0, 0])  # = -(PH * W + PW): position 0 with tap 0 sits PH rows and PW columns before the plane
    if base > 0:
        return None
    if KH > 1:
        widths = [int(idx[0, KW] - idx[0, 0])]
    else:
        widths = [d for d in range(cs, 0, -1) if cs % d == 0]
    ky, kx = taps // KW, taps % KW
    found = None
    for W in widths:
        if W <= 0 or cs % W:
            continue
        H = cs // W
        PH, PW = (-base) // W, (-base) % W
        candidates = [int(breaks[0]) + 1] if len(breaks) else [-(-W // SX)] + [d for d in range(extent, 0, -1) if extent % d == 0 and d != -(-W // SX)]
        for OW in candidates:
            if OW <= 0 or extent % OW:
                continue
            # the row stride: from the first position of the second output row, else (one output row) 1
            SY = 1
            if extent > OW:
                step = int(idx[OW, 0]) - base
                if step <= 0 or step % W:
                    continue
                SY = step // W
            oy, ox = rows // OW, rows % OW
            iy, ix = SY * oy + ky - PH, SX * ox + kx - PW
            valid = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
            model = iy * W + ix
            if np.array_equal(ok, valid) and np.array_equal(idx[valid], model[valid]) and (cond is not None or valid.all()):
                found = (W, H, PH, PW, OW, SY)
                break
        if found:
            break
    if found is None:
        return None
    W, H, PH, PW, found, SY = found
    OW, OH = found, extent // found
    SB = 0
    if nb > 1:
        second = at(1)
        if second is None or not np.array_equal(second[1], ok):
            return None
        delta = second[0] - idx
        SB = int(delta[0, 0])
        if not np.all(delta[valid] == SB) or SB < 0:
            return None
        last = at(nb - 1)
        if last is None or not np.all((last[0] - idx)[valid] == SB * (nb - 1)):
            return None
    length = node.arg[1]
    if (nb - 1) * SB + (C - 1) * cs + H * W > length:
        return None
    return dict(gid=node.arg[0], length=length, T=T, C=C, SC=cs, SB=SB, NB=nb, OW=OW, OH=OH, KW=KW, KH=KH, W=W, H=H, PH=PH, PW=PW, SX=SX, SY=SY)


def _pitch(elems: int) -> int:
    """Channel pitch of a patch copy: a multiple of 16 elements (8 dwords, the width one ds_read_b64_tr_b16 row group
    spans) whose dword count modulo the 64 banks is a multiple of 8 other than 0 and 32, so that the four k rows of a
    transposing read fall on disjoint bank ranges."""
    p = -(-elems // 16) * 16
    while (p // 2) % 64 in (0, 32):
        p += 16
    return p


def gen_conv(kernel, g: dict, oexp: AluExp, numerics: str, name: str, params: str, names: list, epi_fn: str, epi_args: str,
             need: dict, tile: dict, a_gather_fns: Optional[str] = None):
    """KernelSource of the patch-in-LDS convolution for a GEMM whose B operand `oexp` is a stride-1 window walk, or None
    when the shape is outside what the template covers (it then stays on the generic gather loaders)."""
    from .kernelgen import KernelSource, LaunchStep, _prelude, fill, template

    if g.get("b_k0") != g["K"] or (a_gather_fns is None and g["a_k0"] != g["K"]) or len(g["batch"]) > 1:
        return None
    cv = match_conv(oexp, g["N"], g["K"], g["batch"])
    if cv is None:
        return None
    O, C, OW = g["M"], cv["C"], cv["OW"]
    if C % 16 or O % 64:  # whole MFMA k steps, whole 64-channel tiles
        return None
    # Output rows are walked at a width of whole 4-position groups (8-byte aligned row offsets in LDS): the up to three
    # extra columns per row are computed and dropped.  Positions, tiles and the patch pitch all use this width.
    OWP = -(-OW // 4) * 4
    NV = cv["OH"] * OWP
    # 256 positions per tile (wave tile 32 x 128: four MFMAs per A fragment) unless the image is smaller than that;
    # 128 output channels per tile from 256 channels on, as long as that still gives every CU a tile (small images:
    # [32,256,14,14] 44 -> 29 us, [32,512,7,7] 84 -> 52 us with 64)
    from . import tuner
    BN = int(tile.get("CBN", 256 if NV >= 256 else 128))
    wide = O % 128 == 0 and O >= 256 and -(-NV // BN) * (O // 128) * cv["NB"] >= tuner.CU_COUNT
    BM = int(tile.get("CBM", 128 if wide else 64))
    WM, WN = int(tile.get("CWM", 2)), int(tile.get("CWN", 2))
    if O % BM or BM % (32 * WM) or BN % (32 * WN) or BN % 4:
        return None
    # output rows a tile's BN consecutive positions span; the image rows behind them live in SY planes (by row % SY) of
    # RP rows each: plane rows from floor(-PH / SY) to floor((KH - 1 - PH) / SY) past the tile's first and last row
    # The patch holds whole image rows: a row several times as wide as the tile (a long 1-D signal: 1500 positions against
    # 256) would be filled again by every tile along it, slab after slab ([1,384,3000] * [384,384,3] stride 2: 500 us here,
    # 49 us on the gather loaders).
    if OWP > 4 * BN:
        return None
    n_tiles = -(-NV // BN)
    spans = max((min(t * BN + BN - 1, NV - 1) // OWP) - ((t * BN) // OWP) + 1 for t in range(n_tiles))
    SX, SY = cv["SX"], cv["SY"]
    qmin, qmax = (-cv["PH"]) // SY, (cv["KH"] - 1 - cv["PH"]) // SY
    RP = spans + qmax - qmin
    R = SY * RP
    P = _pitch(R * OWP)
    GO = 8 if OWP % 8 == 0 and SX == 1 and cv["W"] >= 8 else 4   # output columns per fill vector (16- or 8-byte LDS stores)
    G = GO * SX                                  # image elements per fill vector
    SR = cv["KW"] - 1 - cv["PW"]
    # neighbour-exchange fill: rows of whole aligned vectors that line up with the output columns
    xch = G in (4, 8) and OWP == OW and cv["W"] % G == 0 and cv["W"] == SX * OW and OW // GO <= 64 and cv["PW"] < G and SR - SX + 1 < G
    # otherwise: unaligned vector loads, clamped into the row and shifted into place; a vector may hang over the row's
    # start by PW and over its end by the window's reach plus the columns the walking width adds
    smax = max(cv["PW"], SR) if xch else max(cv["PW"], max(0, SX * (OWP - GO) + SR - (cv["W"] - G)))
    if not xch and (G not in (4, 8) or cv["W"] < G or smax >= G):
        return None
    # channels per slab: 16 (one MFMA k step per tap) measured fastest on every shape tried -- short slabs keep the fill of
    # the next patch and the MFMAs of this one in step, and leave LDS for a second workgroup per CU
    # (32 when the patch is small and there are many slabs to walk: 3-4 % on the 14x14 and 7x7 shapes)
    CS = int(tile.get("CCS", 32 if C % 32 == 0 and C >= 128 and cv["KW"] * 32 * P * 2 <= 40 * 1024 else 16))
    if not CS or C % CS or cv["KW"] * CS * P * 2 > 160 * 1024:
        return None
    sb_c = g["batch"][0][3] if g["batch"] else 0
    src = _prelude(numerics) + fill(template("conv_f16.hip.inc"), dict(
        OW=OW, OWP=OWP, OH=cv["OH"], W=cv["W"], H=cv["H"], KH=cv["KH"], KW=cv["KW"], PH=cv["PH"], PW=cv["PW"], C=C, O=O,
        SC=cv["SC"], SB=cv["SB"], NB=cv["NB"], BM=BM, BN=BN, WM=WM, WN=WN, CS=CS, R=R, P=P, G=G, SMAX=smax,
        SX=SX, SY=SY, RP=RP, QMIN=qmin, XCH=int(xch),
        EPILOGUE_FN=epi_fn, EPILOGUE_ARGS=epi_args, NAME=name, PARAMS=params, IMG_PTR=names[cv["gid"]],
        A_GATHER=0 if a_gather_fns is None else 1, A_GATHER_FNS=a_gather_fns or "",
        A_OFF=g["a_off"], A_SM=g["a_sm"], A_SK=g["a_sk"], C_SM=g["c_sm"], C_SN=g["c_sn"], C_SB=sb_c))
    T = cv["T"]
    total_w = T * O * C
    nargs = kernel.nargs
    if a_gather_fns is None:
        prep_args = [("in", g["gid_a"]), ("scratch", 0)]
    else:  # the element loader of a gathered filter takes every buffer of the kernel
        prep_args = [("in", i) for i in range(nargs)] + [("out", 0), ("scratch", 0)]
    prep = LaunchStep(name + "_wprep", (-(-total_w // 256), 1, 1), (256, 1, 1), 0, prep_args)
    tiles = n_tiles * (O // BM) * cv["NB"]
    main = LaunchStep(name, (tiles, 1, 1), (64 * WM * WN, 1, 1), 0,
                      [("in", i) for i in range(nargs)] + [("out", 0), ("scratch", 0)])
    need = dict(need)
    if a_gather_fns is None:
        need[g["gid_a"]] = max(need.get(g["gid_a"], 0), g["a_len"] * 2)
    need[cv["gid"]] = max(need.get(cv["gid"], 0), ((cv["NB"] - 1) * cv["SB"] + (C - 1) * cv["SC"] + cv["H"] * cv["W"]) * 2)
    info = dict(BM=BM, BN=BN, WM=WM, WN=WN, BK=16, direct_lds=False, tiles=tiles, M=O, N=g["N"], K=g["K"], nbatch=cv["NB"], splitk=1,
                conv=dict(cv, CS=CS, R=R, P=P, G=G, OWP=OWP, exchange=bool(xch)), gather=dict(a="none" if a_gather_fns is None else "element (pre-pass)", b="patch"))
    return KernelSource([src], [prep, main], [total_w * 2], "gemm", need, info)
