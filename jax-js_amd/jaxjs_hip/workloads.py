"""Traced programs for the benchmark configurations: the fused row-softmax/argmax pair and the
GPT-2-small transformer block.  Each returns a `JitProgram` (a list of Kernels plus buffer
lifetimes) exactly as the restated `jit()` splits it; nothing here is specific to a backend."""

from __future__ import annotations

from typing import Dict, List, Tuple

from . import jit as J
from . import library as L
from .alu import DType
from .jit import JitProgram, ShapedArray


def rowSoftmaxArgmaxProgram(rows: int, cols: int) -> JitProgram:
    """y = sum(exp(x - max(x)) * sigmoid(x), axis=-1) and argmax(x, axis=-1) of x f32 [rows, cols]:
    four streaming row reductions (no common-subexpression elimination across the two maxima)."""
    def f(x):
        m = x.max(-1, keepdims=True)
        y = J.exp(x.sub(m)).mul(L.sigmoid(x)).sum(-1)
        return [y, L.argmax(x, -1)]
    return J.jit(f, [ShapedArray((rows, cols), DType.Float32)])


GPT2_BLOCK_PARAMS = ("ln1_g", "ln1_b", "w_qkv", "b_qkv", "w_o", "b_o", "ln2_g", "ln2_b", "w_fc1", "b_fc1", "w_fc2", "b_fc2")


def gpt2BlockShapes(batch: int, seq: int, d_model: int, d_ff: int) -> Dict[str, Tuple[int, ...]]:
    return dict(x=(batch, seq, d_model), ln1_g=(d_model,), ln1_b=(d_model,), w_qkv=(d_model, 3 * d_model),
                b_qkv=(3 * d_model,), w_o=(d_model, d_model), b_o=(d_model,), ln2_g=(d_model,), ln2_b=(d_model,),
                w_fc1=(d_model, d_ff), b_fc1=(d_ff,), w_fc2=(d_ff, d_model), b_fc2=(d_model,))


def gpt2BlockProgram(batch: int, seq: int, d_model: int, heads: int, d_ff: int, dtype: DType = DType.Float16,
                     fusedAttention: bool = False) -> JitProgram:
    """Pre-LayerNorm transformer block forward under one jit: LayerNorm (standardize * g + b), fused QKV
    projection with bias, causal softmax attention, output projection + residual, LayerNorm, tanh-GELU MLP +
    residual.  Inputs in order: x, then GPT2_BLOCK_PARAMS (weights stored [in, out]).  `fusedAttention` traces
    the attention chain as the backend's `Attention` routine instead of the reference's seven kernels."""
    H = d_model // heads
    shapes = gpt2BlockShapes(batch, seq, d_model, d_ff)

    def f(x, ln1_g, ln1_b, w_qkv, b_qkv, w_o, b_o, ln2_g, ln2_b, w_fc1, b_fc1, w_fc2, b_fc2):
        h = L.standardize(x).mul(ln1_g).add(ln1_b)
        qkv = L.matmul(h, w_qkv).add(b_qkv)
        full = [(0, batch), (0, seq)]
        q, k, v = (J.shrink(qkv, full + [(i * d_model, (i + 1) * d_model)]).reshape([batch, seq, heads, H]) for i in range(3))
        a = L.dotProductAttention(q, k, v, isCausal=True, fused=fusedAttention).reshape([batch, seq, d_model])
        x = x.add(L.matmul(a, w_o).add(b_o))
        h = L.standardize(x).mul(ln2_g).add(ln2_b)
        m = L.gelu(L.matmul(h, w_fc1).add(b_fc1))
        return x.add(L.matmul(m, w_fc2).add(b_fc2))

    avals = [ShapedArray(shapes["x"], dtype)] + [ShapedArray(shapes[n], dtype) for n in GPT2_BLOCK_PARAMS]
    return J.jit(f, avals)
