"""The transformer block of the SD 1.5 / SDXL UNet built from the library's entry points.

Mirrors `BasicTransformerBlock` (Models/UNet.swift:519-565) with `SelfAttention` (:95-156), `CrossAttention`
(:269-320) and the gated `FeedForward` (:506-517) for the fp16 configuration (`upcastAttention: false`, attention
level `.scaleMerged`, no injected KV, no IP adapters).  Thirteen launches: three fp16 LayerNorms, q / k / v of the
self-attention as one Dense launch, attention, the unify-heads projection with the residual in its epilogue (the
reference fuses that projection into the attention op and adds the residual afterwards: the same arithmetic), the
cross-attention's query projection, its key / value projections of the text context as one launch, attention, unify
heads + residual, then fc11 with GELU, fc10 multiplied by it, fc2 + residual.
"""
from typing import Dict

import numpy as np

from . import (ACT_GELU_ERF, DensePost, QxTensor, dense_multi, dense_post, layernorm16, sdpa_segments, _torch)

DENSE_NAMES = ("tokeys1", "toqueries1", "tovalues1", "unifyheads1", "tokeys2", "toqueries2", "tovalues2", "unifyheads2",
               "fc10", "fc11", "fc2")
NO_BIAS = ("tokeys1", "toqueries1", "tovalues1", "tokeys2", "toqueries2", "tovalues2")
NORM_NAMES = ("layerNorm1", "layerNorm2", "layerNorm3")


class BasicTransformerBlock:
    """k = head dimension, h = heads, b = batch, hw = image tokens, t = text tokens.  `weight[name]`: QxTensor
    [out, in]; `bias[name]`: fp16 vector (absent for the six attention input projections); `norm[name]`: (weight,
    bias) fp16 vectors of a LayerNorm."""

    def __init__(self, k: int, h: int, b: int, hw: int, t: int):
        self.k, self.h, self.b, self.hw, self.t = k, h, b, hw, t
        self.weight: Dict[str, QxTensor] = {}
        self.bias: Dict[str, object] = {}
        self.norm: Dict[str, tuple] = {}

    def __call__(self, x, c, stream=None):
        """x [b, hw, h k] fp16, c [b, t, context width] fp16; returns the new x."""
        k, h, b, hw, t = self.k, self.h, self.b, self.hw, self.t
        C = h * k
        if tuple(x.shape) != (b, hw, C) or tuple(c.shape[:2]) != (b, t):
            raise ValueError("x / c do not match the block")
        W, Bv, N = self.weight, self.bias, self.norm
        scale = 1.0 / float(np.sqrt(k))
        x2 = x.reshape(b * hw, C)
        c2 = c.reshape(b * t, c.shape[-1])
        heads = lambda y, s: y.view(b, s, h, k)
        # self-attention
        n1 = layernorm16(x2, *N["layerNorm1"], 1e-5, stream=stream)
        q, kk, v = dense_multi(n1, [W["toqueries1"], W["tokeys1"], W["tovalues1"]], [None] * 3, stream=stream)
        att = sdpa_segments([heads(q, hw)], [heads(kk, hw)], [heads(v, hw)], scale, stream=stream)
        out = dense_post(att.view(b * hw, C), [W["unifyheads1"]], [Bv["unifyheads1"]], [DensePost(addend=x2)],
                         stream=stream)[0]
        # cross-attention
        n2 = layernorm16(out, *N["layerNorm2"], 1e-5, stream=stream)
        q = dense_multi(n2, [W["toqueries2"]], [None], stream=stream)[0]
        kk, v = dense_multi(c2, [W["tokeys2"], W["tovalues2"]], [None] * 2, stream=stream)
        att = sdpa_segments([heads(q, hw)], [heads(kk, t)], [heads(v, t)], scale, stream=stream)
        out = dense_post(att.view(b * hw, C), [W["unifyheads2"]], [Bv["unifyheads2"]], [DensePost(addend=out)],
                         stream=stream)[0]
        # gated feed-forward
        n3 = layernorm16(out, *N["layerNorm3"], 1e-5, stream=stream)
        g = dense_post(n3, [W["fc11"]], [Bv["fc11"]], [DensePost(ACT_GELU_ERF)], stream=stream)[0]
        hid = dense_post(n3, [W["fc10"]], [Bv["fc10"]], [DensePost(multiplicand=g)], stream=stream)[0]
        out = dense_post(hid, [W["fc2"]], [Bv["fc2"]], [DensePost(addend=out)], stream=stream)[0]
        return out.view(b, hw, C)
