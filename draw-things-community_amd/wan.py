"""Wan 2.x attention block built from the library's entry points.

Mirrors `WanAttentionBlock` (Models/Wan.swift:68-277) for the configuration the hot path is quoted on: batch 1, no
causal inference, no injected image, attention level `.scale1` for the self-attention (Q and K each scaled by
k^(-1/4), attention scale 1) and 1 / sqrt(k) for the cross-attention.  Fourteen launches:

  1  LayerNorm + fp32 modulation                                   (dt_layernorm_modulate_f16, DT_MOD_F32)
  1  x_q x_k x_v                                                   (dt_dense_qx_f16)
  2  whole-row RMSNorm, RoPE and the k^(-1/4) scale on Q and K      (dt_qk_norm_rope_f16)
  1  self-attention                                                (dt_sdpa_f16)
  1  x_o with the fp32 gate and residual in the epilogue           (dt_dense_qx_post_f16)
  1  affine LayerNorm (x_norm_3)                                   (dt_layernorm_modulate_f16, DT_MOD_AFFINE_F32)
  1  x_c_q, 1 whole-row RMSNorm, 1 cross-attention over the fixed context K / V
  1  c_o with the residual in the epilogue
  1  LayerNorm + fp32 modulation
  1  x_linear1 with GELU(tanh), 1 x_out_proj with the fp32 gate and residual
"""
from typing import Dict, Sequence

import numpy as np

from . import (ACT_GELU_TANH, DensePost, QxTensor, _side_stream, dense_multi, dense_post, layernorm_modulate,
               qk_norm_rope_, sdpa_segments, _torch)

DENSE_NAMES = ("x_q", "x_k", "x_v", "x_o", "x_c_q", "c_o", "x_linear1", "x_out_proj")
ROW_NORM_NAMES = ("x_norm_q", "x_norm_k", "x_c_norm_q")


class WanAttentionBlock:
    """k = head dimension, h = heads, hw = video tokens (batch 1).  `weight[name]` is a QxTensor [out, in], `bias[name]`
    an fp16 vector, `norm[name]` the fp16 whole-row RMSNorm weight [h k], `norm3_weight` / `norm3_bias` the fp32
    affine parameters of x_norm_3, `modulation[i]` the block's six fp32 attn_ada_ln vectors [h k]."""

    def __init__(self, k: int, h: int, hw: int, intermediateSize: int):
        self.k, self.h, self.hw, self.intermediateSize = k, h, hw, intermediateSize
        self.weight: Dict[str, QxTensor] = {}
        self.bias: Dict[str, object] = {}
        self.norm: Dict[str, object] = {}
        self.norm3_weight = None
        self.norm3_bias = None
        self.modulation = None

    def __call__(self, x, rot, c: Sequence[object], cK, cV, stream=None):
        """x [1, hw, h k] fp32; rot [hw, k] fp16; c: the six fp32 time-modulation vectors [h k] added to the block's own
        (`chunks = c + modulations`); cK / cV [1, t, h, k] fp16, the context keys and values the fixed encoder
        produced.  Returns the new x, fp32."""
        torch = _torch()
        k, h, hw = self.k, self.h, self.hw
        C = h * k
        if tuple(x.shape[-2:]) != (hw, C):
            raise ValueError("x does not match the block's token count and width")
        W, Bv, G = self.weight, self.bias, self.norm
        chunks = [ci.reshape(C) + mi.reshape(C) for ci, mi in zip(c, self.modulation)]  # fp32 adds, 6 x [C]
        # the copy that the residual epilogues accumulate into is made on a second stream, beside the self-attention's
        # projections, which read the original
        main = stream if stream is not None else torch.cuda.current_stream(x.device)
        side = _side_stream(x.device)
        x_in = x.reshape(hw, C)
        out = torch.empty_like(x_in)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            out.copy_(x_in)
        f16 = dict(dtype=torch.float16, device=x.device)
        # self-attention
        xn = layernorm_modulate(x_in, chunks[1], chunks[0], 1e-6, stream=stream)
        qkv = torch.empty((hw, 3, h, k), **f16)
        qkv2 = qkv.view(hw, 3 * C)
        dense_multi(xn, [W["x_q"], W["x_k"], W["x_v"]], [Bv["x_q"], Bv["x_k"], Bv["x_v"]],
                    outs=[qkv2[:, i * C:(i + 1) * C] for i in range(3)], stream=stream)
        q4, k4, v4 = (qkv[:, i].unsqueeze(0) for i in range(3))
        quarter = 1.0 / float(np.sqrt(np.sqrt(k)))
        qk_norm_rope_(q4, G["x_norm_q"], 1e-6, False, rot=rot, post_scale=quarter, stream=stream)
        qk_norm_rope_(k4, G["x_norm_k"], 1e-6, False, rot=rot, post_scale=quarter, stream=stream)
        att = sdpa_segments([q4], [k4], [v4], 1.0, stream=stream)
        main.wait_stream(side)
        dense_post(att.view(hw, C), [W["x_o"]], [Bv["x_o"]],
                   [DensePost(gate=chunks[2], residual=out, keep_output=False)], stream=stream)
        # cross-attention
        xn = layernorm_modulate(out, self.norm3_weight, self.norm3_bias, 1e-6, stream=stream, affine=True)
        cq = dense_multi(xn, [W["x_c_q"]], [Bv["x_c_q"]], stream=stream)[0].view(1, hw, h, k)
        qk_norm_rope_(cq, G["x_c_norm_q"], 1e-6, False, stream=stream)
        cross = sdpa_segments([cq], [cK], [cV], 1.0 / float(np.sqrt(k)), stream=stream)
        dense_post(cross.view(hw, C), [W["c_o"]], [Bv["c_o"]], [DensePost(residual=out, keep_output=False)],
                   stream=stream)
        # feed-forward
        xn = layernorm_modulate(out, chunks[4], chunks[3], 1e-6, stream=stream)
        hid = dense_post(xn, [W["x_linear1"]], [Bv["x_linear1"]], [DensePost(ACT_GELU_TANH)], stream=stream)[0]
        dense_post(hid, [W["x_out_proj"]], [Bv["x_out_proj"]],
                   [DensePost(gate=chunks[5], residual=out, keep_output=False)], stream=stream)
        return out.reshape(x.shape)
