"""Flux.1 joint (double-stream) transformer block built from the library's entry points.

Mirrors `JointTransformerBlock` (Models/Flux1.swift:149-290) for the configuration the hot path is quoted on:
`contextBlockPreOnly: false`, `upcast: false`, attention level `.scaleMerged`.  The reference graph runs about fifty ops
per block; here a block is twelve launches:

  2  LayerNorm + modulation of the two fp32 streams                       (dt_layernorm_modulate_f16)
  1  c_q c_k c_v x_q x_k x_v with per-head RMSNorm and RoPE in the epilogue, written straight into the joint
     [t + hw, 3, h, k] buffer (no concat)                                   (dt_dense_qx_grouped_f16)
  1  attention over the joint sequence                                      (dt_sdpa_f16)
  1  c_o and x_o with gate and fp32 residual accumulation in the epilogue  (dt_dense_qx_grouped_f16 + post)
  2  LayerNorm + modulation
  1  c_linear1 and x_linear1 with GELU(tanh)
  1  c_out_proj and x_out_proj with gate and residual accumulation
"""
from typing import Dict, Optional, Sequence

import numpy as np

from . import (ACT_GELU_TANH, DensePost, HeadEpilogue, QxTensor, _side_stream, dense_grouped, dense_multi, dense_post,
               layernorm_modulate, sdpa_segments, _torch)

DENSE_NAMES = ("c_q", "c_k", "c_v", "x_q", "x_k", "x_v", "c_o", "x_o", "c_linear1", "c_out_proj", "x_linear1",
               "x_out_proj")
NORM_NAMES = ("c_norm_q", "c_norm_k", "x_norm_q", "x_norm_k")


class JointTransformerBlock:
    """k = head dimension, h = heads, t = text tokens, hw = image tokens (batch 1).  `weight[name]` is a QxTensor
    [out, in], `bias[name]` an fp16 vector, `norm[name]` the fp16 RMSNorm weight [k]."""

    def __init__(self, k: int, h: int, t: int, hw: int):
        self.k, self.h, self.t, self.hw = k, h, t, hw
        self.weight: Dict[str, QxTensor] = {}
        self.bias: Dict[str, object] = {}
        self.norm: Dict[str, object] = {}
        self._buffers = None

    def _alloc(self, device):
        torch = _torch()
        if self._buffers is None or self._buffers["qkv"].device != device:
            S, C = self.t + self.hw, self.h * self.k
            f16 = dict(dtype=torch.float16, device=device)
            self._buffers = dict(
                qkv=torch.empty((S, 3, self.h, self.k), **f16), att=torch.empty((1, S, self.h, self.k), **f16),
                cn=torch.empty((self.t, C), **f16), xn=torch.empty((self.hw, C), **f16),
                ch=torch.empty((self.t, 4 * C), **f16), xh=torch.empty((self.hw, 4 * C), **f16))
        return self._buffers

    def __call__(self, context, x, rot, contextChunks: Sequence[object], xChunks: Sequence[object], stream=None):
        """context [1, t, h k] and x [1, hw, h k] fp32, rot [t + hw, k] fp16 (interleaved cos / sin), the six
        modulation vectors of each stream fp16 [h k] (shift, scale, gate for attention, then for the feed-forward;
        the scale already carries its + 1, as the fixed encoder stores it).  Returns the new (context, x), fp32."""
        torch = _torch()
        k, h, t, hw = self.k, self.h, self.t, self.hw
        S, C = t + hw, h * k
        if tuple(context.shape[-2:]) != (t, C) or tuple(x.shape[-2:]) != (hw, C):
            raise ValueError("context / x do not match the block's token counts and width")
        if len(contextChunks) != 6 or len(xChunks) != 6:
            raise ValueError("six modulation vectors per stream")
        W, Bv, G = self.weight, self.bias, self.norm
        buf = self._alloc(x.device)
        qkv, att, cn, xn = buf["qkv"], buf["att"], buf["cn"], buf["xn"]
        # The block returns new streams, so the residual epilogues accumulate into copies.  The copies are made on a
        # second stream beside the attention half's launches, which read the originals; the context stream's
        # LayerNorm launches (short, independent of the image stream's) go there too.
        main = stream if stream is not None else torch.cuda.current_stream(x.device)
        side = _side_stream(x.device)
        c_in, x_in = context.reshape(t, C), x.reshape(hw, C)
        c_res, x_res = torch.empty_like(c_in), torch.empty_like(x_in)
        side.wait_stream(main)
        # attention half
        layernorm_modulate(c_in, contextChunks[1], contextChunks[0], 1e-6, out=cn, stream=side)
        context_normed = side.record_event()
        with torch.cuda.stream(side):
            c_res.copy_(c_in)
            x_res.copy_(x_in)
        copied = side.record_event()
        layernorm_modulate(x_in, xChunks[1], xChunks[0], 1e-6, out=xn, stream=main)
        main.wait_event(context_normed)
        qkv2 = qkv.view(S, 3 * C)
        views = lambda lo, hi: [qkv2[lo:hi, i * C:(i + 1) * C] for i in range(3)]
        epi = lambda q, kk, pos: [HeadEpilogue(G[q], rot, pos, 1e-6, k), HeadEpilogue(G[kk], rot, pos, 1e-6, k), None]
        dense_grouped([
            dict(x=xn, weights=[W["x_q"], W["x_k"], W["x_v"]], biases=[Bv["x_q"], Bv["x_k"], Bv["x_v"]],
                 outs=views(t, S), epilogues=epi("x_norm_q", "x_norm_k", t)),
            dict(x=cn, weights=[W["c_q"], W["c_k"], W["c_v"]], biases=[Bv["c_q"], Bv["c_k"], Bv["c_v"]],
                 outs=views(0, t), epilogues=epi("c_norm_q", "c_norm_k", 0))], stream=stream)
        sdpa_segments([qkv[:, 0].unsqueeze(0)], [qkv[:, 1].unsqueeze(0)], [qkv[:, 2].unsqueeze(0)],
                      1.0 / float(np.sqrt(k)), out=att, stream=stream)
        att2 = att.view(S, C)
        main.wait_event(copied)
        tail = lambda gate, res: [DensePost(gate=gate, residual=res, keep_output=False)]
        dense_grouped([
            dict(x=att2[t:], weights=[W["x_o"]], biases=[Bv["x_o"]], posts=tail(xChunks[2], x_res)),
            dict(x=att2[:t], weights=[W["c_o"]], biases=[Bv["c_o"]], posts=tail(contextChunks[2], c_res))],
            stream=stream)
        # feed-forward half
        side.wait_stream(main)
        layernorm_modulate(c_res, contextChunks[4], contextChunks[3], 1e-6, out=cn, stream=side)
        layernorm_modulate(x_res, xChunks[4], xChunks[3], 1e-6, out=xn, stream=main)
        main.wait_stream(side)
        gelu = [DensePost(ACT_GELU_TANH)]
        dense_grouped([
            dict(x=xn, weights=[W["x_linear1"]], biases=[Bv["x_linear1"]], outs=[buf["xh"]], posts=gelu),
            dict(x=cn, weights=[W["c_linear1"]], biases=[Bv["c_linear1"]], outs=[buf["ch"]], posts=gelu)],
            stream=stream)
        dense_grouped([
            dict(x=buf["xh"], weights=[W["x_out_proj"]], biases=[Bv["x_out_proj"]], posts=tail(xChunks[5], x_res)),
            dict(x=buf["ch"], weights=[W["c_out_proj"]], biases=[Bv["c_out_proj"]],
                 posts=tail(contextChunks[5], c_res))], stream=stream)
        return c_res.reshape(context.shape), x_res.reshape(x.shape)


SINGLE_DENSE_NAMES = ("x_q", "x_k", "x_v", "x_o", "x_linear1", "x_out_proj")
SINGLE_NORM_NAMES = ("x_norm_q", "x_norm_k")


class SingleTransformerBlock:
    """Flux.1 single-stream block (Models/Flux1.swift:367-492, `contextBlockPreOnly: false`, `.scaleMerged`): one
    stream of t + hw tokens, attention and feed-forward in parallel on the same modulated input, their fp16 sum gated
    into the fp32 stream.  Six launches: LayerNorm + modulation; x_q x_k x_v with per-head RMSNorm and RoPE in the
    epilogue; attention; x_linear1 with GELU(tanh); x_o (no bias); x_out_proj whose epilogue adds the x_o result,
    applies the gate and accumulates into the residual."""

    def __init__(self, k: int, h: int, tokens: int):
        self.k, self.h, self.tokens = k, h, tokens
        self.weight: Dict[str, QxTensor] = {}
        self.bias: Dict[str, object] = {}
        self.norm: Dict[str, object] = {}

    def __call__(self, x, rot, xChunks: Sequence[object], stream=None):
        """x [1, t + hw, h k] fp32, rot [t + hw, k] fp16, xChunks: shift, scale (with its + 1), gate, fp16 [h k].
        Returns the new x, fp32."""
        torch = _torch()
        k, h, S = self.k, self.h, self.tokens
        C = h * k
        if tuple(x.shape[-2:]) != (S, C) or len(xChunks) != 3:
            raise ValueError("x / xChunks do not match the block")
        W, Bv, G = self.weight, self.bias, self.norm
        # the copy that the last epilogue accumulates into is made on a second stream, beside the launches below
        main = stream if stream is not None else torch.cuda.current_stream(x.device)
        side = _side_stream(x.device)
        x_in = x.reshape(S, C)
        res = torch.empty_like(x_in)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            res.copy_(x_in)
        xn = layernorm_modulate(x_in, xChunks[1], xChunks[0], 1e-6, stream=stream)
        qkv = torch.empty((S, 3, h, k), dtype=torch.float16, device=x.device)
        qkv2 = qkv.view(S, 3 * C)
        dense_multi(xn, [W["x_q"], W["x_k"], W["x_v"]], [Bv["x_q"], Bv["x_k"], Bv["x_v"]],
                    outs=[qkv2[:, i * C:(i + 1) * C] for i in range(3)], stream=stream,
                    epilogues=[HeadEpilogue(G["x_norm_q"], rot, 0, 1e-6, k), HeadEpilogue(G["x_norm_k"], rot, 0, 1e-6, k),
                               None])
        att = sdpa_segments([qkv[:, 0].unsqueeze(0)], [qkv[:, 1].unsqueeze(0)], [qkv[:, 2].unsqueeze(0)],
                            1.0 / float(np.sqrt(k)), stream=stream)
        hid = dense_post(xn, [W["x_linear1"]], [Bv["x_linear1"]], [DensePost(ACT_GELU_TANH)], stream=stream)[0]
        heads = dense_multi(att.view(S, C), [W["x_o"]], [None], stream=stream)[0]
        main.wait_stream(side)
        dense_post(hid, [W["x_out_proj"]], [Bv["x_out_proj"]],
                   [DensePost(gate=xChunks[2], residual=res, keep_output=False, addend=heads)], stream=stream)
        return res.reshape(x.shape)

