"""GPU parity: a whole Flux.1 joint transformer block composed from the library's entry points against the oracle's
op-by-op restatement of Models/Flux1.swift:149-290.

Bar: the fp32 output streams within max-abs 2e-2 and rel-RMS 2e-3 of the oracle (the Dense bar, twice its rel-RMS: the
block chains four Dense layers and an attention per stream, every intermediate rounded to fp16 on both sides)."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def build_block(dthip, oracle, rng, k, h, t, hw, q, nib):
    import torch
    flux1 = importlib.import_module(dthip.__name__ + ".flux1")
    C = h * k
    blk = flux1.JointTransformerBlock(k, h, t, hw)
    dense, bias, norm = {}, {}, {}
    for name in flux1.DENSE_NAMES:
        N, K = (4 * C, C) if name.endswith("linear1") else (C, 4 * C) if name.endswith("out_proj") else (C, C)
        packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 1.0 / np.sqrt(K))
        b = (rng.standard_normal(N) * 0.05).astype(np.float16)
        blk.weight[name] = dthip.QxTensor.from_packed(packed, q, nib, (N, K))
        blk.bias[name] = torch.from_numpy(b).cuda()
        bias[name] = b
        dense[name] = (lambda p, n, bb: (lambda X: oracle.C.dense_qx(X, p, q, nib, n, bb)))(packed, N, b)
    for name in flux1.NORM_NAMES:
        g = (1 + 0.05 * rng.standard_normal(k)).astype(np.float16)
        blk.norm[name] = torch.from_numpy(g).cuda()
        norm[name] = g
    return blk, dense, bias, norm


@pytest.mark.parametrize("h,t,gh,gw,q,nib", [(2, 128, 32, 32, 6, 4096), (1, 48, 12, 16, 4, 512)])
def test_flux_joint_block_vs_oracle(dthip, oracle, h, t, gh, gw, q, nib):
    import torch
    k = 128
    hw = gh * gw
    C = h * k
    rng = np.random.default_rng(h * 100 + t)
    blk, dense, bias, norm = build_block(dthip, oracle, rng, k, h, t, hw, q, nib)
    rot = dthip.Flux1RotaryPositionEmbedding(gh, gw, t, channels=k).astype(np.float16)
    assert rot.shape == (t + hw, k)
    context = rng.standard_normal((1, t, C)).astype(np.float32) * 2
    x = rng.standard_normal((1, hw, C)).astype(np.float32) * 2
    mk = lambda: [(rng.standard_normal(C) * s + o).astype(np.float16)
                  for s, o in ((0.3, 0), (0.2, 1), (0.3, 0), (0.3, 0), (0.2, 1), (0.3, 0))]
    cch, xch = mk(), mk()
    dev = lambda a: torch.from_numpy(a).cuda()
    print("flux joint block", h, t, hw, q, nib, flush=True)
    got_c, got_x = blk(dev(context), dev(x), dev(rot), [dev(v) for v in cch], [dev(v) for v in xch])
    want_c, want_x = oracle.np_flux_joint_block(context[0], x[0], rot, cch, xch, dense, bias, norm, k, h)
    for name, got, want in (("context", got_c, want_c), ("x", got_x, want_x)):
        g = got.cpu().numpy().reshape(want.shape)
        mx, rr = oracle.err_stats(g, want)
        print(name, "max-abs", mx, "rel-rms", rr, "scale", float(np.abs(want).max()), flush=True)
        assert mx <= 2e-2 and rr <= 2e-3
    # the inputs are left untouched and a second call gives the same result
    again_c, again_x = blk(dev(context), dev(x), dev(rot), [dev(v) for v in cch], [dev(v) for v in xch])
    assert torch.equal(again_c, got_c) and torch.equal(again_x, got_x)


@pytest.mark.parametrize("h,gt,gh,gw,t,q,nib", [(2, 3, 16, 24, 64, 5, 1024), (1, 2, 6, 10, 40, 6, 64)])
def test_wan_attention_block_vs_oracle(dthip, oracle, h, gt, gh, gw, t, q, nib):
    """A whole Wan attention block (self-attention with whole-row RMSNorm, RoPE and the .scale1 convention,
    cross-attention over fixed context K / V, feed-forward; fp32 modulation and fp32 gates) against the oracle's
    op-by-op restatement of Models/Wan.swift:68-277.  Same bar as the Flux block."""
    import torch
    wan = importlib.import_module(dthip.__name__ + ".wan")
    k = 128
    hw, C = gt * gh * gw, h * k
    inter = 3 * C
    rng = np.random.default_rng(hw + t)
    blk = wan.WanAttentionBlock(k, h, hw, inter)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    dense, norm = {}, {}
    for name in wan.DENSE_NAMES:
        N, K = (inter, C) if name == "x_linear1" else (C, inter) if name == "x_out_proj" else (C, C)
        packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 1.0 / np.sqrt(K))
        b = (rng.standard_normal(N) * 0.05).astype(np.float16)
        blk.weight[name] = dthip.QxTensor.from_packed(packed, q, nib, (N, K))
        blk.bias[name] = dev(b)
        dense[name] = (lambda p, n, bb: (lambda X: oracle.C.dense_qx(X, p, q, nib, n, bb)))(packed, N, b)
    for name in wan.ROW_NORM_NAMES:
        g = (1 + 0.05 * rng.standard_normal(C)).astype(np.float16)
        blk.norm[name] = dev(g)
        norm[name] = g
    n3w = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    n3b = (0.1 * rng.standard_normal(C)).astype(np.float32)
    blk.norm3_weight, blk.norm3_bias = dev(n3w), dev(n3b)
    mods = [(0.2 * rng.standard_normal(C)).astype(np.float32) for _ in range(6)]
    cs = [(0.2 * rng.standard_normal(C)).astype(np.float32) for _ in range(6)]
    blk.modulation = [dev(m) for m in mods]
    rot = dthip.WanRotaryPositionEmbedding(gh, gw, gt, channels=k).astype(np.float16)
    assert rot.shape == (hw, k)
    x = (rng.standard_normal((1, hw, C)) * 2).astype(np.float32)
    cK = rng.standard_normal((1, t, h, k)).astype(np.float16)
    cV = rng.standard_normal((1, t, h, k)).astype(np.float16)
    print("wan block", h, hw, t, q, nib, flush=True)
    got = blk(dev(x), dev(rot), [dev(c) for c in cs], dev(cK), dev(cV)).cpu().numpy()[0]
    chunks = [c + m for c, m in zip(cs, mods)]
    want = oracle.np_wan_attention_block(x[0], rot, chunks, cK, cV, dense, norm, n3w, n3b, k, h)
    mx, rr = oracle.err_stats(got, want)
    print("x max-abs", mx, "rel-rms", rr, "scale", float(np.abs(want).max()), flush=True)
    assert mx <= 2e-2 and rr <= 2e-3


@pytest.mark.parametrize("h,t,gh,gw,q,nib", [(2, 128, 30, 30, 6, 4096), (1, 20, 10, 12, 5, 1024)])
def test_flux_single_block_vs_oracle(dthip, oracle, h, t, gh, gw, q, nib):
    """A Flux.1 single-stream block (attention and feed-forward in parallel, summed in fp16, one gate) against the
    oracle's op-by-op restatement of Models/Flux1.swift:367-492.  Same bar as the joint block."""
    import torch
    flux1 = importlib.import_module(dthip.__name__ + ".flux1")
    k = 128
    S, C = t + gh * gw, h * k
    rng = np.random.default_rng(S)
    blk = flux1.SingleTransformerBlock(k, h, S)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    dense, norm = {}, {}
    for name in flux1.SINGLE_DENSE_NAMES:
        N, K = (4 * C, C) if name == "x_linear1" else (C, 4 * C) if name == "x_out_proj" else (C, C)
        packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 1.0 / np.sqrt(K))
        b = None if name == "x_o" else (rng.standard_normal(N) * 0.05).astype(np.float16)
        blk.weight[name] = dthip.QxTensor.from_packed(packed, q, nib, (N, K))
        blk.bias[name] = None if b is None else dev(b)
        dense[name] = (lambda p, n, bb: (lambda X: oracle.C.dense_qx(X, p, q, nib, n, bb)))(packed, N, b)
    for name in flux1.SINGLE_NORM_NAMES:
        g = (1 + 0.05 * rng.standard_normal(k)).astype(np.float16)
        blk.norm[name] = dev(g)
        norm[name] = g
    rot = dthip.Flux1RotaryPositionEmbedding(gh, gw, t, channels=k).astype(np.float16)
    x = (rng.standard_normal((1, S, C)) * 2).astype(np.float32)
    xch = [(rng.standard_normal(C) * s + o).astype(np.float16) for s, o in ((0.3, 0), (0.2, 1), (0.3, 0))]
    print("flux single block", h, S, q, nib, flush=True)
    got = blk(dev(x), dev(rot), [dev(v) for v in xch]).cpu().numpy()[0]
    want = oracle.np_flux_single_block(x[0], rot, xch, dense, norm, k, h)
    mx, rr = oracle.err_stats(got, want)
    print("x max-abs", mx, "rel-rms", rr, "scale", float(np.abs(want).max()), flush=True)
    assert mx <= 2e-2 and rr <= 2e-3


def test_joint_block_replays_as_hip_graph(dthip, oracle):
    """The twelve launches of a whole joint block (LayerNorm-modulate, grouped Dense with head epilogues and with
    elementwise tails, attention) captured as one HIP graph: every replay, with eager runs and synchronisations in
    between, reproduces the eager result bit for bit."""
    import torch
    k, h, t, gh, gw = 128, 2, 128, 32, 32
    hw, C = gh * gw, h * k
    rng = np.random.default_rng(91)
    blk, _, _, _ = build_block(dthip, oracle, rng, k, h, t, hw, 6, 4096)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    rot = dev(dthip.Flux1RotaryPositionEmbedding(gh, gw, t, channels=k).astype(np.float16))
    context = dev(rng.standard_normal((1, t, C)).astype(np.float32))
    x = dev(rng.standard_normal((1, hw, C)).astype(np.float32))
    mk = lambda: [dev((rng.standard_normal(C) * 0.3 + o).astype(np.float16)) for o in (0, 1, 0, 0, 1, 0)]
    cch, xch = mk(), mk()
    print("joint block as hip graph", flush=True)
    want_c, want_x = blk(context, x, rot, cch, xch)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        blk(context, x, rot, cch, xch)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got_c, got_x = blk(context, x, rot, cch, xch)
    for _ in range(3):
        got_c.zero_(); got_x.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got_c, want_c) and torch.equal(got_x, want_x)
        again_c, again_x = blk(context, x, rot, cch, xch)  # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(again_c, want_c) and torch.equal(again_x, want_x)


@pytest.mark.parametrize("k,h,b,gs,t,cw,q", [(40, 8, 2, 32, 77, 768, 6), (64, 2, 1, 7, 10, 96, 16)])
def test_unet_transformer_block_vs_oracle(dthip, oracle, k, h, b, gs, t, cw, q):
    """A whole SD 1.5 transformer block (fp16 stream: affine LayerNorms, self- and cross-attention with head dimension
    40, the erf-GELU gated feed-forward, fp16 residual additions in the Dense epilogues) against the oracle's
    op-by-op restatement of Models/UNet.swift:519-565.  q = 16: plain fp16 weights."""
    import torch
    unet = importlib.import_module(dthip.__name__ + ".unet")
    hw, C = gs * gs, h * k
    inter = 4 * C
    rng = np.random.default_rng(C + hw)
    blk = unet.BasicTransformerBlock(k, h, b, hw, t)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    dense, norm = {}, {}
    for name in unet.DENSE_NAMES:
        K = cw if name in ("tokeys2", "tovalues2") else inter if name == "fc2" else C
        N = inter if name in ("fc10", "fc11") else C
        bias = None if name in unet.NO_BIAS else (rng.standard_normal(N) * 0.05).astype(np.float16)
        if q == 16:
            Wh = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float16)
            blk.weight[name] = dthip.QxTensor.from_f16(Wh)
            dense[name] = (lambda w_, bb: (lambda X: oracle.C.dense(np.ascontiguousarray(X), w_, bb)))(Wh, bias)
        else:
            packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, 4096, 1.0 / np.sqrt(K))
            blk.weight[name] = dthip.QxTensor.from_packed(packed, q, 4096, (N, K))
            dense[name] = (lambda p, n, bb: (lambda X: oracle.C.dense_qx(np.ascontiguousarray(X), p, q, 4096, n, bb)))(packed, N, bias)
        if bias is not None:
            blk.bias[name] = dev(bias)
    for name in unet.NORM_NAMES:
        g = (1 + 0.1 * rng.standard_normal(C)).astype(np.float16)
        bb = (0.1 * rng.standard_normal(C)).astype(np.float16)
        blk.norm[name] = (dev(g), dev(bb))
        norm[name] = (g, bb)
    x = rng.standard_normal((b, hw, C)).astype(np.float16)
    c = rng.standard_normal((b, t, cw)).astype(np.float16)
    print("unet block", k, h, b, hw, t, q, flush=True)
    got = blk(dev(x), dev(c)).cpu().numpy()
    want = oracle.np_unet_transformer_block(x, c, dense, norm, k, h)
    mx, rr = oracle.err_stats(got, want)
    print("x max-abs", mx, "rel-rms", rr, "scale", float(np.abs(want.astype(np.float32)).max()), flush=True)
    assert mx <= 2e-2 and rr <= 2e-3



def test_flux_step_full_size_sampled(dthip, oracle):
    """The benchmark's own step at full size -- 512 text + 4096 image tokens, 24 heads x 128, q6p (nib 4096) -- as
    the exact three calls the benchmark makes: the grouped QKV launch (image and context problems, per-head RMSNorm
    + RoPE in the epilogue, rot_pos0 512 / 0) writing one strided [S, 3, H, D] buffer; attention reading Q, K, V as
    strided views of that buffer; the grouped output projections.  Sampled token rows (0, 511, 512 and 4607 among
    them) against the oracle's op-by-op chain Dense -> RMSNorm -> cmul -> attention -> Dense
    (Models/Flux1.swift:161-245) at the block bar."""
    import torch

    T, gh, gw, H, D, q, nib = 512, 64, 64, 24, 128, 6, 4096
    HW, C = gh * gw, H * D
    S = T + HW
    rng = np.random.default_rng(4608)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    f16 = lambda a: np.asarray(a, dtype=np.float16)
    packs, w, bias = {}, {}, {}
    for name in ("c_q", "c_k", "c_v", "x_q", "x_k", "x_v", "c_o", "x_o"):
        packs[name], _, _ = oracle.synth_qx_weight(rng, C, C, q, nib)
        w[name] = dthip.QxTensor.from_packed(packs[name], q, nib, (C, C))
        bias[name] = f16(rng.standard_normal(C) * 0.02)
    gam = {n: f16(1 + 0.02 * rng.standard_normal(D)) for n in ("c_q", "c_k", "x_q", "x_k")}
    rot = f16(dthip.Flux1RotaryPositionEmbedding(gh, gw, T, channels=D))
    ctx, img = f16(rng.standard_normal((T, C))), f16(rng.standard_normal((HW, C)))
    scale = 1.0 / float(np.sqrt(D))

    # ---- the benchmark's three calls
    qkv = torch.full((S, 3, H, D), float("nan"), dtype=torch.float16, device="cuda")
    att = torch.full((1, S, H, D), float("nan"), dtype=torch.float16, device="cuda")
    out_c = torch.full((T, C), float("nan"), dtype=torch.float16, device="cuda")
    out_x = torch.full((HW, C), float("nan"), dtype=torch.float16, device="cuda")
    qkv2 = qkv.view(S, 3 * C)
    views = lambda lo, hi: [qkv2[lo:hi, i * C:(i + 1) * C] for i in range(3)]
    d_rot = dev(rot)
    epi = lambda s, pos0: [dthip.HeadEpilogue(dev(gam[s + "_q"]), d_rot, pos0, 1e-6, D),
                           dthip.HeadEpilogue(dev(gam[s + "_k"]), d_rot, pos0, 1e-6, D), None]
    d_ctx, d_img = dev(ctx), dev(img)
    d_bias = {n: dev(b) for n, b in bias.items()}
    print("flux step at full size: grouped QKV", flush=True)
    dthip.dense_grouped([
        dict(x=d_img, weights=[w["x_q"], w["x_k"], w["x_v"]], biases=[d_bias["x_q"], d_bias["x_k"], d_bias["x_v"]],
             outs=views(T, S), epilogues=epi("x", T)),
        dict(x=d_ctx, weights=[w["c_q"], w["c_k"], w["c_v"]], biases=[d_bias["c_q"], d_bias["c_k"], d_bias["c_v"]],
             outs=views(0, T), epilogues=epi("c", 0))])
    print("flux step at full size: attention on strided views", flush=True)
    q4, k4, v4 = (qkv[:, i].unsqueeze(0) for i in range(3))
    dthip.sdpa_segments([q4], [k4], [v4], scale, out=att)
    print("flux step at full size: grouped out-projections", flush=True)
    att2 = att.view(S, C)
    dthip.dense_grouped([dict(x=att2[T:], weights=[w["x_o"]], biases=[d_bias["x_o"]], outs=[out_x]),
                         dict(x=att2[:T], weights=[w["c_o"]], biases=[d_bias["c_o"]], outs=[out_c])])
    torch.cuda.synchronize()
    got_qkv, got_att = qkv.cpu().numpy(), att.cpu().numpy()[0]
    got_out = np.concatenate([out_c.cpu().numpy(), out_x.cpu().numpy()])
    assert np.isfinite(got_qkv.astype(np.float32)).all() and np.isfinite(got_out.astype(np.float32)).all()

    # ---- the oracle: K and V for every token, Q / attention / output for the sampled rows
    rows = np.sort(np.unique(np.concatenate([[0, 255, 256, T - 1, T, T + 255, T + 256, S - 257, S - 256, S - 1],
                                             rng.choice(S, size=14, replace=False)])))
    x_all = np.concatenate([ctx, img])
    heads = lambda a: a.reshape(-1, H, D)

    def proj(n, sel=None):
        """Dense of stream-specific weights over the joint sequence's rows (all, or the selected ones)."""
        idx = np.arange(S) if sel is None else sel
        out = np.empty((idx.size, C), dtype=np.float16)
        for s, lo, hi in (("c", 0, T), ("x", T, S)):
            m = (idx >= lo) & (idx < hi)
            if m.any():
                out[m] = oracle.C.dense_qx(np.ascontiguousarray(x_all[idx[m]]), packs[f"{s}_{n}"], q, nib, C, bias[f"{s}_{n}"])
        return out

    def norm_rot(y, n, idx):
        out = np.empty((idx.size, H, D), dtype=np.float16)
        for s, lo, hi in (("c", 0, T), ("x", T, S)):
            m = (idx >= lo) & (idx < hi)
            if m.any():
                out[m] = oracle.C.cmul(oracle.C.rmsnorm(heads(y[m]), gam[f"{s}_{n}"], 1e-6), rot[idx[m]])
        return out

    all_rows = np.arange(S)
    want_k = norm_rot(proj("k"), "k", all_rows)
    want_v = heads(proj("v"))
    want_q = norm_rot(proj("q", rows), "q", rows)
    # the projections with their fused epilogue, where they landed in the strided buffer
    for name, g, wnt in (("q", got_qkv[rows, 0], want_q), ("k", got_qkv[:, 1], want_k), ("v", got_qkv[:, 2], want_v)):
        mx, rr = oracle.err_stats(g, wnt)
        print("qkv", name, "max-abs", mx, "rel-rms", rr, flush=True)
        assert mx <= 2e-2 and rr <= 1e-3, (name, mx, rr)
    want_att = oracle.C.sdpa(want_q[None], want_k[None], want_v[None], scale)[0]
    mx, rr = oracle.err_stats(got_att[rows], want_att)
    print("attention max-abs", mx, "rel-rms", rr, flush=True)
    assert mx <= 2e-2 and rr <= 1e-3, (mx, rr)
    want_out = np.empty((rows.size, C), dtype=np.float16)
    for s, lo, hi in (("c", 0, T), ("x", T, S)):
        m = (rows >= lo) & (rows < hi)
        want_out[m] = oracle.C.dense_qx(np.ascontiguousarray(want_att[m].reshape(-1, C)), packs[f"{s}_o"], q, nib, C,
                                        bias[f"{s}_o"])
    mx, rr = oracle.err_stats(got_out[rows], want_out)
    print("out max-abs", mx, "rel-rms", rr, flush=True)
    assert mx <= 2e-2 and rr <= 2e-3, (mx, rr)


def test_four_host_threads_on_four_streams(dthip, oracle):
    """The reference runs a model on up to four concurrent streams (maxConcurrency = .limit(4),
    Models/UNetProtocol.swift:2011).  Four host threads, each with a stream and inputs of its own, run the same
    chain -- palettized QKV projection with the fused head epilogue, attention (one thread's launch small enough to
    be key-split, each call with a workspace of its own), output projection -- several times over at once; every
    thread's result must equal, bit for bit, what the same chain gives when it runs alone."""
    import threading

    import torch

    H, D, q, nib = 4, 128, 6, 4096
    C = H * D
    rng = np.random.default_rng(2011)
    f16 = lambda a: np.asarray(a, dtype=np.float16)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    ws = {}
    for name in ("q", "k", "v", "o"):
        packed, _, _ = oracle.synth_qx_weight(rng, C, C, q, nib)
        ws[name] = dthip.QxTensor.from_packed(packed, q, nib, (C, C))
    gam = dev(f16(1 + 0.02 * rng.standard_normal(D)))
    sizes = [1300, 900, 4096, 700]  # (4 heads x 4096 tokens is split along the keys by the library's own estimate)
    assert dthip.lib().dt_sdpa_workspace_bytes(1, H, H, D, 4096, 4096, 0, 0) > 0
    rots = [dev(f16(dthip.WanRotaryPositionEmbedding(1, S, 1, channels=D))) for S in sizes]
    xs = [dev(f16(rng.standard_normal((S, C)))) for S in sizes]

    def chain(i, stream):
        S = sizes[i]
        epi = [dthip.HeadEpilogue(gam, rots[i], 0, 1e-6, D), dthip.HeadEpilogue(gam, rots[i], 0, 1e-6, D), None]
        qo, ko, vo = dthip.dense_multi(xs[i], [ws["q"], ws["k"], ws["v"]], [None] * 3, epilogues=epi, stream=stream)
        att = dthip.sdpa_segments([qo.view(1, S, H, D)], [ko.view(1, S, H, D)], [vo.view(1, S, H, D)], 1 / np.sqrt(D),
                                  stream=stream)
        return dthip.dense_multi(att.view(S, C), [ws["o"]], [None], stream=stream)[0]

    torch.cuda.synchronize()
    alone = []
    for i in range(4):
        alone.append(chain(i, None))
        torch.cuda.synchronize()
    results, errors = [None] * 4, []

    def worker(i):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            out = None
            for _ in range(6):
                out = chain(i, stream)
            stream.synchronize()
            results[i] = out
        except Exception as e:  # surfaces in the main thread below
            errors.append((i, repr(e)))

    print("four threads, four streams", flush=True)
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i in range(4):
        assert torch.equal(results[i], alone[i]), i
    # and the chain itself is right: one thread's result against the oracle
    i, S = 1, sizes[1]
    x = xs[i].cpu().numpy()
    heads = lambda a: a.reshape(S, H, D)
    pk = {n: oracle.C.depalettize(q, nib, C * C, ws[n].data.cpu().numpy()[: dthip.qx_bytes(q, nib, C * C)]).reshape(C, C) for n in ws}
    g, r = gam.cpu().numpy(), rots[i].cpu().numpy()
    rq = oracle.C.cmul(oracle.C.rmsnorm(heads(oracle.C.dense(x, pk["q"], None)), g, 1e-6), r)
    rk = oracle.C.cmul(oracle.C.rmsnorm(heads(oracle.C.dense(x, pk["k"], None)), g, 1e-6), r)
    rv = heads(oracle.C.dense(x, pk["v"], None))
    att = oracle.C.sdpa(rq[None], rk[None], rv[None], 1 / np.sqrt(D)).reshape(S, C)
    want = oracle.C.dense(att, pk["o"], None)
    mx, rr = oracle.err_stats(results[i].cpu().numpy(), want)
    assert mx <= 2e-2 and rr <= 2e-3, (mx, rr)
