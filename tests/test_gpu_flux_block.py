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
