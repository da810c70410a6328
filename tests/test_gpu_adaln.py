"""GPU parity: LayerNorm + adaLN modulation (K4) against the CPU oracle, through the C ABI.

Bar: two fp16 ulps of the result (the fp32 statistics are summed in a different order on the device, and a value that
sits on a rounding boundary after the first of the three roundings carries its flip through the next two)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def close(got, want, shift=None):
    """Two fp16 ulps of the larger of the result and the terms of the final addition (where the modulated value and the
    shift cancel, the result inherits the rounding of the terms, not of its own small magnitude)."""
    w = want.astype(np.float32)
    mag = np.abs(w)
    if shift is not None:
        sh = np.broadcast_to(shift.astype(np.float32), w.shape)
        mag = np.maximum(mag, np.maximum(np.abs(sh), np.abs(w - sh)))
    tol = 2 * np.maximum(np.spacing(mag.astype(np.float16)).astype(np.float32), np.float32(2.0 ** -24))
    return np.all(np.abs(got.astype(np.float32) - w) <= tol)


@pytest.mark.parametrize("M,C", [(7, 256), (300, 3072), (64, 5120), (5, 8192), (9, 1000), (3, 130), (2, 8200), (1, 4)])
@pytest.mark.parametrize("mod", ["f16", "f32", "affine"])
def test_layernorm_modulate_vs_oracle(dthip, oracle, M, C, mod):
    import torch
    rng = np.random.default_rng(M * 31 + C)
    x = (rng.standard_normal((M, C)) * 2 + 0.5).astype(np.float32)
    dt = np.float16 if mod == "f16" else np.float32
    scale = ((0 if mod == "f32" else 1) + 0.3 * rng.standard_normal(C)).astype(dt)
    shift = (0.5 * rng.standard_normal(C)).astype(dt)
    xd, sd, hd = torch.from_numpy(x).cuda(), torch.from_numpy(scale).cuda(), torch.from_numpy(shift).cuda()
    print("adaln", M, C, mod, flush=True)
    aff = mod == "affine"
    got = dthip.layernorm_modulate(xd, sd, hd, 1e-6, affine=aff).cpu().numpy()
    assert close(got, oracle.np_layernorm_modulate16(x, scale, shift, 1e-6, mod), shift)
    # no modulation, scale only, shift only
    assert close(dthip.layernorm_modulate(xd, None, None, 1e-6).cpu().numpy(),
                 oracle.np_layernorm_modulate16(x, None, None, 1e-6, mod))
    assert close(dthip.layernorm_modulate(xd, sd, None, 1e-6, affine=aff).cpu().numpy(),
                 oracle.np_layernorm_modulate16(x, scale, None, 1e-6, mod))
    assert close(dthip.layernorm_modulate(xd, None, hd, 1e-6, affine=aff).cpu().numpy(),
                 oracle.np_layernorm_modulate16(x, None, shift, 1e-6, mod), shift)


def test_layernorm_modulate_views_and_edges(dthip, oracle):
    import torch
    rng = np.random.default_rng(3)
    M, C = 33, 512
    x = rng.standard_normal((M, C)).astype(np.float32)
    scale = (1 + 0.1 * rng.standard_normal(C)).astype(np.float16)
    want = oracle.np_layernorm_modulate16(x, scale, None, 1e-6, "f16")
    # row-strided input and output views, with guard columns that must stay untouched
    big = torch.zeros((M, C + 8), dtype=torch.float32, device="cuda")
    big[:, 4:4 + C].copy_(torch.from_numpy(x))
    out = torch.full((M, C + 16), 7.0, dtype=torch.float16, device="cuda")
    sd = torch.from_numpy(scale).cuda()
    print("adaln views", flush=True)
    dthip.layernorm_modulate(big[:, 4:4 + C], sd, None, 1e-6, out=out[:, 8:8 + C])
    assert close(out[:, 8:8 + C].cpu().numpy(), want)
    assert float((out[:, :8] - 7).abs().max()) == 0 and float((out[:, 8 + C:] - 7).abs().max()) == 0
    # unaligned views (odd column offset) take the any-shape kernel: same results
    out2 = torch.full((M, C + 16), 7.0, dtype=torch.float16, device="cuda")
    big2 = torch.zeros((M, C + 8), dtype=torch.float32, device="cuda")
    big2[:, 3:3 + C].copy_(torch.from_numpy(x))
    dthip.layernorm_modulate(big2[:, 3:3 + C], sd, None, 1e-6, out=out2[:, 5:5 + C])
    assert torch.equal(out2[:, 5:5 + C], out[:, 8:8 + C])
    assert float((out2[:, :5] - 7).abs().max()) == 0 and float((out2[:, 5 + C:] - 7).abs().max()) == 0
    # constant rows normalise to zero: the shift alone comes out; a batch dimension is flattened
    sh = torch.from_numpy(rng.standard_normal(C).astype(np.float16)).cuda()
    const = torch.full((2, 3, C), 4.5, dtype=torch.float32, device="cuda")
    y = dthip.layernorm_modulate(const, None, sh, 1e-6)
    assert y.shape == (2, 3, C) and torch.equal(y, sh.expand(2, 3, C))
    # empty input, bad arguments
    assert dthip.layernorm_modulate(torch.zeros((0, C), dtype=torch.float32, device="cuda")).shape == (0, C)
    with pytest.raises(TypeError):
        dthip.layernorm_modulate(torch.zeros((2, C), dtype=torch.float16, device="cuda"))
    with pytest.raises(TypeError):
        dthip.layernorm_modulate(torch.zeros((2, C), dtype=torch.float32, device="cuda"), sd, sh.float())
    with pytest.raises(ValueError):
        dthip.layernorm_modulate(torch.zeros((2, C), dtype=torch.float32, device="cuda"), sd[:-1])
    with pytest.raises(dthip.DtError):
        dthip.layernorm_modulate(torch.zeros((2, C), dtype=torch.float32, device="cuda"), epsilon=-1.0)
    ln = dthip.LayerNorm(1e-6, [2], elementwiseAffine=False)
    assert close(ln(torch.from_numpy(x).cuda().reshape(3, 11, C)).cpu().numpy().reshape(M, C),
                 oracle.np_layernorm_modulate16(x, None, None, 1e-6, "f16"))


def test_layernorm_modulate_flux_full_size(dthip, oracle):
    """The image stream of the benchmark block (4096 x 3072) and the Wan stream (32760 x 5120): sampled rows against
    the oracle, every row's fp16 statistics against the size-independent property mean = shift-free 0 / variance 1."""
    import torch
    rng = np.random.default_rng(8)
    for M, C, mod in ((4096, 3072, "f16"), (32760, 5120, "f32")):
        print("adaln full", M, C, mod, flush=True)
        x = torch.randn((M, C), dtype=torch.float32, device="cuda") * 3 + 1
        y = dthip.layernorm_modulate(x, None, None, 1e-6).float()
        assert float(y.mean(dim=1).abs().max()) < 2e-3 and float((y.var(dim=1, unbiased=False) - 1).abs().max()) < 5e-3
        rows = rng.choice(M, 16, replace=False)
        dt = np.float16 if mod == "f16" else np.float32
        scale = (0.2 * rng.standard_normal(C)).astype(dt)
        shift = (0.5 * rng.standard_normal(C)).astype(dt)
        got = dthip.layernorm_modulate(x, torch.from_numpy(scale).cuda(), torch.from_numpy(shift).cuda(), 1e-6)
        want = oracle.np_layernorm_modulate16(x[rows].cpu().numpy(), scale, shift, 1e-6, mod)
        assert close(got[rows].cpu().numpy(), want, shift)


@pytest.mark.parametrize("M,C", [(9, 320), (300, 1280), (5, 4096), (7, 100), (3, 4104), (2, 8)])
def test_layernorm16_vs_oracle(dthip, oracle, M, C):
    """LayerNorm with fp16 affine weight and bias on an fp16 tensor (the UNet block's norms): one fp16 ulp of the
    oracle's float64 statement (two where the affine step cancels); strided views; in place."""
    import torch
    rng = np.random.default_rng(M + C)
    x = (rng.standard_normal((M, C)) * 2 + 0.5).astype(np.float16)
    g = (1 + 0.2 * rng.standard_normal(C)).astype(np.float16)
    b = (0.3 * rng.standard_normal(C)).astype(np.float16)
    xd, gd, bd = (torch.from_numpy(a).cuda() for a in (x, g, b))
    print("layernorm16", M, C, flush=True)
    assert close(dthip.layernorm16(xd, gd, bd, 1e-5).cpu().numpy(), oracle.np_layernorm16(x, g, b, 1e-5), b)
    assert close(dthip.layernorm16(xd, None, None, 1e-5).cpu().numpy(), oracle.np_layernorm16(x, None, None, 1e-5))
    big = torch.zeros((M, C + 16), dtype=torch.float16, device="cuda")
    big[:, 8:8 + C].copy_(xd)
    out = torch.full((M, C + 16), 3.0, dtype=torch.float16, device="cuda")
    dthip.layernorm16(big[:, 8:8 + C], gd, bd, 1e-5, out=out[:, 8:8 + C])
    assert torch.equal(out[:, 8:8 + C], dthip.layernorm16(xd, gd, bd, 1e-5))
    assert float((out[:, :8] - 3).abs().max()) == 0 and float((out[:, 8 + C:] - 3).abs().max()) == 0
    same = xd.clone()
    dthip.layernorm16(same, gd, bd, 1e-5, out=same)
    assert torch.equal(same, dthip.layernorm16(xd, gd, bd, 1e-5))
    ln = dthip.LayerNorm(1e-5, [1])
    ln.weight, ln.bias = gd, bd
    assert torch.equal(ln(xd), dthip.layernorm16(xd, gd, bd, 1e-5))

