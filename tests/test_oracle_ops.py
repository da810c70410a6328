"""Pins the oracle's floating-point functions by closed forms, invariants,
float64 brute force and special cases that reduce to library routines.
Tolerances: the oracle rounds once to fp16, so |err| <= ~1 ulp(fp16) of the
float64 result (rel 2^-10) unless stated."""
import numpy as np
import pytest


def f16(a):
    return np.asarray(a, dtype=np.float16)


def assert_close16(got, want64, extra=0.0):
    """got (fp16) equals want (float64) to within one fp16 rounding (+ extra abs slack)."""
    got = got.astype(np.float64)
    tol = np.abs(want64) * 2.0 ** -10 + 2.0 ** -24 + extra
    assert np.all(np.abs(got - want64) <= tol), float(np.max(np.abs(got - want64) - tol))


# ------------------------------------------------------------------ Dense

def test_dense_vs_float64(oracle):
    rng = np.random.default_rng(1)
    M, N, K = 37, 53, 200
    X = f16(rng.standard_normal((M, K)))
    W = f16(rng.standard_normal((N, K)) * 0.05)
    b = f16(rng.standard_normal(N) * 0.1)
    assert_close16(oracle.C.dense(X, W, b), oracle.np_dense64(X, W, b), extra=2e-5)
    assert_close16(oracle.C.dense(X, W, None), oracle.np_dense64(X, W), extra=2e-5)


def test_dense_transposed_operand_would_fail(oracle):
    """W is [out, in]: with X = I_K the product is W^T exactly (bit-exact, fp16 values)."""
    rng = np.random.default_rng(2)
    N, K = 24, 16
    W = f16(rng.standard_normal((N, K)))
    Y = oracle.C.dense(f16(np.eye(K)), W)
    assert np.array_equal(Y.view(np.uint16), np.ascontiguousarray(W.T).view(np.uint16))


def test_dense_strided_rows_and_bias_only(oracle):
    rng = np.random.default_rng(3)
    big = f16(rng.standard_normal((10, 64)))
    Xv = big[:, :32]  # row stride 64, width 32
    W = f16(rng.standard_normal((8, 32)))
    assert np.array_equal(oracle.C.dense(Xv, W), oracle.C.dense(np.ascontiguousarray(Xv), W))
    b = f16(rng.standard_normal(8))
    Y = oracle.C.dense(f16(np.zeros((5, 32))), W, b)
    assert np.array_equal(Y, np.broadcast_to(b, (5, 8)))


@pytest.mark.parametrize("q,nib", [(8, 64), (6, 32), (5, 64), (4, 32), (7, 32)])
def test_dense_qx_special_cases(oracle, q, nib):
    rng = np.random.default_rng(q)
    M, N, K = 9, 12, 40  # N*K = 480: several blocks, ragged last block for nib=64
    X = f16(rng.standard_normal((M, K)))
    nblocks = (N * K + nib - 1) // nib
    idx = rng.integers(0, 1 << q, size=N * K, dtype=np.uint8)
    # zero palette -> Y = bias
    b = f16(rng.standard_normal(N))
    packed = oracle.C.palettize_pack(q, nib, np.zeros((nblocks, 1 << q), np.float16), idx)
    assert np.array_equal(oracle.C.dense_qx(X, packed, q, nib, N, b), np.broadcast_to(b, (M, N)))
    # single-valued palette c -> Y[m, n] = c * rowsum(X[m])
    c = np.float16(0.5)
    packed = oracle.C.palettize_pack(q, nib, np.full((nblocks, 1 << q), c, np.float16), idx)
    want = 0.5 * X.astype(np.float64).sum(axis=1, keepdims=True) * np.ones((1, N))
    assert_close16(oracle.C.dense_qx(X, packed, q, nib, N), want, extra=2e-6)
    # random palette: equals dense over the closed-form dequantized weight
    pal = f16(rng.standard_normal((nblocks, 1 << q)) * 0.02)
    packed = oracle.C.palettize_pack(q, nib, pal, idx)
    Wd = pal[np.arange(N * K) // nib, idx].reshape(N, K)
    assert np.array_equal(oracle.C.dense_qx(X, packed, q, nib, N, b), oracle.C.dense(X, Wd, b))


# ------------------------------------------------------------------ RMSNorm / cmul

def test_rmsnorm_closed_forms(oracle):
    rng = np.random.default_rng(4)
    x = f16(rng.standard_normal((6, 5, 128)))
    g = f16(1 + 0.02 * rng.standard_normal(128))
    assert_close16(oracle.C.rmsnorm(x, g), oracle.np_rmsnorm64(x, g), extra=1e-6)
    # constant row c, gamma 1: y = sign(c) / sqrt(1 + eps / c^2)
    for c in (0.5, -2.0, 3.0):
        y = oracle.C.rmsnorm(f16(np.full((2, 64), c)), None, eps=1e-6)
        want = np.sign(c) / np.sqrt(1 + 1e-6 / c ** 2)
        assert_close16(y, np.full((2, 64), want))
    # torch's library routine on the same fp16-rounded input
    torch = pytest.importorskip("torch")
    xt = torch.from_numpy(x.astype(np.float32))
    yt = torch.nn.functional.rms_norm(xt, (128,), torch.from_numpy(g.astype(np.float32)), 1e-6).numpy()
    assert_close16(oracle.C.rmsnorm(x, g), yt.astype(np.float64), extra=1e-5)


def test_cmul_identities(oracle):
    rng = np.random.default_rng(5)
    S, H, D = 7, 3, 16
    x = f16(rng.standard_normal((S, H, D)))
    theta = rng.uniform(-3, 3, size=(S, D // 2))
    rot = np.empty((S, D), np.float64)
    rot[:, 0::2] = np.cos(theta)
    rot[:, 1::2] = np.sin(theta)
    y = oracle.C.cmul(x, f16(rot))
    assert_close16(y, oracle.np_cmul64(x, f16(rot)), extra=1e-6)
    # theta = 0 -> identity, bit-exact
    ident = np.zeros((S, D), np.float16)
    ident[:, 0::2] = 1
    assert np.array_equal(oracle.C.cmul(x, ident).view(np.uint16), x.view(np.uint16))
    # rotation preserves each pair's magnitude (to fp16 rounding of table and output)
    m0 = np.hypot(x[..., 0::2].astype(np.float64), x[..., 1::2].astype(np.float64))
    m1 = np.hypot(y[..., 0::2].astype(np.float64), y[..., 1::2].astype(np.float64))
    assert np.allclose(m0, m1, rtol=3e-3, atol=3e-3)
    # theta = pi/2 -> (a, b) -> (-b, a): a sign or swap slip fails here
    q = np.zeros((S, D), np.float16)
    q[:, 1::2] = 1
    yq = oracle.C.cmul(x, q)
    assert np.array_equal(yq[..., 0::2], -x[..., 1::2]) and np.array_equal(yq[..., 1::2], x[..., 0::2])


# ------------------------------------------------------------------ rotary tables

def test_rope_flux_properties(oracle):
    h, w, t = 6, 5, 4
    tab = oracle.C.rope_flux(h, w, t, 128)
    assert tab.shape == (t + h * w, 128)
    cos, sin = tab[:, 0::2].astype(np.float64), tab[:, 1::2].astype(np.float64)
    assert np.allclose(cos ** 2 + sin ** 2, 1, atol=1e-6)
    # text rows first, all (1, 0)
    assert np.all(tab[:t, 0::2] == 1) and np.all(tab[:t, 1::2] == 0)
    # axis widths 16 / 56 / 56 -> 8 / 28 / 28 pairs; axis 0 is position 0 for image tokens
    assert np.all(tab[:, 0:16:2] == 1) and np.all(tab[:, 1:16:2] == 0)
    # spot values: token (y=1, x=0), first pair of axis 1 has theta = 1 rad; (y=0,x=1) first pair of axis 2
    i = 1 * w + 0 + t
    assert tab[i, 16] == np.float32(np.cos(1.0)) and tab[i, 17] == np.float32(np.sin(1.0))
    i = 0 * w + 1 + t
    assert tab[i, 16 + 56] == np.float32(np.cos(1.0)) and tab[i, 16 + 57] == np.float32(np.sin(1.0))
    assert tab[i, 16] == 1 and tab[i, 17] == 0
    # closed form for every entry: theta = pos / 10000^(2k/dim)
    for y in range(h):
        for x in range(w):
            row = tab[y * w + x + t]
            for (off, dim, pos) in ((0, 16, 0), (16, 56, y), (72, 56, x)):
                k = np.arange(dim // 2)
                th = pos / np.power(10000.0, 2 * k / dim)
                assert np.array_equal(row[off:off + dim:2], np.cos(th).astype(np.float32))
                assert np.array_equal(row[off + 1:off + dim:2], np.sin(th).astype(np.float32))
    # factorisation: the y-part depends on y only, the x-part on x only
    a = tab[t:].reshape(h, w, 128)
    assert np.all(a[:, :, 16:72] == a[:, :1, 16:72]) and np.all(a[:, :, 72:] == a[:1, :, 72:])


def test_rope_flux_reference_images(oracle):
    h, w, t = 4, 4, 2
    tab = oracle.C.rope_flux(h, w, t, 128, ref_sizes=[(2, 3), (3, 2)])
    assert tab.shape == (t + 16 + 6 + 6, 128)
    base = t + h * w
    # first reference: h=0,w=0 -> 2+0 > 3+0 false -> hOffset = 0; time index 1
    r0 = tab[base:base + 6].reshape(2, 3, 128)
    assert r0[0, 0, 0] == np.float32(np.cos(1.0)) and r0[0, 0, 1] == np.float32(np.sin(1.0))
    assert r0[1, 0, 16] == np.float32(np.cos(1.0)) and r0[0, 2, 72] == np.float32(np.cos(2.0))
    # second reference: now h=2, w=3; 3+2 > 2+3 false -> hOffset = 2
    r1 = tab[base + 6:base + 12].reshape(3, 2, 128)
    assert r1[0, 0, 16] == np.float32(np.cos(2.0)) and r1[0, 1, 72] == np.float32(np.cos(1.0))


def test_rope_wan_properties(oracle):
    T, h, w = 3, 4, 5
    tab = oracle.C.rope_wan(h, w, T, 128)
    assert tab.shape == (T * h * w, 128)
    # widths 44 / 42 / 42
    a = tab.reshape(T, h, w, 128)
    assert np.all(a[:, :, :, :44] == a[:, :1, :1, :44])
    assert np.all(a[:, :, :, 44:86] == a[:1, :, :1, 44:86])
    assert np.all(a[:, :, :, 86:] == a[:1, :1, :, 86:])
    assert a[1, 0, 0, 0] == np.float32(np.cos(1.0)) and a[0, 1, 0, 44] == np.float32(np.cos(1.0))
    assert a[0, 0, 1, 87] == np.float32(np.sin(1.0))
    k = np.arange(22)
    th = 2 / np.power(10000.0, 2 * k / 44)
    assert np.array_equal(a[2, 0, 0, 0:44:2], np.cos(th).astype(np.float32))
    c, s = tab[:, 0::2].astype(np.float64), tab[:, 1::2].astype(np.float64)
    assert np.allclose(c * c + s * s, 1, atol=1e-6)


# ------------------------------------------------------------------ SDPA

def rand_qkv(rng, B, Sq, Skv, Hq, Hk, D):
    return (f16(rng.standard_normal((B, Sq, Hq, D))), f16(rng.standard_normal((B, Skv, Hk, D))),
            f16(rng.standard_normal((B, Skv, Hk, D))))


@pytest.mark.parametrize("shape", [(1, 5, 7, 2, 2, 8), (2, 8, 3, 4, 2, 4), (1, 33, 77, 2, 1, 40)])
def test_sdpa_vs_bruteforce64(oracle, shape):
    rng = np.random.default_rng(6)
    q, k, v = rand_qkv(rng, *shape)
    scale = 1 / np.sqrt(shape[-1])
    o = oracle.C.sdpa(q, k, v, scale)
    assert_close16(o, oracle.np_sdpa64(q, k, v, scale), extra=3e-6)


def test_sdpa_invariants(oracle):
    rng = np.random.default_rng(7)
    B, Sq, Skv, H, D = 1, 9, 21, 2, 16
    q, k, v = rand_qkv(rng, B, Sq, Skv, H, H, D)
    scale = 0.25
    o = oracle.C.sdpa(q, k, v, scale)
    # constant V -> O equals that constant (rows of P sum to 1)
    vc = np.broadcast_to(f16(rng.standard_normal((1, 1, H, D))), v.shape).copy()
    oc = oracle.C.sdpa(q, k, vc, scale)
    assert_close16(oc, np.broadcast_to(vc[:, :1].astype(np.float64), oc.shape), extra=1e-6)
    # joint permutation of K/V rows leaves O unchanged (up to fp32 summation order)
    perm = rng.permutation(Skv)
    op = oracle.C.sdpa(q, k[:, perm].copy(), v[:, perm].copy(), scale)
    assert np.max(np.abs(op.astype(np.float64) - o.astype(np.float64))) <= 2e-3
    # strided views (a concatenated buffer sliced in place) == contiguous copies
    buf = f16(rng.standard_normal((B, Skv + 5, H, 2 * D)))
    kv = buf[:, 2:2 + Skv, :, :D]
    assert np.array_equal(oracle.C.sdpa(q, kv, kv, scale), oracle.C.sdpa(q, kv.copy(), kv.copy(), scale))
    # scale1 convention (Q and K pre-multiplied by D^-1/4, scale 1) == scaleMerged within fp16 rounding of Q, K
    s4 = np.float16(D ** -0.25)
    o1 = oracle.C.sdpa(f16(q * s4), f16(k * s4), v, 1.0)
    om = oracle.C.sdpa(q, k, v, 1 / np.sqrt(D))
    assert np.max(np.abs(o1.astype(np.float64) - om.astype(np.float64))) <= 2e-2
    # one-hot attention: huge matching key dominates -> O row == that V row
    kk = f16(np.zeros((1, 4, 1, 8)))
    kk[0, 2, 0, 0] = 60
    qq = f16(np.zeros((1, 1, 1, 8)))
    qq[0, 0, 0, 0] = 60
    vv = f16(rng.standard_normal((1, 4, 1, 8)))
    assert np.array_equal(oracle.C.sdpa(qq, kk, vv, 1.0)[0, 0, 0], vv[0, 2, 0])


def test_sdpa_round_mid_is_within_tolerance(oracle):
    """Whether the reference keeps fp32 or fp16 intermediates moves results by far less than the
    path's tolerance (max-abs 2e-2, rel-RMS 1e-3 is the GPU bar; here rel-RMS of the two choices)."""
    rng = np.random.default_rng(8)
    q, k, v = rand_qkv(rng, 1, 64, 256, 2, 2, 64)
    a = oracle.C.sdpa(q, k, v, 0.125, round_mid=0)
    b = oracle.C.sdpa(q, k, v, 0.125, round_mid=1)
    mx, rr = oracle.err_stats(b, a)
    assert mx < 2e-2 and rr < 5e-3


def test_instruction_counts(oracle):
    # DenseInstructionCount = M*N*K, SDPA = B*H*(2D+5)*Sa*Sb
    assert oracle.C.dense_instruction_count(4608, 3072, 3072) == 4608 * 3072 * 3072
    assert oracle.C.sdpa_instruction_count(1, 24, 128, 4608, 4608) == 24 * 261 * 4608 * 4608


def test_elementwise_tails_pinned(oracle):
    """GELU(tanh), swish and the gated residual against what the mathematics fixes."""
    import math
    x = np.linspace(-8, 8, 4001).astype(np.float16)
    g = oracle.np_gelu_tanh16(x).astype(np.float64)
    xd = x.astype(np.float64)
    # odd-part identity of any 0.5*x*(1+odd(x)) function: gelu(x) - gelu(-x) = x
    assert np.max(np.abs((g - g[::-1]) - xd)) <= 2e-3 * (1 + np.abs(xd)).max()
    # float64 statement of the same formula, rounded once
    want = 0.5 * xd * (1 + np.tanh(math.sqrt(2 / math.pi) * (xd + 0.044715 * xd ** 3)))
    assert np.array_equal(oracle.np_gelu_tanh16(x), want.astype(np.float16)) or \
        np.max(np.abs(g - want)) <= np.finfo(np.float16).eps * np.maximum(1, np.abs(want)).max()
    # the tanh form stays within 5e-4 + 0.5 % of the exact erf GELU it approximates, and has its limits
    erf = np.vectorize(math.erf)
    exact = 0.5 * xd * (1 + erf(xd / math.sqrt(2)))
    assert np.max(np.abs(g - exact)) <= 3e-3
    assert g[x == 0][0] == 0 and abs(g[-1] - 8) < 1e-2 and abs(g[0]) < 1e-3
    # swish(x) = x * sigmoid(x); swish(x) + swish(-x) = x * tanh(x / 2)
    s = oracle.np_swish16(x).astype(np.float64)
    assert np.max(np.abs(s - xd / (1 + np.exp(-xd)))) <= 4e-3
    assert np.max(np.abs((s + s[::-1]) - xd * np.tanh(xd / 2))) <= 8e-3
    # gated residual: exact on values that need no rounding; gate broadcast over rows; fp16 rounding of the product
    res = np.array([[1.0, 2.0], [3.0, 4.0]], np.float32)
    y = np.array([[0.5, -1.0], [2.0, 0.25]], np.float16)
    gate = np.array([2.0, 4.0], np.float16)
    assert np.array_equal(oracle.np_gated_residual(res, y, gate), np.array([[2.0, -2.0], [7.0, 5.0]], np.float32))
    assert np.array_equal(oracle.np_gated_residual(res, y), res + y.astype(np.float32))
    y2 = np.array([[1.0009765625]], np.float16)            # 1 + 2^-10
    g2 = np.array([1.0009765625], np.float16)
    # (1 + 2^-10)^2 = 1 + 2^-9 + 2^-20 rounds to 1 + 2^-9 in fp16 before it reaches the fp32 stream
    assert oracle.np_gated_residual(np.zeros((1, 1), np.float32), y2, g2)[0, 0] == np.float32(1 + 2.0 ** -9)


def test_lora_branch_pinned(oracle):
    """The low-rank branch up(scale * down(x)) and the fp16 sum, against what the mathematics fixes: exact small
    integers, the rank-1 outer-product form, exact doubling by a power-of-two scale, the merged-weight form
    x (up down)^T within fp16 rounding, and where the intermediate rounding must show."""
    rng = np.random.default_rng(5)
    # small integers: every product and sum is exact in fp16
    X = rng.integers(-3, 4, (7, 8)).astype(np.float16)
    D = rng.integers(-2, 3, (4, 8)).astype(np.float16)
    U = rng.integers(-2, 3, (6, 4)).astype(np.float16)
    want = (X.astype(np.int64) @ D.astype(np.int64).T) @ U.astype(np.int64).T
    assert np.array_equal(oracle.np_lora_branch16(X, D, U).astype(np.int64), want)
    assert np.array_equal(oracle.np_lora_branch16(X, D, U, 2.0).astype(np.int64), 2 * want)
    # a transposed operand or a swapped pair fails the shapes or the values
    assert oracle.np_lora_branch16(X, D, U).shape == (7, 6)
    # rank 1: branch[m, n] = u[n] * fp16(v . x[m])
    v = rng.standard_normal((1, 8)).astype(np.float16)
    u = rng.standard_normal((6, 1)).astype(np.float16)
    Xr = rng.standard_normal((5, 8)).astype(np.float16)
    d = (Xr.astype(np.float64) @ v.astype(np.float64).T).astype(np.float16)
    assert np.array_equal(oracle.np_lora_branch16(Xr, v, u), (d.astype(np.float64) * u.astype(np.float64).T).astype(np.float16))
    # merged weight: equal up to the fp16 rounding of the intermediate and the output
    Dg = (rng.standard_normal((16, 64)) * 0.1).astype(np.float16)
    Ug = (rng.standard_normal((32, 16)) * 0.1).astype(np.float16)
    Xg = rng.standard_normal((9, 64)).astype(np.float16)
    merged = Xg.astype(np.float64) @ (Ug.astype(np.float64) @ Dg.astype(np.float64)).T
    got = oracle.np_lora_branch16(Xg, Dg, Ug, 0.5).astype(np.float64)
    assert np.max(np.abs(got - 0.5 * merged)) <= 4e-3 * np.abs(merged).max()
    # scale by 1/3 is its own rounding step: not the same as scaling the output
    third = oracle.np_lora_branch16(Xg, Dg, Ug, 1 / 3)
    assert np.max(np.abs(third.astype(np.float64) - merged / 3)) <= 4e-3 * np.abs(merged).max()
    # fp16 sum: exact where representable, one rounding (ties to even) where not
    a = np.array([1.0, 2048.0, 2048.0, -0.5], np.float16)
    b = np.array([0.5, 1.0, 3.0, 0.5], np.float16)
    assert np.array_equal(oracle.np_add16(a, b), np.array([1.5, 2048.0, 2052.0, 0.0], np.float16))



def test_layernorm_modulate_pinned(oracle):
    """LayerNorm + adaLN modulation against a library routine (torch layer_norm, fp32) and what the mathematics fixes:
    zero mean / unit variance, invariance under a shift of the input, the two-valued row's closed form, the constant
    row, and the place of each rounding."""
    import torch
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((6, 96)) * 3 + 1.5).astype(np.float32)
    plain = oracle.np_layernorm_modulate16(x, None, None, 1e-6, "f32").astype(np.float64)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (96,), eps=1e-6).numpy().astype(np.float64)
    assert np.max(np.abs(plain - ref)) <= 2.0 ** -10 * np.maximum(1, np.abs(ref)).max()
    assert np.max(np.abs(plain.mean(axis=1))) < 2e-3 and np.max(np.abs(plain.var(axis=1) - 1)) < 5e-3
    # LN(x + c) = LN(x): the mean is subtracted, not ignored
    moved = oracle.np_layernorm_modulate16(x + np.float32(8), None, None, 1e-6, "f32").astype(np.float64)
    assert np.max(np.abs(moved - plain)) <= 2.0 ** -9 * np.abs(plain).max()
    # a row of +a / -a: mean 0, variance a^2 -> +-1 / sqrt(1 + eps / a^2); eps inside the root, added to the variance
    a = np.float32(0.01)
    row = np.tile(np.array([a, -a], np.float32), 8)[None, :]
    want = 1 / np.sqrt(1 + 1e-2 / float(a) ** 2)
    got = oracle.np_layernorm_modulate16(row, None, None, 1e-2, "f32").astype(np.float64)
    assert np.allclose(got, np.tile([want, -want], 8)[None, :], rtol=2e-3)
    # constant row -> zeros -> the shift alone
    sh = rng.standard_normal(16).astype(np.float16)
    const = np.full((1, 16), 3.25, np.float32)
    assert np.array_equal(oracle.np_layernorm_modulate16(const, None, sh, 1e-6, "f16"), sh[None, :])
    # the two modes: "f16" rounds three times and multiplies by scale; "f32" adds 1 to scale and rounds once
    sc16 = (1 + 0.2 * rng.standard_normal(96)).astype(np.float16)
    sh16 = rng.standard_normal(96).astype(np.float16)
    n16 = ref.astype(np.float32).astype(np.float16)
    step = (n16.astype(np.float32) * sc16.astype(np.float32)).astype(np.float16)
    want16 = (step.astype(np.float32) + sh16.astype(np.float32)).astype(np.float16)
    got16 = oracle.np_layernorm_modulate16(x, sc16, sh16, 1e-6, "f16")
    assert np.max(np.abs(got16.astype(np.float64) - want16.astype(np.float64))) <= 2e-3 * np.maximum(1, np.abs(want16)).max()
    sc32 = (0.2 * rng.standard_normal(96)).astype(np.float32)
    sh32 = rng.standard_normal(96).astype(np.float32)
    want32 = ref * (sc32.astype(np.float64) + 1) + sh32.astype(np.float64)
    got32 = oracle.np_layernorm_modulate16(x, sc32, sh32, 1e-6, "f32").astype(np.float64)
    assert np.max(np.abs(got32 - want32)) <= 2.0 ** -10 * np.maximum(1, np.abs(want32)).max()
    # scale = 0 in "f32" mode leaves the normalised value (the +1), in "f16" mode it zeroes it
    z32 = oracle.np_layernorm_modulate16(x, np.zeros(96, np.float32), None, 1e-6, "f32")
    assert np.array_equal(z32, oracle.np_layernorm_modulate16(x, None, None, 1e-6, "f32"))
    assert not oracle.np_layernorm_modulate16(x, np.zeros(96, np.float16), None, 1e-6, "f16").any()
    # "affine": the LayerNorm's own weight and bias, no + 1; the fp32 gate of the residual update multiplies in fp32
    aff = oracle.np_layernorm_modulate16(x, sc32 + 1, sh32, 1e-6, "affine")
    assert np.array_equal(aff, oracle.np_layernorm_modulate16(x, sc32, sh32, 1e-6, "f32")) or \
        np.max(np.abs(aff.astype(np.float64) - got32)) <= 2.0 ** -10 * np.maximum(1, np.abs(want32)).max()
    res = np.array([[1.0, 2.0]], np.float32)
    y = np.array([[1.0009765625, -3.0]], np.float16)
    g = np.array([1.0009765625, 0.5], np.float32)
    # (1 + 2^-10)^2 keeps its 2^-20 term in fp32 (the fp16 gate would round it away)
    assert np.array_equal(oracle.np_gated_residual32(res, y, g),
                          np.array([[np.float32(1) + np.float32(1.0009765625) ** 2, 0.5]], np.float32))
    assert np.array_equal(oracle.np_gated_residual32(res, y), res + y.astype(np.float32))


def test_unet_block_pieces_pinned(oracle):
    """The fp16 LayerNorm with affine, the erf GELU and the fp16 product against library routines and closed forms."""
    import math
    import torch
    rng = np.random.default_rng(21)
    x = (rng.standard_normal((5, 320)) * 2 + 0.3).astype(np.float16)
    g = (1 + 0.2 * rng.standard_normal(320)).astype(np.float16)
    b = (0.3 * rng.standard_normal(320)).astype(np.float16)
    got = oracle.np_layernorm16(x, g, b, 1e-5).astype(np.float64)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x.astype(np.float32)), (320,), torch.from_numpy(g.astype(np.float32)),
                                         torch.from_numpy(b.astype(np.float32)), 1e-5).numpy().astype(np.float64)
    assert np.max(np.abs(got - ref)) <= 2.0 ** -10 * np.maximum(1, np.abs(ref)).max()
    # weight 1 / bias 0 equals no affine; a constant row gives the bias alone
    assert np.array_equal(oracle.np_layernorm16(x, None, None, 1e-5),
                          oracle.np_layernorm16(x, np.ones(320, np.float16), np.zeros(320, np.float16), 1e-5))
    assert np.array_equal(oracle.np_layernorm16(np.full((1, 320), 2.5, np.float16), g, b, 1e-5), b[None, :])
    # erf GELU: torch's exact form; gelu(x) - gelu(-x) = x; it differs from the tanh form (by up to ~5e-4 around |x| = 2)
    t = np.linspace(-6, 6, 2401).astype(np.float16)
    ge = oracle.np_gelu_erf16(t).astype(np.float64)
    ref = torch.nn.functional.gelu(torch.from_numpy(t.astype(np.float64))).numpy()
    assert np.max(np.abs(ge - ref)) <= 2.0 ** -11 * np.maximum(1, np.abs(ref)).max()
    assert np.max(np.abs((ge - ge[::-1]) - t.astype(np.float64))) <= 4e-3
    assert abs(float(oracle.np_gelu_erf16(np.array([1.0], np.float16))[0]) - 0.5 * (1 + math.erf(1 / math.sqrt(2)))) < 1e-3
    assert np.max(np.abs(ge - oracle.np_gelu_tanh16(t).astype(np.float64))) > 1e-4
    # fp16 product: exact where representable, one rounding otherwise
    a = np.array([1.5, 3.0, 1.0009765625], np.float16)
    c = np.array([2.0, 0.5, 1.0009765625], np.float16)
    assert np.array_equal(oracle.np_mul16(a, c), np.array([3.0, 1.5, 1.001953125], np.float16))

