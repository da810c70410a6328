"""GPU parity: palettized Dense (K0 depalettize, K1 GEMM) against the CPU oracle, through the C ABI.

Bars: palette lookup / index unpack bit-exact; GEMM outputs max-abs <= 2e-2 and rel-RMS <= 1e-3
(fp16 outputs, fp32 accumulation on both sides)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 2e-2, 1e-3


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available()
    return torch


def to_dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_weight(dthip, oracle, rng, N, K, q, nib, std=0.02):
    packed, pal, idx = oracle.synth_qx_weight(rng, N, K, q, nib, std)
    return dthip.QxTensor.from_packed(packed, q, nib, (N, K)), packed


@pytest.mark.parametrize("q", [4, 5, 6, 7, 8])
@pytest.mark.parametrize("nib", [32, 512, 1024, 4096, 16384, 24])
def test_depalettize_bit_exact(dthip, oracle, torch_cuda, q, nib):
    torch = torch_cuda
    rng = np.random.default_rng(q * 1000 + nib)
    for count in (1, 31, 32, 33, nib - 1, nib, nib + 1, 5 * nib + 77, 64 * 1024 + 8):
        print("depalettize", q, nib, count, flush=True)
        packed, pal, idx = oracle.synth_qx_weight(rng, 1, count, q, nib, 1.0)
        w = dthip.QxTensor.from_packed(packed, q, nib, (1, count))
        got = w.dequantize().cpu().numpy().reshape(-1)
        want = oracle.C.depalettize(q, nib, count, packed)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


CASES = [
    # (M, N, K, q, nib)  -- chosen to hit: every palette placement, ragged M / N edges, both tile shapes
    (256, 256, 256, 8, 16384),    # shared palettes, nib > K
    (300, 200, 512, 6, 4096),     # shared palettes, ragged M and N (small tile)
    (1100, 520, 512, 6, 4096),    # big tile, ragged M and N
    (1024, 512, 1024, 4, 512),    # per-row palettes (nib < K, K % nib == 0)
    (1024, 256, 2048, 5, 1024),   # per-row palettes
    (128, 384, 768, 4, 512),      # nib < K, K % nib != 0 -> lookups from global memory
    (257, 129, 320, 6, 4096),     # SD1.5-like K = 320
    (64, 96, 96, 7, 64),          # small everything
    (1024, 256, 512, 8, 512),     # q8 with nib == K (many palettes -> global or shared)
    (130, 70, 100, 6, 32),        # K % 32 != 0 -> generic kernel
    (130, 70, 128, 6, 24),        # nib % 32 != 0 -> generic kernel
    (1024, 200, 512, 6, 4096),    # big tile, ragged N only
    (1536, 384, 256, 5, 1024),    # q5p, a palette block per four rows
    (4100, 130, 128, 4, 512),     # ragged last token tile and a two-row last feature tile
    (2048, 256, 192, 6, 64),      # the palette block changes inside a row every two K-tiles
    (1300, 1024, 1024, 8, 4096),  # 256-entry palettes with small blocks: fit beside no big tile -> small tile, per-row table
    (1100, 520, 768, 8, 512),     # the same with several blocks per row (K % nib != 0), ragged edges
    (1100, 768, 512, 7, 1024),    # 128-entry palettes, two rows per block
    (2600, 2304, 512, 8, 512),    # the same palettes with enough work for the 256-token x 128-feature tile; ragged M
    (2560, 2500, 768, 8, 4096),   # that tile with K % nib != 0 and a ragged last feature tile
    (3000, 2200, 512, 7, 1024),   # that tile with 128-entry palettes, ragged both ways
]


@pytest.mark.parametrize("M,N,K,q,nib", CASES)
def test_dense_qx_vs_oracle(dthip, oracle, torch_cuda, M, N, K, q, nib):
    torch = torch_cuda
    rng = np.random.default_rng(hash((M, N, K, q, nib)) % (2 ** 32))
    print("dense", M, N, K, q, nib, flush=True)
    X = rng.standard_normal((M, K)).astype(np.float16)
    w, packed = make_weight(dthip, oracle, rng, N, K, q, nib)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    d = dthip.Dense(count=N, name="x_q")
    d.weight, d.bias = w, to_dev(torch, bias)
    got = d(to_dev(torch, X)).cpu().numpy()
    want = oracle.C.dense_qx(X, packed, q, nib, N, bias)
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    # no-bias variant
    d2 = dthip.Dense(count=N, noBias=True)
    d2.weight = w
    got2 = d2(to_dev(torch, X)).cpu().numpy()
    mx, rr = oracle.err_stats(got2, oracle.C.dense_qx(X, packed, q, nib, N, None))
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


@pytest.mark.parametrize("q,nib,K,N", [(8, 16384, 256, 320), (6, 4096, 512, 256), (5, 1024, 2048, 256),
                                       (4, 512, 1024, 300), (4, 512, 768, 128), (7, 8192, 128, 256),
                                       (8, 4096, 1024, 6144)])  # (the last: 256 x 128 tile, per-row 256-entry tables)
def test_effective_weights_bit_exact(dthip, oracle, torch_cuda, q, nib, K, N):
    """X = I_K makes Y = W^T exactly (one nonzero product per output, fp16-representable):
    the weights the fused kernel multiplies by are bit-for-bit the dequantized tensor."""
    torch = torch_cuda
    rng = np.random.default_rng(q + K)
    print("effective weights", q, nib, K, N, flush=True)
    w, packed = make_weight(dthip, oracle, rng, N, K, q, nib, std=1.0)
    d = dthip.Dense(count=N, noBias=True)
    d.weight = w
    Y = d(to_dev(torch, np.eye(K, dtype=np.float16))).cpu().numpy()
    W = oracle.C.depalettize(q, nib, N * K, packed).reshape(N, K)
    assert np.array_equal(Y.view(np.uint16), np.ascontiguousarray(W.T).view(np.uint16))


def test_dense_shared_input_three_weights_and_views(dthip, oracle, torch_cuda):
    """x_q / x_k / x_v in one launch, input a strided row view, outputs written into one wide buffer."""
    torch = torch_cuda
    rng = np.random.default_rng(11)
    M, K, N = 640, 512, 256
    big = rng.standard_normal((M, K + 64)).astype(np.float16)
    xb = to_dev(torch, big)
    xv = xb[:, 32:32 + K]  # row stride K + 64, base offset 32 elements (16-byte aligned)
    ws, packs, biases = [], [], []
    for i in range(3):
        w, p = make_weight(dthip, oracle, rng, N, K, 6, 4096)
        ws.append(w)
        packs.append(p)
        biases.append((rng.standard_normal(N) * 0.02).astype(np.float16))
    out = torch.zeros((M, 3 * N), dtype=torch.float16, device="cuda")
    outs = [out[:, i * N:(i + 1) * N] for i in range(3)]
    print("dense 3 weights", flush=True)
    dthip.dense_multi(xv, ws, [to_dev(torch, b) for b in biases[:2]] + [None], outs=outs)
    got = out.cpu().numpy()
    X = np.ascontiguousarray(big[:, 32:32 + K])
    for i in range(3):
        want = oracle.C.dense_qx(X, packs[i], 6, 4096, N, biases[i] if i < 2 else None)
        mx, rr = oracle.err_stats(got[:, i * N:(i + 1) * N], want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)


def test_dense_plain_fp16_weight(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(12)
    M, N, K = 333, 320, 320
    X = rng.standard_normal((M, K)).astype(np.float16)
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    b = (rng.standard_normal(N) * 0.05).astype(np.float16)
    d = dthip.Dense(count=N)
    d.weight, d.bias = dthip.QxTensor.from_f16(W), to_dev(torch, b)
    print("dense fp16", flush=True)
    got = d(to_dev(torch, X)).cpu().numpy()
    mx, rr = oracle.err_stats(got, oracle.C.dense(X, W, b))
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_dense_special_cases(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(13)
    M, N, K, q, nib = 256, 256, 512, 6, 4096
    X = rng.standard_normal((M, K)).astype(np.float16)
    nblocks = (N * K + nib - 1) // nib
    idx = rng.integers(0, 1 << q, size=N * K, dtype=np.uint8)
    b = rng.standard_normal(N).astype(np.float16)
    # zero palette -> Y == bias exactly
    w = dthip.QxTensor.from_packed(dthip.pack_qx(q, nib, np.zeros((nblocks, 1 << q), np.float16), idx), q, nib, (N, K))
    d = dthip.Dense(count=N)
    d.weight, d.bias = w, to_dev(torch, b)
    print("dense special", flush=True)
    assert np.array_equal(d(to_dev(torch, X)).cpu().numpy(), np.broadcast_to(b, (M, N)))
    # single-valued palette -> Y = c * rowsum(X)
    w = dthip.QxTensor.from_packed(dthip.pack_qx(q, nib, np.full((nblocks, 1 << q), 0.5, np.float16), idx), q, nib, (N, K))
    d = dthip.Dense(count=N, noBias=True)
    d.weight = w
    got = d(to_dev(torch, X)).cpu().numpy().astype(np.float64)
    want = 0.5 * X.astype(np.float64).sum(axis=1, keepdims=True) * np.ones((1, N))
    assert np.max(np.abs(got - want)) <= np.max(np.abs(want)) * 2.0 ** -10 + 1e-3
    # empty batch is a no-op
    assert dthip.Dense.__call__(d, torch.zeros((0, K), dtype=torch.float16, device="cuda")).shape == (0, N)


def test_dense_rows_beyond_4gib(dthip, oracle, torch_cuda):
    """X rows spread over more than 4 GiB (a view with a huge row stride): the tiled kernel's 32-bit byte offsets do
    not reach, so the call takes the any-shape kernel -- same results as the compact copy of the same rows."""
    torch = torch_cuda
    rng = np.random.default_rng(12)
    K, N, ld = 128, 192, (1 << 30) + 8
    w, packed = make_weight(dthip, oracle, rng, N, K, 6, 4096, std=0.05)
    rows = rng.standard_normal((3, K)).astype(np.float16)
    big = torch.empty(2 * ld + K, dtype=torch.float16, device="cuda")
    view = torch.as_strided(big, (3, K), (ld, 1))
    view.copy_(to_dev(torch, rows))
    print("dense rows beyond 4 GiB", flush=True)
    got = dthip.dense_multi(view, [w], [None])[0].cpu().numpy()
    mx, rr = oracle.err_stats(got, oracle.C.dense_qx(rows, packed, 6, 4096, N, None))
    assert mx <= MAX_ABS and rr <= REL_RMS
    del big, view


def test_dense_rejects_bad_arguments(dthip, torch_cuda):
    torch = torch_cuda
    w = dthip.QxTensor(torch.zeros(1024, dtype=torch.uint8, device="cuda"), 3, 32, (4, 32))
    d = dthip.Dense(count=4, noBias=True)
    d.weight = w
    with pytest.raises(dthip.DtError) as e:
        d(torch.zeros((8, 32), dtype=torch.float16, device="cuda"))
    assert e.value.status == dthip.DT_INVALID


def test_dense_flux_qkv_full_size_sampled(dthip, oracle, torch_cuda):
    """Headline benchmark shape (M 4608, K 3072, three N 3072 q6p weights in one launch): a sample of rows
    against the oracle, plus linearity Y(2x) == 2 Y(x) (power-of-two scaling is exact in fp32 and in normal fp16)."""
    torch = torch_cuda
    rng = np.random.default_rng(14)
    M, K, N, q, nib = 4608, 3072, 3072, 6, 4096
    X = rng.standard_normal((M, K)).astype(np.float16)
    ws, packs, biases = [], [], []
    for i in range(3):
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib)
        ws.append(w)
        packs.append(p)
        biases.append((rng.standard_normal(N) * 0.02).astype(np.float16))
    xd = to_dev(torch, X)
    print("dense full size", flush=True)
    outs = dthip.dense_multi(xd, ws, [to_dev(torch, b) for b in biases])
    rows = np.sort(rng.choice(M, size=24, replace=False))
    rows[0], rows[-1] = 0, M - 1
    for i in range(3):
        got = outs[i].cpu().numpy()[rows]
        want = oracle.C.dense_qx(np.ascontiguousarray(X[rows]), packs[i], q, nib, N, biases[i])
        mx, rr = oracle.err_stats(got, want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)
    o1 = dthip.dense_multi(xd, ws, [None] * 3)
    o2 = dthip.dense_multi(xd * 2, ws, [None] * 3)
    for a, b in zip(o1, o2):
        # exact wherever 2y is a normal fp16 number; subnormal results may round differently
        normal = a.abs() >= 2.0 ** -13
        assert torch.equal((a * 2)[normal], b[normal])
        assert float((a.float() * 2 - b.float()).abs().max()) <= 2.0 ** -23


def test_dense_plain_fp16_full_size_equals_palettized(dthip, oracle, torch_cuda):
    """Plain fp16 weights at the benchmark's shape (M 4608, K 3072, three N 3072 weights in one launch, the plain
    path's own schedule: one barrier per pair of K-tiles): sampled rows against the oracle, and bit for bit what the
    palettized path gives for the same effective weights (both accumulate the k-steps in the same order)."""
    torch = torch_cuda
    rng = np.random.default_rng(41)
    M, K, N, q, nib = 4608, 3072, 3072, 6, 4096
    X = rng.standard_normal((M, K)).astype(np.float16)
    ws, biases = [], []
    for i in range(3):
        w, _ = make_weight(dthip, oracle, rng, N, K, q, nib)
        ws.append(w)
        biases.append((rng.standard_normal(N) * 0.02).astype(np.float16))
    plain = [dthip.QxTensor.from_f16(w.dequantize()) for w in ws]
    xd = to_dev(torch, X)
    bd = [to_dev(torch, b) for b in biases]
    print("dense plain fp16 full size", flush=True)
    got = dthip.dense_multi(xd, plain, bd)
    ref = dthip.dense_multi(xd, ws, bd)
    rows = np.sort(rng.choice(M, size=16, replace=False))
    rows[0], rows[-1] = 0, M - 1
    for i in range(3):
        assert torch.equal(got[i], ref[i]), i
        W = plain[i].data.cpu().numpy()
        want = oracle.C.dense(np.ascontiguousarray(X[rows]), W, biases[i])
        mx, rr = oracle.err_stats(got[i].cpu().numpy()[rows], want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)
    # a launch of less than two pairs of K-tiles, and one whose token count leaves a ragged last tile
    for (m, k) in ((300, 64), (1500, 128), (4100, 192)):
        x = to_dev(torch, rng.standard_normal((m, k)).astype(np.float16))
        w, _ = make_weight(dthip, oracle, rng, 512, k, q, 512)
        p = dthip.QxTensor.from_f16(w.dequantize())
        assert torch.equal(dthip.dense_multi(x, [p], [None])[0], dthip.dense_multi(x, [w], [None])[0]), (m, k)


@pytest.mark.parametrize("M,head_dim,q,nib", [(700, 128, 6, 4096), (300, 128, 8, 16384), (130, 64, 6, 4096),
                                              (1024, 128, 6, 4096), (4200, 128, 5, 1024)])
def test_dense_fused_head_norm_rope(dthip, oracle, torch_cuda, M, head_dim, q, nib):
    """x_q / x_k / x_v with the per-head RMSNorm + RoPE of Q and K fused behind the projection (V left plain):
    equals Dense -> RMSNorm(axis: [3]) -> cmul(rot) of the oracle.  head_dim 128 runs inside the GEMM epilogue,
    64 as a pass after it."""
    torch = torch_cuda
    rng = np.random.default_rng(M + head_dim)
    K, H = 512, 3
    N = H * head_dim
    pos0 = 11
    X = rng.standard_normal((M, K)).astype(np.float16)
    ws, packs, biases, gammas = [], [], [], []
    for i in range(3):
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
        ws.append(w)
        packs.append(p)
        biases.append((rng.standard_normal(N) * 0.05).astype(np.float16))
        gammas.append((1 + 0.05 * rng.standard_normal(head_dim)).astype(np.float16))
    theta = rng.uniform(-3, 3, size=(pos0 + M, head_dim // 2))
    rot = np.empty((pos0 + M, head_dim), np.float16)
    rot[:, 0::2] = np.cos(theta)
    rot[:, 1::2] = np.sin(theta)
    rot_d = to_dev(torch, rot)
    epi = [dthip.HeadEpilogue(to_dev(torch, gammas[0]), rot_d, pos0, 1e-6, head_dim),
           dthip.HeadEpilogue(to_dev(torch, gammas[1]), rot_d, pos0, 1e-6, head_dim), None]
    out = torch.zeros((M, 3 * N), dtype=torch.float16, device="cuda")
    outs = [out[:, i * N:(i + 1) * N] for i in range(3)]
    print("dense fused heads", M, head_dim, q, flush=True)
    dthip.dense_multi(to_dev(torch, X), ws, [to_dev(torch, b) for b in biases], outs=outs, epilogues=epi)
    got = out.cpu().numpy()
    for i in range(3):
        y = oracle.C.dense_qx(X, packs[i], q, nib, N, biases[i])
        if i < 2:
            y = oracle.C.cmul(oracle.C.rmsnorm(y.reshape(M, H, head_dim), gammas[i], 1e-6), rot[pos0:]).reshape(M, N)
        mx, rr = oracle.err_stats(got[:, i * N:(i + 1) * N], y)
        assert mx <= MAX_ABS and rr <= 2 * REL_RMS, (i, mx, rr)
    # norm only / rotation only
    for epi1 in (dthip.HeadEpilogue(to_dev(torch, gammas[0]), None, 0, 1e-6, head_dim),
                 dthip.HeadEpilogue(None, rot_d, pos0, 1e-6, head_dim)):
        o1 = dthip.dense_multi(to_dev(torch, X), [ws[0]], [None], epilogues=[epi1])[0].cpu().numpy()
        y = oracle.C.dense_qx(X, packs[0], q, nib, N, None).reshape(M, H, head_dim)
        y = oracle.C.rmsnorm(y, gammas[0], 1e-6) if epi1.rot is None else oracle.C.cmul(y, rot[pos0:])
        mx, rr = oracle.err_stats(o1, y.reshape(M, N))
        assert mx <= MAX_ABS and rr <= 2 * REL_RMS, (mx, rr)


@pytest.mark.parametrize("Ms,q,nib", [((1100, 200), 6, 4096), ((1030, 70, 300), 4, 512), ((200, 90), 6, 4096), ((1024, 256), 16, 0)])
def test_dense_grouped_equals_separate(dthip, oracle, torch_cuda, Ms, q, nib):
    """Independent problems (different X, weights, epilogues) enqueued as one call give bit-identical results to
    one dt_dense call per problem, and both match the oracle.  The first two cases go out as a single launch
    (a problem with >= 1024 rows), the third falls back to problem-by-problem."""
    torch = torch_cuda
    rng = np.random.default_rng(sum(Ms) + q)
    K, H, hd = 256, 2, 128
    N = H * hd
    problems, packs, Xs, gam = [], [], [], []
    for gi, M in enumerate(Ms):
        X = rng.standard_normal((M, K)).astype(np.float16)
        Xs.append(X)
        ws, ps = [], []
        for i in range(2):
            if q == 16:
                Wh = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
                ws.append(dthip.QxTensor.from_f16(Wh))
                ps.append(Wh)
            else:
                w, p = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
                ws.append(w)
                ps.append(p)
        packs.append(ps)
        g = (1 + 0.05 * rng.standard_normal(hd)).astype(np.float16)
        gam.append(g)
        epi = [dthip.HeadEpilogue(to_dev(torch, g), None, 0, 1e-6, hd), None] if gi != 1 else None
        problems.append(dict(x=to_dev(torch, X), weights=ws, biases=[None, None], epilogues=epi))
    print("dense grouped", Ms, q, flush=True)
    together = dthip.dense_grouped(problems)
    for gi, p in enumerate(problems):
        alone = dthip.dense_multi(p["x"], p["weights"], p["biases"], epilogues=p["epilogues"])
        for i in range(2):
            assert torch.equal(together[gi][i], alone[i]), (gi, i)
            ref = oracle.C.dense(Xs[gi], packs[gi][i]) if q == 16 else oracle.C.dense_qx(Xs[gi], packs[gi][i], q, nib, N)
            if p["epilogues"] is not None and i == 0:
                ref = oracle.C.rmsnorm(ref.reshape(-1, H, hd), gam[gi], 1e-6).reshape(-1, N)
            mx, rr = oracle.err_stats(together[gi][i].cpu().numpy(), ref)
            assert mx <= MAX_ABS and rr <= 2 * REL_RMS, (gi, i, mx, rr)


def test_dense_grouped_empty_and_bad(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(5)
    assert dthip.dense_grouped([]) == []
    w, _ = make_weight(dthip, oracle, rng, 64, 64, 6, 64)
    x0 = torch.zeros((0, 64), dtype=torch.float16, device="cuda")
    x1 = to_dev(torch, rng.standard_normal((5, 64)).astype(np.float16))
    outs = dthip.dense_grouped([dict(x=x0, weights=[w], biases=[None]), dict(x=x1, weights=[w], biases=[None])])
    assert outs[0][0].shape == (0, 64) and outs[1][0].shape == (5, 64)
    assert torch.equal(outs[1][0], dthip.dense_multi(x1, [w], [None])[0])
    bad = dthip.QxTensor(w.data, 3, w.nib, w.shape)
    with pytest.raises(dthip.DtError):
        dthip.dense_grouped([dict(x=x1, weights=[w], biases=[None]), dict(x=x1, weights=[bad], biases=[None])])


@pytest.mark.parametrize("M,N,K,q,nib", [(300, 512, 256, 6, 4096), (1100, 384, 128, 4, 512), (70, 100, 96, 6, 64), (257, 256, 192, 16, 0)])
def test_dense_post_feed_forward_and_residual(dthip, oracle, torch_cuda, M, N, K, q, nib):
    """Dense with the elementwise tails of the block's feed-forward / residual paths in the epilogue:
    linear1(x).GELU(tanh), swish, and x + (y .* gate).to(of: x) into an fp32 residual stream (with and without keeping
    the fp16 result), against the oracle's Dense followed by its numpy tails.  One fp16 ulp on the activations (the
    device evaluates tanh / sigmoid through exp2 and an approximate reciprocal)."""
    torch = torch_cuda
    rng = np.random.default_rng(M + N)
    X = rng.standard_normal((M, K)).astype(np.float16)
    if q == 16:
        Wh = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
        w, ref = dthip.QxTensor.from_f16(Wh), lambda b: oracle.C.dense(X, Wh, b)
    else:
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
        ref = lambda b: oracle.C.dense_qx(X, p, q, nib, N, b)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16)
    gate = (1 + 0.3 * rng.standard_normal(N)).astype(np.float16)
    res0 = rng.standard_normal((M, N)).astype(np.float32)
    y = ref(bias)
    xd, bd, gd = to_dev(torch, X), to_dev(torch, bias), to_dev(torch, gate)
    print("dense post", M, N, K, q, flush=True)

    def ulps(a, b):
        ai, bi = a.view(np.int16).astype(np.int32), b.view(np.int16).astype(np.int32)
        ai = np.where(ai < 0, -32768 - ai, ai)
        bi = np.where(bi < 0, -32768 - bi, bi)
        return np.abs(ai - bi).max()

    # GELU / swish on two projections sharing x, plain third
    outs = dthip.dense_post(xd, [w, w, w], [bd, bd, bd], [dthip.DensePost(dthip.ACT_GELU_TANH), dthip.DensePost(dthip.ACT_SWISH), None])
    plain = dthip.dense_multi(xd, [w], [bd])[0]
    assert torch.equal(outs[2], plain)
    mx, rr = oracle.err_stats(plain.cpu().numpy(), y)
    assert mx <= MAX_ABS and rr <= 2 * REL_RMS
    y_dev = plain.cpu().numpy()              # tails are checked on the device's own Dense result: exact op-by-op semantics
    assert ulps(outs[0].cpu().numpy(), oracle.np_gelu_tanh16(y_dev)) <= 1
    assert ulps(outs[1].cpu().numpy(), oracle.np_swish16(y_dev)) <= 1
    # gated residual, fp16 result kept
    res = torch.from_numpy(res0.copy()).cuda()
    o = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(gate=gd, residual=res)])[0]
    want16 = (y_dev.astype(np.float32) * gate.astype(np.float32)[None, :]).astype(np.float16)
    assert np.array_equal(o.cpu().numpy().view(np.uint16), want16.view(np.uint16))
    assert np.array_equal(res.cpu().numpy(), oracle.np_gated_residual(res0, y_dev, gate))
    # accumulate only (no fp16 output), no gate, GELU first; residual is a row-strided view
    big = torch.zeros((M, N + 8), dtype=torch.float32, device="cuda")
    view = big[:, 4:4 + N]
    view.copy_(torch.from_numpy(res0))
    o2 = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(dthip.ACT_GELU_TANH, residual=view, keep_output=False)])[0]
    assert o2 is None
    got = view.cpu().numpy()
    want = oracle.np_gated_residual(res0, oracle.np_gelu_tanh16(y_dev))
    assert np.max(np.abs(got - want)) <= 2.0 ** -10 * np.maximum(1, np.abs(y_dev.astype(np.float32))).max()
    assert float(big[:, :4].abs().max()) == 0 and float(big[:, 4 + N:].abs().max()) == 0


@pytest.mark.parametrize("M,N,K,q,nib,rank,scale", [
    (300, 512, 256, 6, 4096, 16, 1.0),     # rank below a K-tile: the up projection takes the generic kernel
    (1100, 384, 128, 4, 512, 64, 0.5),     # tiled up projection, scaled branch
    (513, 256, 192, 16, 0, 128, 0.75),     # plain fp16 base
    (70, 100, 96, 6, 64, 8, 2.0),          # everything through the generic kernel
])
def test_lora_dense(dthip, oracle, torch_cuda, M, N, K, q, nib, rank, scale):
    """LoRADense: dense(x) + up(scale * down(x)) with the base left palettized (Models/LoRA.swift:85-142).  The
    epilogue's scale and addend steps are checked bit for bit on the device's own intermediates (exact op-by-op
    rounding), the whole chain against the oracle's composition within the Dense bar."""
    torch = torch_cuda
    rng = np.random.default_rng(M + rank)
    X = rng.standard_normal((M, K)).astype(np.float16)
    if q == 16:
        Wh = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
        w, ref = dthip.QxTensor.from_f16(Wh), lambda b: oracle.C.dense(X, Wh, b)
    else:
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
        ref = lambda b: oracle.C.dense_qx(X, p, q, nib, N, b)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16)
    down = (rng.standard_normal((rank, K)) * 0.1).astype(np.float16)
    up = (rng.standard_normal((N, rank)) * 0.1).astype(np.float16)
    xd, bd = to_dev(torch, X), to_dev(torch, bias)
    print("lora dense", M, N, K, q, rank, scale, flush=True)
    layer = dthip.LoRADense(N, dthip.LoRANetworkConfiguration(rank, scale))
    layer.weight, layer.bias = w, bd
    layer.down, layer.up = dthip.QxTensor.from_f16(down), dthip.QxTensor.from_f16(up)
    out = layer(xd).cpu().numpy()
    # whole chain against the oracle
    want = oracle.np_add16(ref(bias), oracle.np_lora_branch16(X, down, up, scale))
    mx, rr = oracle.err_stats(out, want)
    assert mx <= MAX_ABS and rr <= 2 * REL_RMS
    # the steps one by one on the device's own intermediates: exact
    # (the layer pads the rank to a multiple of 64 with zeros; the same padded pair is used here)
    base = dthip.dense_multi(xd, [w], [bd])[0]
    dn, upp = layer._padded()
    assert dn.shape[0] % 64 == 0 and upp.shape == (N, dn.shape[0])
    d0 = dthip.dense_multi(xd, [dn], [None])[0]
    d1 = dthip.dense_post(xd, [dn], [None], [dthip.DensePost(scale=scale)])[0]
    assert np.array_equal(d1.cpu().numpy().view(np.uint16),
                          (d0.cpu().numpy().astype(np.float32) * np.float32(scale)).astype(np.float16).view(np.uint16))
    assert float(d1[:, rank:].abs().max()) == 0 if dn.shape[0] > rank else True
    branch = dthip.dense_multi(d1, [upp], [None])[0]
    assert np.array_equal(out.view(np.uint16), oracle.np_add16(base.cpu().numpy(), branch.cpu().numpy()).view(np.uint16))
    # the unpadded pair (any-shape kernel where the rank is no multiple of 64) agrees within the Dense bar
    b2 = dthip.dense_multi(dthip.dense_post(xd, [layer.down], [None], [dthip.DensePost(scale=scale)])[0], [layer.up], [None])[0]
    mx, rr = oracle.err_stats(b2.cpu().numpy(), branch.cpu().numpy())
    assert mx <= MAX_ABS and rr <= 2 * REL_RMS
    # in place: the branch buffer receives the sum; a row-strided addend view; then GELU behind the sum
    buf = branch.clone()
    o = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(addend=buf)], outs=[buf])[0]
    assert np.array_equal(o.cpu().numpy().view(np.uint16), out.view(np.uint16))
    wide = torch.zeros((M, N + 8), dtype=torch.float16, device="cuda")
    wide[:, 4:4 + N].copy_(branch)
    o = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(dthip.ACT_GELU_TANH, addend=wide[:, 4:4 + N])])[0]
    g = layer(xd, post=dthip.DensePost(dthip.ACT_GELU_TANH))
    assert torch.equal(o, g)
    # the layer forks its down projection onto a second stream and joins it again: as a captured graph too
    cs = torch.cuda.Stream()
    cs.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(cs):
        layer(xd)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cs):
            captured = layer(xd)
        for _ in range(2):
            captured.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(captured.cpu().numpy().view(np.uint16), out.view(np.uint16))
            layer(xd)  # eager work between the replays
            torch.cuda.synchronize()
    torch.cuda.current_stream().wait_stream(cs)
    # one fp16 ulp, or 2^-19 where GELU's 1 + tanh cancels (inputs below -3: results of 1e-4 and less)
    got16, want16 = o.cpu().numpy(), oracle.np_gelu_tanh16(out)
    tol = np.maximum(np.spacing(np.abs(want16)).astype(np.float32), np.float32(2.0 ** -19))
    assert np.all(np.abs(got16.astype(np.float32) - want16.astype(np.float32)) <= tol)
    # rank 0 / no matching keys: the plain Dense
    plain = dthip.LoRADense(N, dthip.LoRANetworkConfiguration(0))
    plain.weight, plain.bias = w, bd
    assert torch.equal(plain(xd), base)


def test_dense_grouped_with_tails_equals_separate(dthip, oracle, torch_cuda):
    """Problems that carry elementwise tails share a launch like plain ones (c_o / x_o with gate and residual,
    c_linear1 / x_linear1 with GELU): bit-identical to one dt_dense_qx_post_f16 call per problem, for the fused launch
    (a problem with M >= 1024), the problem-by-problem route (small M) and a mix of a tail problem with a head-epilogue
    problem, which must not share a launch."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    K, N, q, nib = 256, 384, 6, 4096
    for Ms in ((1100, 200), (150, 60)):
        print("dense grouped tails", Ms, flush=True)
        xs = [to_dev(torch, rng.standard_normal((M, K)).astype(np.float16)) for M in Ms]
        ws = [make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)[0] for _ in Ms]
        bs = [to_dev(torch, (rng.standard_normal(N) * 0.1).astype(np.float16)) for _ in Ms]
        gates = [to_dev(torch, (1 + 0.3 * rng.standard_normal(N)).astype(np.float16)) for _ in Ms]
        res0 = [torch.randn((M, N), dtype=torch.float32, device="cuda") for M in Ms]
        # gate + residual, accumulate only
        want = [r.clone() for r in res0]
        for x, w, b, g, r in zip(xs, ws, bs, gates, want):
            assert dthip.dense_post(x, [w], [b], [dthip.DensePost(gate=g, residual=r, keep_output=False)])[0] is None
        got = [r.clone() for r in res0]
        outs = dthip.dense_grouped([dict(x=x, weights=[w], biases=[b],
                                         posts=[dthip.DensePost(gate=g, residual=r, keep_output=False)])
                                    for x, w, b, g, r in zip(xs, ws, bs, gates, got)])
        assert all(o == [None] for o in outs)
        assert all(torch.equal(a, b) for a, b in zip(got, want))
        assert not torch.equal(got[0], res0[0])
        # GELU with the fp16 result kept
        want = [dthip.dense_post(x, [w], [b], [dthip.DensePost(dthip.ACT_GELU_TANH)])[0] for x, w, b in zip(xs, ws, bs)]
        outs = dthip.dense_grouped([dict(x=x, weights=[w], biases=[b], posts=[dthip.DensePost(dthip.ACT_GELU_TANH)])
                                    for x, w, b in zip(xs, ws, bs)])
        assert all(torch.equal(o[0], wv) for o, wv in zip(outs, want))
    # a tail problem next to a head-epilogue problem
    M, D = 1100, 128
    x = to_dev(torch, rng.standard_normal((M, K)).astype(np.float16))
    wh, _ = make_weight(dthip, oracle, rng, 2 * D, K, q, nib, std=0.05)
    gamma = to_dev(torch, (1 + 0.1 * rng.standard_normal(D)).astype(np.float16))
    epi = dthip.HeadEpilogue(gamma, None, 0, 1e-6, D)
    want_h = dthip.dense_multi(x, [wh], [None], epilogues=[epi])[0]
    want_t = dthip.dense_post(xs[0][:100], [ws[0]], [bs[0]], [dthip.DensePost(dthip.ACT_SWISH)])[0]
    outs = dthip.dense_grouped([dict(x=x, weights=[wh], biases=[None], epilogues=[epi]),
                                dict(x=xs[0][:100], weights=[ws[0]], biases=[bs[0]], posts=[dthip.DensePost(dthip.ACT_SWISH)])])
    assert torch.equal(outs[0][0], want_h) and torch.equal(outs[1][0], want_t)
    # fp32 gate: the residual receives float(result) * gate, the product formed in fp32; exact against numpy
    g32 = (1 + 0.3 * rng.standard_normal(N)).astype(np.float32)
    r0 = rng.standard_normal((100, N)).astype(np.float32)
    r = to_dev(torch, r0)
    plain = dthip.dense_multi(xs[0][:100], [ws[0]], [bs[0]])[0].cpu().numpy()
    kept = dthip.dense_post(xs[0][:100], [ws[0]], [bs[0]], [dthip.DensePost(gate=to_dev(torch, g32), residual=r)])[0]
    assert np.array_equal(kept.cpu().numpy().view(np.uint16), plain.view(np.uint16))  # the output is the ungated result
    assert np.array_equal(r.cpu().numpy(), oracle.np_gated_residual32(r0, plain, g32))
    with pytest.raises(dthip.DtError):  # an fp32 gate needs a residual to go into
        dthip.dense_post(xs[0][:100], [ws[0]], [bs[0]], [dthip.DensePost(gate=to_dev(torch, g32))])
    # a problem may not carry both
    with pytest.raises(dthip.DtError):
        dthip.dense_grouped([dict(x=x, weights=[wh], biases=[None], epilogues=[epi], posts=[dthip.DensePost()])])


@pytest.mark.parametrize("M,N,K,q,nib", [(1100, 384, 128, 6, 4096), (70, 100, 96, 6, 64), (300, 320, 320, 16, 0)])
def test_dense_post_multiplicand_and_erf_gelu(dthip, oracle, torch_cuda, M, N, K, q, nib):
    """The gated feed-forward of the UNet block, fc10(x) .* GELU()(fc11(x)): the product step bit for bit on the
    device's own Dense result (in place over the multiplicand too), the erf GELU within one fp16 ulp."""
    torch = torch_cuda
    rng = np.random.default_rng(M + K)
    X = rng.standard_normal((M, K)).astype(np.float16)
    if q == 16:
        w = dthip.QxTensor.from_f16((rng.standard_normal((N, K)) * 0.05).astype(np.float16))
    else:
        w, _ = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
    bias = to_dev(torch, (rng.standard_normal(N) * 0.1).astype(np.float16))
    xd = to_dev(torch, X)
    print("dense multiplicand", M, N, K, q, flush=True)
    plain = dthip.dense_multi(xd, [w], [bias])[0]
    g = dthip.dense_post(xd, [w], [bias], [dthip.DensePost(dthip.ACT_GELU_ERF)])[0]
    got, want = g.cpu().numpy(), oracle.np_gelu_erf16(plain.cpu().numpy())
    tol = np.maximum(np.spacing(np.abs(want)).astype(np.float32), np.float32(2.0 ** -19))
    assert np.all(np.abs(got.astype(np.float32) - want.astype(np.float32)) <= tol)
    m = to_dev(torch, rng.standard_normal((M, N)).astype(np.float16))
    prod = dthip.dense_post(xd, [w], [bias], [dthip.DensePost(multiplicand=m)])[0]
    assert np.array_equal(prod.cpu().numpy().view(np.uint16), oracle.np_mul16(plain.cpu().numpy(), m.cpu().numpy()).view(np.uint16))
    buf = m.clone()
    dthip.dense_post(xd, [w], [bias], [dthip.DensePost(multiplicand=buf)], outs=[buf])
    assert torch.equal(buf, prod)
    with pytest.raises(ValueError):
        dthip.dense_post(xd, [w], [bias], [dthip.DensePost(multiplicand=m[:, :-1])])


def test_dense_post_bad_args(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(9)
    w, _ = make_weight(dthip, oracle, rng, 64, 64, 6, 64)
    x = to_dev(torch, rng.standard_normal((4, 64)).astype(np.float16))
    with pytest.raises(dthip.DtError):
        dthip.dense_post(x, [w], [None], [dthip.DensePost(activation=7)])
    with pytest.raises((ValueError, TypeError)):
        dthip.dense_post(x, [w], [None], [dthip.DensePost(residual=torch.zeros((4, 64), dtype=torch.float16, device="cuda"))])
    with pytest.raises(ValueError):
        dthip.dense_post(x, [w], [None], [dthip.DensePost(gate=torch.zeros(3, dtype=torch.float16, device="cuda"))])
    with pytest.raises(ValueError):
        dthip.dense_post(x, [w], [None], [dthip.DensePost(addend=torch.zeros((4, 32), dtype=torch.float16, device="cuda"))])
    with pytest.raises(dthip.DtError):
        dthip.dense_post(x, [w], [None], [dthip.DensePost(scale=float("inf"))])


def test_dense_flux_2048_q4p_full_size_sampled(dthip, oracle, torch_cuda):
    """Long-sequence Flux shape (M 16896, K 3072, three N 3072 q4p weights with 512-element blocks -- six palette
    blocks per weight row -- in one launch): a sample of rows against the oracle, plus linearity Y(2x) == 2 Y(x)."""
    torch = torch_cuda
    rng = np.random.default_rng(16)
    M, K, N, q, nib = 16896, 3072, 3072, 4, 512
    ws, packs, biases = [], [], []
    for i in range(3):
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib)
        ws.append(w)
        packs.append(p)
        biases.append((rng.standard_normal(N) * 0.02).astype(np.float16))
    gen = torch.Generator(device="cuda").manual_seed(16)
    xd = torch.randn((M, K), device="cuda", generator=gen).half()
    print("dense flux 2048 q4p full size", flush=True)
    outs = dthip.dense_multi(xd, ws, [to_dev(torch, b) for b in biases])
    rows = np.sort(rng.choice(M, size=16, replace=False))
    rows[0], rows[-1] = 0, M - 1
    rt = torch.from_numpy(rows).cuda()
    xr = np.ascontiguousarray(xd[rt].cpu().numpy())
    for i in range(3):
        want = oracle.C.dense_qx(xr, packs[i], q, nib, N, biases[i])
        mx, rr = oracle.err_stats(outs[i][rt].cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)
    o1 = dthip.dense_multi(xd, ws, [None] * 3)
    o2 = dthip.dense_multi(xd * 2, ws, [None] * 3)
    for a, b in zip(o1, o2):
        normal = a.abs() >= 2.0 ** -13
        assert torch.equal((a * 2)[normal], b[normal])
        assert float((a.float() * 2 - b.float()).abs().max()) <= 2.0 ** -23


def test_dense_wan_full_size_sampled(dthip, oracle, torch_cuda):
    """The largest benchmark Dense (M 32760, 5120 -> 5120, q5p with 1024-element blocks: five palette blocks per weight
    row): a sample of rows against the oracle, plus linearity Y(2x) == 2 Y(x)."""
    torch = torch_cuda
    rng = np.random.default_rng(15)
    M, K, N, q, nib = 32760, 5120, 5120, 5, 1024
    w, p = make_weight(dthip, oracle, rng, N, K, q, nib)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    gen = torch.Generator(device="cuda").manual_seed(15)
    xd = torch.randn((M, K), device="cuda", generator=gen).half()
    print("dense wan full size", flush=True)
    out = dthip.dense_multi(xd, [w], [to_dev(torch, bias)])[0]
    rows = np.sort(rng.choice(M, size=16, replace=False))
    rows[0], rows[-1] = 0, M - 1
    rt = torch.from_numpy(rows).cuda()
    want = oracle.C.dense_qx(np.ascontiguousarray(xd[rt].cpu().numpy()), p, q, nib, N, bias)
    mx, rr = oracle.err_stats(out[rt].cpu().numpy(), want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    a = dthip.dense_multi(xd, [w], [None])[0]
    b = dthip.dense_multi(xd * 2, [w], [None])[0]
    normal = a.abs() >= 2.0 ** -13
    assert torch.equal((a * 2)[normal], b[normal])
    assert float((a.float() * 2 - b.float()).abs().max()) <= 2.0 ** -23


def test_dense_post_activations_over_every_fp16_input(dthip, oracle, torch_cuda):
    """Every finite fp16 value goes through a Dense with an identity weight (one non-zero term per output: y == x)
    and then through each activation of the elementwise tail: the result is within one fp16 ulp of the function
    evaluated in float64 and rounded once, over the whole input domain (tiny outputs for x < -3 included, where
    1 + tanh(u) and 1 + erf(z) would cancel)."""
    torch = torch_cuda
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x16 = bits.view(np.float16).copy()
    x16[~np.isfinite(x16)] = 0
    x16 = x16.reshape(1024, 64)
    w = dthip.QxTensor.from_f16(np.eye(64, dtype=np.float16))
    xd = to_dev(torch, x16)
    print("dense post activations, whole fp16 domain", flush=True)
    plain = dthip.dense_multi(xd, [w], [None])[0].cpu().numpy()
    assert np.array_equal(plain, x16)  # (as values: -0 comes back as +0)

    def ulps(a, b):
        ai, bi = a.view(np.int16).astype(np.int32), b.view(np.int16).astype(np.int32)
        ai = np.where(ai < 0, -32768 - ai, ai)
        bi = np.where(bi < 0, -32768 - bi, bi)
        return np.abs(ai - bi)

    for act, fn in ((dthip.ACT_GELU_TANH, oracle.np_gelu_tanh16), (dthip.ACT_SWISH, oracle.np_swish16),
                    (dthip.ACT_GELU_ERF, oracle.np_gelu_erf16)):
        got = dthip.dense_post(xd, [w], [None], [dthip.DensePost(act)])[0].cpu().numpy()
        want = fn(x16)
        assert np.array_equal(np.isfinite(got), np.isfinite(want)), act
        ok = np.isfinite(want)
        assert int(ulps(got, want)[ok].max()) <= 1, (act, int(ulps(got, want)[ok].max()))


def test_dense_q8p_full_size_sampled(dthip, oracle, torch_cuda):
    """"Palettized Dense alone" at its full shape with 8-bit indices: M 4608, K 3072, three N 3072 q8p weights (256-entry
    palettes, 16384 elements per block: a block spans 5 1/3 weight rows, so a 256-row tile holds about 50 palettes) in
    one launch, and the single 3072 -> 3072 output projection.  Sampled rows against the oracle, and the weights the
    kernel multiplies by checked bit for bit at K = 3072 (X = I makes Y = W^T exactly)."""
    torch = torch_cuda
    rng = np.random.default_rng(28)
    M, K, N, q, nib = 4608, 3072, 3072, 8, 16384
    X = rng.standard_normal((M, K)).astype(np.float16)
    ws, packs, biases = [], [], []
    for i in range(3):
        w, p = make_weight(dthip, oracle, rng, N, K, q, nib)
        ws.append(w)
        packs.append(p)
        biases.append((rng.standard_normal(N) * 0.02).astype(np.float16))
    xd = to_dev(torch, X)
    print("dense q8p full size", flush=True)
    outs = dthip.dense_multi(xd, ws, [to_dev(torch, b) for b in biases])
    rows = np.sort(rng.choice(M, size=24, replace=False))
    rows[0], rows[-1] = 0, M - 1
    for i in range(3):
        got = outs[i].cpu().numpy()[rows]
        want = oracle.C.dense_qx(np.ascontiguousarray(X[rows]), packs[i], q, nib, N, biases[i])
        mx, rr = oracle.err_stats(got, want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)
    one = dthip.dense_multi(xd, [ws[1]], [to_dev(torch, biases[1])])[0]
    assert torch.equal(one, outs[1])
    print("dense q8p effective weights at K = 3072", flush=True)
    eye = torch.eye(K, dtype=torch.float16, device="cuda")
    for i in (0, 2):
        Y = dthip.dense_multi(eye, [ws[i]], [None])[0].cpu().numpy()
        W = oracle.C.depalettize(q, nib, N * K, packs[i]).reshape(N, K)
        assert np.array_equal(Y.view(np.uint16), np.ascontiguousarray(W.T).view(np.uint16))


def test_lora_dense_swap_and_zero_scale(dthip, oracle, torch_cuda):
    """A second LoRA of the same shape replaces the first (its tensors may land at the addresses the first pair's
    had: the padded copies must follow the new pair, and an in-place update of a pair too); a scale of zero switches
    the branch off as `0 * down(x)` does (Models/LoRA.swift:129-134)."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    M, N, K, q, nib, rank = 200, 256, 192, 6, 4096, 16
    X = rng.standard_normal((M, K)).astype(np.float16)
    w, p = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
    xd = to_dev(torch, X)
    layer = dthip.LoRADense(N, dthip.LoRANetworkConfiguration(rank, 1.0), noBias=True)
    layer.weight = w
    base = oracle.C.dense_qx(X, p, q, nib, N, None)
    print("lora swap", flush=True)
    for trial in range(3):
        down = (rng.standard_normal((rank, K)) * 0.1).astype(np.float16)
        up = (rng.standard_normal((N, rank)) * 0.1).astype(np.float16)
        layer.down = layer.up = None          # the old pair is released before the new one is made
        torch.cuda.empty_cache() if trial == 2 else None
        layer.down, layer.up = dthip.QxTensor.from_f16(down), dthip.QxTensor.from_f16(up)
        out = layer(xd).cpu().numpy()
        want = oracle.np_add16(base, oracle.np_lora_branch16(X, down, up, 1.0))
        mx, rr = oracle.err_stats(out, want)
        assert mx <= MAX_ABS and rr <= 2 * REL_RMS, (trial, mx, rr)
    # in-place update of the current pair
    down2 = (rng.standard_normal((rank, K)) * 0.1).astype(np.float16)
    layer.down.data.copy_(to_dev(torch, down2))
    out = layer(xd).cpu().numpy()
    want = oracle.np_add16(base, oracle.np_lora_branch16(X, down2, up, 1.0))
    mx, rr = oracle.err_stats(out, want)
    assert mx <= MAX_ABS and rr <= 2 * REL_RMS, (mx, rr)
    # scale 0: the plain Dense
    zero = dthip.LoRADense(N, dthip.LoRANetworkConfiguration(rank, 0.0), noBias=True)
    zero.weight, zero.down, zero.up = w, layer.down, layer.up
    assert torch.equal(zero(xd), dthip.dense_multi(xd, [w], [None])[0])
    with pytest.raises(ValueError):
        dthip.dense_post(xd, [w], [None], [dthip.DensePost(scale=0.0)])


def test_operators_on_a_side_stream(dthip, oracle, torch_cuda):
    """`stream=` other than the current stream: the operator's own allocations, copies and launches all go to that
    stream (clone-then-launch operators such as RMSNorm and cmul, and attention with its workspace)."""
    torch = torch_cuda
    rng = np.random.default_rng(78)
    B, S, H, D = 1, 300, 4, 128
    x = rng.standard_normal((B, S, H, D)).astype(np.float16)
    g = (1 + 0.02 * rng.standard_normal(D)).astype(np.float16)
    rot = dthip.Flux1RotaryPositionEmbedding(15, 20, 0, channels=D).astype(np.float16)
    side = torch.cuda.Stream()
    want_y = oracle.C.rmsnorm(x[0], g, 1e-6)
    xd, gd, rd, yd = to_dev(torch, x), to_dev(torch, g), to_dev(torch, rot), to_dev(torch, want_y[None])
    torch.cuda.synchronize()  # the uploads above ran on the default stream
    print("operators on a side stream", flush=True)
    n = dthip.RMSNorm(epsilon=1e-6, axis=[3])
    n.weight = gd
    y = n(xd, stream=side)
    z = dthip.Functional.cmul(yd, rd.reshape(1, S, 1, D), stream=side)
    o = dthip.sdpa_segments([xd], [xd], [xd], 1 / np.sqrt(D), gamma_q=[gd], gamma_k=[gd], rot_q=rd, rot_k=rd, stream=side)
    side.synchronize()
    want_z = oracle.C.cmul(want_y, rot)
    assert np.all(np.abs(y.cpu().numpy()[0].astype(np.float32) - want_y.astype(np.float32)) <= np.abs(want_y.astype(np.float32)) * 2.0 ** -10 + 2.0 ** -24)
    assert np.array_equal(z.cpu().numpy()[0].view(np.uint16), want_z.view(np.uint16))
    want_o = oracle.C.sdpa(want_z[None], want_z[None], x, 1 / np.sqrt(D))
    mx, rr = oracle.err_stats(o.cpu().numpy(), want_o)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


@pytest.mark.parametrize("M,N,K,q,nib,rank,scale", [(300, 512, 256, 6, 4096, 16, 1.0), (1100, 384, 192, 4, 512, 64, 0.5),
                                                     (70, 100, 96, 16, 0, 8, 2.0), (4608, 3072, 3072, 6, 4096, 32, 0.75)])
def test_lora_dense_high_precision(dthip, oracle, torch_cuda, M, N, K, q, nib, rank, scale):
    """LoRADense with highPrecision: the low-rank pair is fp32 and the branch fp16(up(scale * down(float(x)))) is
    computed in fp32 throughout (Models/LoRA.swift:117-139).  The branch against float64 (one fp16 ulp, or 2^-16 of the
    row's largest entry where cancellation leaves less), the sum bit for bit on the device's own base and branch."""
    torch = torch_cuda
    rng = np.random.default_rng(M + rank)
    X = rng.standard_normal((M, K)).astype(np.float16)
    if q == 16:
        Wh = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
        w = dthip.QxTensor.from_f16(Wh)
    else:
        w, _ = make_weight(dthip, oracle, rng, N, K, q, nib, std=0.05)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16)
    down = (rng.standard_normal((rank, K)) * 0.1).astype(np.float32)
    up = (rng.standard_normal((N, rank)) * 0.1).astype(np.float32)
    xd, bd = to_dev(torch, X), to_dev(torch, bias)
    print("lora dense high precision", M, N, K, q, rank, scale, flush=True)
    layer = dthip.LoRADense(N, dthip.LoRANetworkConfiguration(rank, scale, highPrecision=True))
    layer.weight, layer.bias = w, bd
    layer.down = dthip.QxTensor(to_dev(torch, down), 32, 0, down.shape)
    layer.up = dthip.QxTensor(to_dev(torch, up), 32, 0, up.shape)
    out = layer(xd).cpu().numpy()
    # the branch alone, through the C ABI
    T = torch.empty((M, rank), dtype=torch.float32, device="cuda")
    br = torch.empty((M, N), dtype=torch.float16, device="cuda")
    st = dthip.lib().dt_lora_branch_f32_f16(None, M, K, xd.data_ptr(), K, layer.down.data.data_ptr(), rank,
                                            layer.up.data.data_ptr(), N, scale, T.data_ptr(), br.data_ptr(), N)
    assert st == 0
    got, want = br.cpu().numpy().astype(np.float64), oracle.np_lora_branch32(X, down, up, scale).astype(np.float64)
    tol = np.maximum(np.abs(want) * 2.0 ** -10, np.abs(want).max(axis=1, keepdims=True) * 2.0 ** -16) + 2.0 ** -24
    assert np.all(np.abs(got - want) <= tol), float(np.max(np.abs(got - want) / tol))
    base = dthip.dense_multi(xd, [w], [bd])[0].cpu().numpy()
    assert np.array_equal(out.view(np.uint16), oracle.np_add16(base, br.cpu().numpy()).view(np.uint16))
    # with a tail behind the sum
    g = layer(xd, post=dthip.DensePost(dthip.ACT_GELU_TANH))
    o = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(dthip.ACT_GELU_TANH, addend=br)])[0]
    assert torch.equal(g, o)


@pytest.mark.parametrize("M,K,N,codec", [(8192, 320, 320, "q6p"), (8192, 320, 320, "f16"), (154, 768, 320, "q6p"),
                                         (154, 768, 320, "f16")])
def test_dense_sd15_shapes_full_size(dthip, oracle, M, K, N, codec):
    """SD 1.5 attention projections at full size (Models/UNet.swift:105-107, 277-279, 307): toqueries / tokeys /
    tovalues / unifyheads 320 -> 320 over batch 2 x 4096 tokens, and the cross-attention tokeys / tovalues
    768 -> 320 over 2 x 77 context tokens; palettized (q6p) and plain fp16 weights, every output element."""
    import torch

    rng = np.random.default_rng(M + K)
    x = (rng.standard_normal((M, K))).astype(np.float16)
    b = (rng.standard_normal(N) * 0.02).astype(np.float16)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    if codec == "f16":
        w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
        qx = dthip.QxTensor.from_f16(w)
        want = oracle.C.dense(x, w, b)
    else:
        q, nib = dthip.CODEC[codec]
        packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 0.05)
        qx = dthip.QxTensor.from_packed(packed, q, nib, (N, K))
        want = oracle.C.dense_qx(x, packed, q, nib, N, b)
    print("dense sd1.5 shape", M, K, N, codec, flush=True)
    got = dthip.dense_multi(dev(x), [qx], [dev(b)])[0].cpu().numpy()
    mx, rr = oracle.err_stats(got, want)
    assert mx <= 2e-2 and rr <= 1e-3, (mx, rr)
