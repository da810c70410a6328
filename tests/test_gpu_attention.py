"""GPU parity: RMSNorm + RoPE (K2) and ScaledDotProductAttention (K3) against the CPU oracle, through the C ABI.

Bar for attention outputs: max-abs <= 2e-2, rel-RMS <= 1e-3.  The norm / rotate pass rounds where the oracle
rounds, so it is held to one fp16 ulp."""
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


def f16(a):
    return np.asarray(a, dtype=np.float16)


def ulp_close(got, want, ulps=1):
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    tol = ulps * (np.abs(want) * 2.0 ** -10 + 2.0 ** -24)
    return np.all(np.abs(got - want) <= tol)


# ------------------------------------------------------------------ K2

@pytest.mark.parametrize("D,H", [(128, 24), (64, 8), (40, 8), (32, 5)])
def test_rmsnorm_per_head(dthip, oracle, torch_cuda, D, H):
    torch = torch_cuda
    rng = np.random.default_rng(D)
    x = f16(rng.standard_normal((2, 37, H, D)))
    g = f16(1 + 0.02 * rng.standard_normal(D))
    n = dthip.RMSNorm(epsilon=1e-6, axis=[3], name="x_norm_q")
    n.weight = to_dev(torch, g)
    print("rmsnorm head", D, H, flush=True)
    got = n(to_dev(torch, x)).cpu().numpy()
    assert ulp_close(got, oracle.C.rmsnorm(x, g, 1e-6))


def test_rmsnorm_whole_row(dthip, oracle, torch_cuda):
    """Wan: RMSNorm(axis: [2]) over the 5120-wide row before the head split."""
    torch = torch_cuda
    rng = np.random.default_rng(1)
    x = f16(rng.standard_normal((1, 50, 5120)))
    g = f16(1 + 0.02 * rng.standard_normal(5120))
    n = dthip.RMSNorm(epsilon=1e-6, axis=[2], name="x_norm_k")
    n.weight = to_dev(torch, g)
    print("rmsnorm row", flush=True)
    got = n(to_dev(torch, x)).cpu().numpy()
    assert ulp_close(got, oracle.C.rmsnorm(x, g, 1e-6))


def test_cmul_rope(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(2)
    h, w, t = 6, 5, 7
    S = t + h * w
    x = f16(rng.standard_normal((1, S, 4, 128)))
    rot = f16(dthip.Flux1RotaryPositionEmbedding(h, w, t, channels=128))
    print("cmul", flush=True)
    got = dthip.Functional.cmul(to_dev(torch, x), to_dev(torch, rot.reshape(1, S, 1, 128))).cpu().numpy()
    want = oracle.C.cmul(x[0], rot)
    assert np.array_equal(got[0].view(np.uint16), want.view(np.uint16))
    # text rows (theta = 0) pass through unchanged
    assert np.array_equal(got[0, :t], x[0, :t])


def test_norm_rope_scale_in_place_on_strided_view(dthip, oracle, torch_cuda):
    """Flux per-head norm + RoPE at a joint-sequence offset, then Wan's D^-1/4 scale, on a view into a wider buffer."""
    torch = torch_cuda
    rng = np.random.default_rng(3)
    B, S, H, D, pos0 = 2, 33, 3, 128, 9
    buf = f16(rng.standard_normal((B, S, 3 * H * D)))
    g = f16(1 + 0.02 * rng.standard_normal(D))
    rot = f16(dthip.Flux1RotaryPositionEmbedding(7, 6, pos0, channels=D))
    dev = to_dev(torch, buf)
    view = dev[:, :, H * D:2 * H * D].unflatten(2, (H, D))  # the K third of a fused QKV buffer
    s4 = float(D) ** -0.25
    print("norm rope in place", flush=True)
    dthip.qk_norm_rope_(view, to_dev(torch, g), 1e-6, True, rot=to_dev(torch, rot), rot_pos0=pos0, post_scale=s4)
    got = dev.cpu().numpy()
    x = np.ascontiguousarray(buf[:, :, H * D:2 * H * D]).reshape(B, S, H, D)
    want = np.stack([oracle.C.cmul(oracle.C.rmsnorm(x[b], g, 1e-6), rot[pos0:pos0 + S]) for b in range(B)])
    want = f16(want.astype(np.float32) * np.float32(s4))
    assert ulp_close(got[:, :, H * D:2 * H * D].reshape(B, S, H, D), want)
    # everything outside the view is untouched
    assert np.array_equal(got[:, :, :H * D], buf[:, :, :H * D]) and np.array_equal(got[:, :, 2 * H * D:], buf[:, :, 2 * H * D:])


def test_norm_rope_rows_not_16_byte_aligned(dthip, oracle, torch_cuda):
    """A view whose rows start 4 bytes off a 16-byte boundary takes the pair-per-lane kernel: same results."""
    torch = torch_cuda
    rng = np.random.default_rng(4)
    B, S, H, D = 1, 41, 3, 128
    buf = f16(rng.standard_normal((B, S, H * D + 2)))
    g = f16(1 + 0.02 * rng.standard_normal(D))
    rot = f16(dthip.Flux1RotaryPositionEmbedding(6, 6, 5, channels=D))
    dev = to_dev(torch, buf)
    view = dev[:, :, 2:].unflatten(2, (H, D))
    print("norm rope unaligned", flush=True)
    dthip.qk_norm_rope_(view, to_dev(torch, g), 1e-6, True, rot=to_dev(torch, rot), rot_pos0=0)
    got = dev.cpu().numpy()
    x = np.ascontiguousarray(buf[:, :, 2:]).reshape(B, S, H, D)
    want = oracle.C.cmul(oracle.C.rmsnorm(x[0], g, 1e-6), rot[:S])
    assert ulp_close(got[0, :, 2:].reshape(S, H, D), want)
    assert np.array_equal(got[:, :, :2], buf[:, :, :2])


# ------------------------------------------------------------------ K3

def rand_qkv(rng, B, Sq, Skv, Hq, Hk, D):
    return (f16(rng.standard_normal((B, Sq, Hq, D))), f16(rng.standard_normal((B, Skv, Hk, D))),
            f16(rng.standard_normal((B, Skv, Hk, D))))


SDPA_CASES = [
    # B, Sq, Skv, Hq, Hk, D
    (1, 128, 64, 2, 2, 128),
    (1, 256, 256, 2, 2, 128),
    (2, 200, 333, 3, 3, 128),     # ragged both ways
    (1, 1, 1, 1, 1, 128),         # single query, single key
    (1, 70, 77, 8, 8, 40),        # SD1.5 cross-attention shape (D = 40, 77 keys)
    (2, 300, 300, 8, 8, 40),      # SD1.5 self-attention (reduced sequence)
    (1, 130, 190, 4, 2, 64),      # grouped heads, D = 64
    (1, 2100, 150, 2, 1, 128),    # long query side (nine 256-row workgroups per head), grouped heads
    (1, 2050, 257, 2, 2, 64),
]


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hk,D", SDPA_CASES)
def test_sdpa_vs_oracle(dthip, oracle, torch_cuda, B, Sq, Skv, Hq, Hk, D):
    torch = torch_cuda
    rng = np.random.default_rng(B * 1000 + Sq + Skv + D)
    q, k, v = rand_qkv(rng, B, Sq, Skv, Hq, Hk, D)
    scale = 1 / np.sqrt(D)
    print("sdpa", B, Sq, Skv, Hq, Hk, D, flush=True)
    op = dthip.ScaledDotProductAttention(scale=scale, flags=dthip.GEMMFlag.Float16)
    got = op(to_dev(torch, q), to_dev(torch, k), to_dev(torch, v)).cpu().numpy()
    want = oracle.C.sdpa(q, k, v, scale)
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_invariants(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(5)
    B, Sq, Skv, H, D = 1, 150, 210, 2, 128
    q, k, v = rand_qkv(rng, B, Sq, Skv, H, H, D)
    op = dthip.ScaledDotProductAttention(scale=1 / np.sqrt(D))
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    print("sdpa invariants", flush=True)
    base = op(qd, kd, vd).cpu().numpy()
    # constant V -> O is that constant
    vc = np.broadcast_to(f16(rng.standard_normal((1, 1, H, D))), v.shape).copy()
    oc = op(qd, kd, to_dev(torch, vc)).cpu().numpy()
    assert np.max(np.abs(oc.astype(np.float64) - vc[:, :1].astype(np.float64))) <= 2e-3
    # joint permutation of K / V rows
    perm = rng.permutation(Skv)
    op_ = op(qd, to_dev(torch, k[:, perm]), to_dev(torch, v[:, perm])).cpu().numpy()
    assert np.max(np.abs(op_.astype(np.float64) - base.astype(np.float64))) <= 4e-3
    # .scale1 convention: Q, K pre-multiplied by D^-1/4 and scale 1  ==  .scaleMerged within tolerance
    s4 = np.float16(D ** -0.25)
    o1 = dthip.ScaledDotProductAttention(scale=1.0)(to_dev(torch, f16(q * s4)), to_dev(torch, f16(k * s4)), vd)
    mx, rr = oracle.err_stats(o1.cpu().numpy(), base)
    assert mx <= MAX_ABS and rr <= 5e-3
    # large logits stay finite (running max is subtracted before the exponential)
    big = op(to_dev(torch, f16(q * 30)), to_dev(torch, f16(k * 30)), vd).cpu().numpy()
    assert np.all(np.isfinite(big))
    mx, rr = oracle.err_stats(big, oracle.C.sdpa(f16(q * 30), f16(k * 30), v, 1 / np.sqrt(D)))
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_segments_equal_concat_and_strided_views(dthip, oracle, torch_cuda):
    """text || image passed as two segments == the concatenated call; Q/K/V are slices of one fused QKV buffer."""
    torch = torch_cuda
    rng = np.random.default_rng(6)
    B, T, HW, H, D = 1, 70, 200, 3, 128
    ctx = f16(rng.standard_normal((B, T, 3, H, D)))      # fused [q|k|v] buffers: stride_s = 3*H*D
    img = f16(rng.standard_normal((B, HW, 3, H, D)))
    cd, xd = to_dev(torch, ctx), to_dev(torch, img)
    scale = 1 / np.sqrt(D)
    print("sdpa segments", flush=True)
    got = dthip.sdpa_segments([cd[:, :, 0], xd[:, :, 0]], [cd[:, :, 1], xd[:, :, 1]], [cd[:, :, 2], xd[:, :, 2]],
                              scale).cpu().numpy()
    q = np.concatenate([ctx[:, :, 0], img[:, :, 0]], axis=1)
    k = np.concatenate([ctx[:, :, 1], img[:, :, 1]], axis=1)
    v = np.concatenate([ctx[:, :, 2], img[:, :, 2]], axis=1)
    want = oracle.C.sdpa(q, k, v, scale)
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    cat = dthip.ScaledDotProductAttention(scale=scale)(to_dev(torch, q), to_dev(torch, k), to_dev(torch, v))
    assert np.array_equal(cat.cpu().numpy().view(np.uint16), got.view(np.uint16))


@pytest.mark.parametrize("lens,D", [((5, 130, 1, 64), 64), ((64, 64, 200), 128), ((3, 2, 1, 70), 40)])
def test_sdpa_many_segments(dthip, oracle, torch_cuda, lens, D):
    """Up to four K/V segments, some shorter than a 64-key tile (several segment boundaries inside one tile) and some
    ending on a tile boundary: bit-identical to the concatenated call, and equal to the oracle."""
    torch = torch_cuda
    rng = np.random.default_rng(sum(lens) + D)
    B, Hq, Hk = 2, 4, 2
    ks = [f16(rng.standard_normal((B, n, Hk, D))) for n in lens]
    vs = [f16(rng.standard_normal((B, n, Hk, D))) for n in lens]
    q = f16(rng.standard_normal((B, 90, Hq, D)))
    scale = 1 / np.sqrt(D)
    print("sdpa many segments", lens, D, flush=True)
    got = dthip.sdpa_segments([to_dev(torch, q)], [to_dev(torch, t) for t in ks], [to_dev(torch, t) for t in vs], scale)
    k, v = np.concatenate(ks, axis=1), np.concatenate(vs, axis=1)
    cat = dthip.ScaledDotProductAttention(scale=scale)(to_dev(torch, q), to_dev(torch, k), to_dev(torch, v))
    assert torch.equal(got, cat)
    mx, rr = oracle.err_stats(got.cpu().numpy(), oracle.C.sdpa(q, k, v, scale))
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_fused_norm_rope_joint(dthip, oracle, torch_cuda):
    """The Flux joint block's attention input stage fused into the call: per-segment per-head RMSNorm
    (c_norm_* / x_norm_*), RoPE over the joint order, then attention."""
    torch = torch_cuda
    rng = np.random.default_rng(7)
    B, T, h, w, H, D = 1, 40, 12, 10, 2, 128
    HW = h * w
    segs = {n: (f16(rng.standard_normal((B, T, H, D))), f16(rng.standard_normal((B, HW, H, D)))) for n in "qkv"}
    gam = {n: (f16(1 + 0.05 * rng.standard_normal(D)), f16(1 + 0.05 * rng.standard_normal(D))) for n in "qk"}
    rot = f16(dthip.Flux1RotaryPositionEmbedding(h, w, T, channels=D))
    scale = 1 / np.sqrt(D)
    dev = lambda a: to_dev(torch, a)
    print("sdpa fused prep", flush=True)
    got = dthip.sdpa_segments(
        [dev(t) for t in segs["q"]], [dev(t) for t in segs["k"]], [dev(t) for t in segs["v"]], scale,
        gamma_q=[dev(g) for g in gam["q"]], gamma_k=[dev(g) for g in gam["k"]], rot_q=dev(rot), rot_k=dev(rot),
    ).cpu().numpy()

    def prep(n):
        parts = [oracle.C.rmsnorm(segs[n][i][0], gam[n][i], 1e-6) for i in range(2)]
        return oracle.C.cmul(np.concatenate(parts, axis=0), rot)[None]

    want = oracle.C.sdpa(prep("q"), prep("k"), np.concatenate(segs["v"], axis=1), scale)
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hk,D,q_only,misalign", [
    (2, 300, 77, 8, 8, 40, True, False),     # SD-style head size 40 (padded to 64 inside): norm on Q only, nothing staged
    (1, 270, 530, 4, 2, 64, False, False),   # grouped heads, D = 64, norm + rotation on both sides, B = 1
    (1, 513, 200, 2, 2, 128, True, True),    # norm weight and table not 16-byte aligned; rotation on Q only
])
def test_sdpa_fused_norm_rope_on_queries_in_kernel(dthip, oracle, torch_cuda, B, Sq, Skv, Hq, Hk, D, q_only, misalign):
    """Per-head RMSNorm and rotation of the queries happen inside the attention kernel (on the query fragments in
    registers), K goes through the staging pass only when it asks for it: against the oracle's RMSNorm -> cmul ->
    attention chain, and -- with prep on the query side only -- with no workspace at all."""
    torch = torch_cuda
    rng = np.random.default_rng(Sq + D)
    q, k, v = rand_qkv(rng, B, Sq, Skv, Hq, Hk, D)
    gq, gk = f16(1 + 0.05 * rng.standard_normal(D)), f16(1 + 0.05 * rng.standard_normal(D))
    use_rot = D % 16 == 0
    n_pos = max(Sq, Skv)
    rot = f16(dthip.WanRotaryPositionEmbedding(1, n_pos, 1, channels=D)) if use_rot else None
    scale = 1 / np.sqrt(D)

    def dev_off(a):
        """On the device, at an address that is 4-byte but not 16-byte aligned when `misalign` asks for it."""
        if not misalign:
            return to_dev(torch, a)
        flat = torch.zeros(a.size + 2, dtype=torch.float16, device="cuda")
        flat[2:] = to_dev(torch, a).reshape(-1)
        return flat[2:].view(*a.shape)

    def prep(x, g, S):
        y = np.stack([oracle.C.rmsnorm(x[b], g, 1e-6) for b in range(B)])
        if use_rot:
            y = np.stack([oracle.C.cmul(y[b], rot[:S]) for b in range(B)])
        return y

    want = oracle.C.sdpa(prep(q, gq, Sq), k if q_only else prep(k, gk, Skv), v, scale)
    kw = dict(gamma_q=[dev_off(gq)], rot_q=None if rot is None else dev_off(rot))
    if not q_only:
        kw.update(gamma_k=[to_dev(torch, gk)], rot_k=None if rot is None else to_dev(torch, rot))
    print("sdpa fused prep on queries", B, Sq, Skv, Hq, Hk, D, q_only, misalign, flush=True)
    got = dthip.sdpa_segments([to_dev(torch, q)], [to_dev(torch, k)], [to_dev(torch, v)], scale, **kw).cpu().numpy()
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_fused_output_projection(dthip, oracle, torch_cuda):
    """SD1.5: multiHeadOutputProjectionFused -- the op owns W_o [HD, HD] and b_o and returns [B, S, HD]."""
    torch = torch_cuda
    rng = np.random.default_rng(8)
    B, Sq, Skv, H, D = 2, 200, 77, 8, 40
    q, k, v = rand_qkv(rng, B, Sq, Skv, H, H, D)
    Wo = f16(rng.standard_normal((H * D, H * D)) * 0.05)
    bo = f16(rng.standard_normal(H * D) * 0.05)
    op = dthip.ScaledDotProductAttention(scale=1 / np.sqrt(D), multiHeadOutputProjectionFused=True)
    op.weight, op.bias = to_dev(torch, Wo), to_dev(torch, bo)
    print("sdpa fused out-proj", flush=True)
    got = op(to_dev(torch, q), to_dev(torch, k), to_dev(torch, v)).cpu().numpy()
    att = oracle.C.sdpa(q, k, v, 1 / np.sqrt(D)).reshape(B * Sq, H * D)
    want = oracle.C.dense(att, Wo, bo).reshape(B, Sq, H * D)
    mx, rr = oracle.err_stats(got, want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    # an output whose batches are padded apart takes the projection batch by batch: same numbers
    buf = torch.zeros((B, Sq + 3, H * D), dtype=torch.float16, device="cuda")
    dthip.sdpa_segments([to_dev(torch, q)], [to_dev(torch, k)], [to_dev(torch, v)], 1 / np.sqrt(D),
                        Wo=op.weight, bo=op.bias, out=buf[:, :Sq])
    assert np.array_equal(buf[:, :Sq].cpu().numpy(), got)
    assert float(buf[:, Sq:].abs().max()) == 0.0


def test_sdpa_rejects_bad_arguments(dthip, torch_cuda):
    torch = torch_cuda
    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
    with pytest.raises(dthip.DtError) as e:
        dthip.sdpa_segments([z(1, 8, 3, 64)], [z(1, 8, 2, 64)], [z(1, 8, 2, 64)], 1.0)  # 2 does not divide 3
    assert e.value.status == dthip.DT_INVALID
    with pytest.raises(dthip.DtError) as e:
        dthip.sdpa_segments([z(1, 8, 2, 136)], [z(1, 8, 2, 136)], [z(1, 8, 2, 136)], 1.0)  # D > 128
    assert e.value.status == dthip.DT_NO_KERNEL
    with pytest.raises(dthip.DtError) as e:
        dthip.sdpa_segments([z(1, 8, 2, 64)], [z(1, 0, 2, 64)], [z(1, 0, 2, 64)], 1.0)  # no keys
    assert e.value.status == dthip.DT_INVALID
    assert dthip.sdpa_segments([z(1, 0, 2, 64)], [z(1, 4, 2, 64)], [z(1, 4, 2, 64)], 1.0).shape == (1, 0, 2, 64)


def test_entry_points_run_past_a_stale_benign_runtime_error(dthip, oracle, torch_cuda):
    """A host that checks HIP return codes directly (as ccv does) leaves non-fatal codes in the thread's error slot:
    a rejected argument, a second hipDeviceEnablePeerAccess.  The entry points must not take such a leftover for a
    fault: they run, and their own launch status is what they return."""
    import ctypes

    torch = torch_cuda
    dthip.lib()
    hip = ctypes.CDLL("libamdhip64.so.7")  # the runtime already loaded in this process (same soname)
    for f in (hip.hipPeekAtLastError, hip.hipGetLastError):
        f.restype, f.argtypes = ctypes.c_int, []
    hip.hipMemcpy.restype = ctypes.c_int
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    hip.hipDeviceEnablePeerAccess.restype = ctypes.c_int
    hip.hipDeviceEnablePeerAccess.argtypes = [ctypes.c_int, ctypes.c_uint]
    torch.cuda.synchronize()
    hip.hipGetLastError()
    rng = np.random.default_rng(77)
    q, k, v = rand_qkv(rng, 1, 96, 80, 2, 2, 64)
    want = oracle.C.sdpa(q, k, v, 0.125)
    x = f16(rng.standard_normal((40, 64)))
    w = f16(rng.standard_normal((24, 64)) * 0.1)
    provoked = 0
    for provoke in (lambda: hip.hipMemcpy(None, None, 16, 3), lambda: hip.hipDeviceEnablePeerAccess(0, 0)):
        rc = provoke()
        if rc == 0 or hip.hipPeekAtLastError() == 0:
            continue  # this runtime does not keep that one
        provoked += 1
        print("stale runtime error left in place:", rc, flush=True)
        got = dthip.sdpa_segments([to_dev(torch, q)], [to_dev(torch, k)], [to_dev(torch, v)], 0.125)
        torch.cuda.synchronize()
        mx, rr = oracle.err_stats(got.cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
        assert hip.hipPeekAtLastError() == 0
        provoke()
        y = dthip.dense_multi(to_dev(torch, x), [dthip.QxTensor.from_f16(w)], [None])[0]
        torch.cuda.synchronize()
        mx, rr = oracle.err_stats(y.cpu().numpy(), oracle.C.dense(x, w, None))
        assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    assert provoked >= 1, "no benign runtime error could be provoked"


def test_sdpa_flux_full_size_sampled(dthip, oracle, torch_cuda):
    """Headline benchmark shape (1, 24 heads x 128, 512 text + 4096 image tokens): sampled rows of two heads against
    the oracle, and the constant-V property over the whole output."""
    torch = torch_cuda
    rng = np.random.default_rng(9)
    B, T, HW, H, D = 1, 512, 4096, 24, 128
    S = T + HW
    q, k, v = rand_qkv(rng, B, S, S, H, H, D)
    scale = 1 / np.sqrt(D)
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    print("sdpa full size", flush=True)
    got = dthip.sdpa_segments([qd[:, :T], qd[:, T:]], [kd[:, :T], kd[:, T:]], [vd[:, :T], vd[:, T:]], scale).cpu().numpy()
    rows = np.sort(rng.choice(S, size=48, replace=False))
    rows[0], rows[-1] = 0, S - 1
    for h in (0, 23):
        want = oracle.C.sdpa(np.ascontiguousarray(q[:, rows, h:h + 1]), np.ascontiguousarray(k[:, :, h:h + 1]),
                             np.ascontiguousarray(v[:, :, h:h + 1]), scale)
        mx, rr = oracle.err_stats(got[:, rows, h:h + 1], want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (h, mx, rr)
    vc = torch.from_numpy(f16(rng.standard_normal((1, 1, H, D)))).cuda().expand(B, S, H, D).contiguous()
    oc = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vc)
    assert float((oc.float() - vc.float()).abs().max()) <= 2e-3


def test_sdpa_flux_2048_full_size_sampled(dthip, oracle, torch_cuda):
    """Long-sequence Flux shape (512 text + 16384 image tokens, 24 heads x 128), text and image as two segments:
    sampled rows of two heads against the oracle, the constant-V property over the whole output, and the joint call
    equal to the call on the concatenated tensors."""
    torch = torch_cuda
    rng = np.random.default_rng(22)
    B, T, HW, H, D = 1, 512, 16384, 24, 128
    S = T + HW
    gen = torch.Generator(device="cuda").manual_seed(22)
    qd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    kd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    vd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    scale = 1 / np.sqrt(D)
    print("sdpa flux 2048 full size", flush=True)
    got = dthip.sdpa_segments([qd[:, :T], qd[:, T:]], [kd[:, :T], kd[:, T:]], [vd[:, :T], vd[:, T:]], scale)
    rows = np.sort(rng.choice(S, size=24, replace=False))
    rows[0], rows[1], rows[-1] = 0, T, S - 1
    rows = np.unique(rows)
    rt = torch.from_numpy(rows).cuda()
    for h in (0, 23):
        want = oracle.C.sdpa(np.ascontiguousarray(qd[:, rt, h:h + 1].cpu().numpy()), np.ascontiguousarray(kd[:, :, h:h + 1].cpu().numpy()),
                             np.ascontiguousarray(vd[:, :, h:h + 1].cpu().numpy()), scale)
        mx, rr = oracle.err_stats(got[:, rt, h:h + 1].cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (h, mx, rr)
    whole = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vd)
    assert torch.equal(got, whole)
    vc = torch.from_numpy(f16(rng.standard_normal((1, 1, H, D)))).cuda().expand(B, S, H, D).contiguous()
    oc = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vc)
    assert float((oc.float() - vc.float()).abs().max()) <= 2e-3


def test_sdpa_wan_full_size_sampled(dthip, oracle, torch_cuda):
    """The largest benchmark shape (1, 40 heads x 128, 32760 tokens; Q and K pre-scaled by D^-1/4 and scale 1, the
    `.scale1` convention of Models/Wan.swift:95-103): sampled rows of two heads against the oracle, the
    constant-V property over the whole output, and scale1 == scaleMerged on the sampled rows' neighbourhood."""
    torch = torch_cuda
    rng = np.random.default_rng(21)
    B, S, H, D = 1, 32760, 40, 128
    gen = torch.Generator(device="cuda").manual_seed(21)
    qd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    kd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    vd = torch.randn((B, S, H, D), device="cuda", generator=gen).half()
    s4 = float(D) ** -0.25
    q1, k1 = (qd.float() * s4).half(), (kd.float() * s4).half()
    print("sdpa wan full size", flush=True)
    got = dthip.ScaledDotProductAttention(scale=1.0)(q1, k1, vd)
    rows = np.sort(rng.choice(S, size=16, replace=False))
    rows[0], rows[-1] = 0, S - 1
    rt = torch.from_numpy(rows).cuda()
    for h in (0, 39):
        want = oracle.C.sdpa(np.ascontiguousarray(q1[:, rt, h:h + 1].cpu().numpy()), np.ascontiguousarray(k1[:, :, h:h + 1].cpu().numpy()),
                             np.ascontiguousarray(vd[:, :, h:h + 1].cpu().numpy()), 1.0)
        mx, rr = oracle.err_stats(got[:, rt, h:h + 1].cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (h, mx, rr)
    del got
    vc = torch.randn((1, 1, H, D), device="cuda", generator=gen).half().expand(B, S, H, D).contiguous()
    oc = dthip.ScaledDotProductAttention(scale=1.0)(q1, k1, vc)
    assert float((oc.float() - vc.float()).abs().max()) <= 2e-3


def test_block_step_replays_as_hip_graph(dthip, oracle, torch_cuda):
    """The three launches of a joint block (grouped QKV Dense with the fused norm / RoPE epilogue, attention, grouped
    out-projection) captured as one HIP graph: every replay, with eager runs and synchronisations in between,
    reproduces the eager result bit for bit (no call on this path allocates or clears memory behind the capture)."""
    torch = torch_cuda
    rng = np.random.default_rng(33)
    T, HW, H, D = 64, 320, 2, 128
    C, S = H * D, 64 + 320
    def mk():
        packed, _, _ = oracle.synth_qx_weight(rng, C, C, 6, 4096, 0.05)
        return dthip.QxTensor.from_packed(packed, 6, 4096, (C, C))
    w = {n: mk() for n in ("c_q", "c_k", "c_v", "x_q", "x_k", "x_v", "c_o", "x_o")}
    f = lambda shape, s=1.0: to_dev(torch, (rng.standard_normal(shape) * s).astype(np.float16))
    ctx, img = f((T, C)), f((HW, C))
    gam = {n: f((D,), 0.05) + 1 for n in ("c_q", "c_k", "x_q", "x_k")}
    rot = to_dev(torch, dthip.Flux1RotaryPositionEmbedding(16, 20, T, channels=D).astype(np.float16))
    qkv = torch.zeros((S, 3, H, D), dtype=torch.float16, device="cuda")
    att = torch.zeros((1, S, H, D), dtype=torch.float16, device="cuda")
    out_c = torch.zeros((T, C), dtype=torch.float16, device="cuda")
    out_x = torch.zeros((HW, C), dtype=torch.float16, device="cuda")
    qkv2 = qkv.view(S, 3 * C)
    views = lambda lo, hi: [qkv2[lo:hi, i * C:(i + 1) * C] for i in range(3)]
    epi = lambda a, b, pos: [dthip.HeadEpilogue(gam[a], rot, pos, 1e-6, D), dthip.HeadEpilogue(gam[b], rot, pos, 1e-6, D), None]
    att2 = att.view(S, C)

    def step():
        dthip.dense_grouped([
            dict(x=img, weights=[w["x_q"], w["x_k"], w["x_v"]], biases=[None] * 3, outs=views(T, S), epilogues=epi("x_q", "x_k", T)),
            dict(x=ctx, weights=[w["c_q"], w["c_k"], w["c_v"]], biases=[None] * 3, outs=views(0, T), epilogues=epi("c_q", "c_k", 0))])
        dthip.sdpa_segments([qkv[:, 0].unsqueeze(0)], [qkv[:, 1].unsqueeze(0)], [qkv[:, 2].unsqueeze(0)], 1 / np.sqrt(D), out=att)
        dthip.dense_grouped([dict(x=att2[T:], weights=[w["x_o"]], biases=[None], outs=[out_x]),
                             dict(x=att2[:T], weights=[w["c_o"]], biases=[None], outs=[out_c])])

    print("block step as hip graph", flush=True)
    step()
    torch.cuda.synchronize()
    want = (out_x.clone(), out_c.clone(), att.clone())
    assert float(want[0].abs().max()) > 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(4):
        out_x.zero_(); out_c.zero_(); att.zero_(); qkv.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for a_, b_ in zip((out_x, out_c, att), want):
            assert torch.equal(a_, b_)
        step()
        torch.cuda.synchronize()


@pytest.mark.parametrize("B,S,H,D", [(1, 1024, 2, 128), (2, 512, 8, 40), (1, 1536, 3, 128)])
def test_sdpa_vs_op_by_op_fp16_graph(dthip, oracle, torch_cuda, B, S, H, D):
    """The `.none` attention path of the reference (Matmul(transposeB:) -> softmax -> Matmul on fp16 tensors with the
    scale applied to Q first, Models/Flux1.swift:192-223, Models/UNet.swift:217-262) is what an op-by-op CPU run
    executes: scaled Q, scores and probabilities are each stored as fp16 between the three ops.  The fused kernel
    keeps them in fp32; the two must agree within the attention bar (max-abs 2e-2, rel-RMS 1e-3)."""
    torch = torch_cuda
    rng = np.random.default_rng(S + D)
    q, k, v = rand_qkv(rng, B, S, S, H, H, D)
    scale = 1 / np.sqrt(D)
    print("sdpa vs op-by-op graph", B, S, H, D, flush=True)
    got = dthip.ScaledDotProductAttention(scale=scale, flags=dthip.GEMMFlag.Float16)(
        to_dev(torch, q), to_dev(torch, k), to_dev(torch, v)).cpu().numpy()
    want = oracle.C.sdpa(q, k, v, scale, round_mid=1)
    mx, rr = oracle.err_stats(got, want)
    print("  gap to the op-by-op fp16 graph: max-abs %.3e rel-RMS %.3e" % (mx, rr), flush=True)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_sd15_full_size_sampled(dthip, oracle, torch_cuda):
    """SD 1.5 UNet attention at its full shape (batch 2, 8 heads x 40, 64 x 64 latent = 4096 tokens): self-attention
    over 4096 keys and cross-attention over 77 keys with the unify-heads projection fused
    (Models/UNet.swift:122-155, 311-319).  Sampled rows against the oracle, constant-V over the whole output."""
    torch = torch_cuda
    rng = np.random.default_rng(40)
    B, S, T, H, D = 2, 4096, 77, 8, 40
    scale = 1 / np.sqrt(D)
    q, k, v = rand_qkv(rng, B, S, S, H, H, D)
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    print("sdpa sd15 self full size", flush=True)
    got = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vd).cpu().numpy()
    rows = np.sort(rng.choice(S, size=40, replace=False))
    rows[0], rows[-1] = 0, S - 1
    want = oracle.C.sdpa(np.ascontiguousarray(q[:, rows]), k, v, scale)
    mx, rr = oracle.err_stats(got[:, rows], want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    vc = torch.from_numpy(f16(rng.standard_normal((1, 1, H, D)))).cuda().expand(B, S, H, D).contiguous()
    oc = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vc)
    assert float((oc.float() - vc.float()).abs().max()) <= 2e-3
    # cross-attention, 77 keys, fused output projection
    kc, vcx = f16(rng.standard_normal((B, T, H, D))), f16(rng.standard_normal((B, T, H, D)))
    Wo = f16(rng.standard_normal((H * D, H * D)) * 0.05)
    bo = f16(rng.standard_normal(H * D) * 0.05)
    op = dthip.ScaledDotProductAttention(scale=scale, multiHeadOutputProjectionFused=True)
    op.weight, op.bias = to_dev(torch, Wo), to_dev(torch, bo)
    print("sdpa sd15 cross full size, fused unify-heads", flush=True)
    gotc = op(qd, to_dev(torch, kc), to_dev(torch, vcx)).cpu().numpy()
    assert gotc.shape == (B, S, H * D)
    att = oracle.C.sdpa(np.ascontiguousarray(q[:, rows]), kc, vcx, scale).reshape(B * rows.size, H * D)
    wantc = oracle.C.dense(att, Wo, bo).reshape(B, rows.size, H * D)
    mx, rr = oracle.err_stats(gotc[:, rows], wantc)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_wan_cross_attention_full_size_sampled(dthip, oracle, torch_cuda):
    """Wan cross-attention at its full shape: 32760 query tokens against 512 text keys, 40 heads x 128, scale
    1/sqrt(128) (Models/Wan.swift:163-174).  Sampled rows of two heads against the oracle; constant-V property."""
    torch = torch_cuda
    rng = np.random.default_rng(41)
    B, Sq, Skv, H, D = 1, 32760, 512, 40, 128
    gen = torch.Generator(device="cuda").manual_seed(41)
    qd = torch.randn((B, Sq, H, D), device="cuda", generator=gen).half()
    kd = torch.randn((B, Skv, H, D), device="cuda", generator=gen).half()
    vd = torch.randn((B, Skv, H, D), device="cuda", generator=gen).half()
    scale = 1 / np.sqrt(D)
    print("sdpa wan cross full size", flush=True)
    got = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vd)
    rows = np.sort(rng.choice(Sq, size=64, replace=False))
    rows[0], rows[-1] = 0, Sq - 1
    rt = torch.from_numpy(rows).cuda()
    for h in (0, 17, 39):
        want = oracle.C.sdpa(np.ascontiguousarray(qd[:, rt, h:h + 1].cpu().numpy()), np.ascontiguousarray(kd[:, :, h:h + 1].cpu().numpy()),
                             np.ascontiguousarray(vd[:, :, h:h + 1].cpu().numpy()), scale)
        mx, rr = oracle.err_stats(got[:, rt, h:h + 1].cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (h, mx, rr)
    vc = torch.randn((1, 1, H, D), device="cuda", generator=gen).half().expand(B, Skv, H, D).contiguous()
    oc = dthip.ScaledDotProductAttention(scale=scale)(qd, kd, vc)
    assert float((oc.float() - vc[:, :1].float()).abs().max()) <= 2e-3


def test_qk_row_norm_rope_wan_full_size(dthip, oracle, torch_cuda):
    """Wan 14B at full size: RMSNorm(axis: [2]) over the 5120-wide row of all 32760 tokens, then the 3-axis rotation
    (table 21 x 30 x 52, dims 44 / 42 / 42) and the .scale1 pre-multiplication by 128^(-1/4), in place
    (Models/Wan.swift:87-98).  Sampled rows against the oracle, one fp16 ulp per stage."""
    torch = torch_cuda
    gt, gh, gw, H, D = 21, 30, 52, 40, 128
    S, C = gt * gh * gw, H * D
    assert S == 32760
    g = torch.Generator(device="cuda").manual_seed(5120)
    x = torch.randn((1, S, C), device="cuda", generator=g).half()
    gam = f16(1 + 0.02 * np.random.default_rng(3).standard_normal(C))
    rot = f16(dthip.WanRotaryPositionEmbedding(gh, gw, gt, channels=D))
    assert rot.shape == (S, D)
    rows = np.sort(np.unique(np.concatenate([[0, 1, S - 1, gh * gw - 1, gh * gw],
                                             np.random.default_rng(4).choice(S, size=27, replace=False)])))
    xs = x[0, torch.from_numpy(rows).cuda()].cpu().numpy()
    post = float(128 ** -0.25)
    print("row norm + rope at the Wan shape", flush=True)
    y = dthip.qk_norm_rope_(x.view(1, S, H, D), to_dev(torch, gam), 1e-6, False, rot=to_dev(torch, rot),
                            post_scale=post)
    got = y[0, torch.from_numpy(rows).cuda()].cpu().numpy()
    normed = oracle.C.rmsnorm(xs, gam, 1e-6).reshape(rows.size, H, D)
    rotated = oracle.C.cmul(normed, rot[rows])
    want = (rotated.astype(np.float32) * np.float32(post)).astype(np.float16)
    # one ulp per stage (norm, rotation, scale), on the scale of the rotated pair's magnitude
    pair = np.sqrt((rotated.astype(np.float64).reshape(rows.size, H, D // 2, 2) ** 2).sum(-1, keepdims=True))
    tol = 3 * (np.broadcast_to(pair, (rows.size, H, D // 2, 2)).reshape(rows.size, H, D) * post * 2.0 ** -10 + 2.0 ** -24)
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= tol)
    # the rest of the tensor was processed too: every row has unit RMS before gamma, so no element can be large
    assert bool(torch.isfinite(y.float()).all()) and float(y.float().abs().max()) < 40.0


def test_sdpa_wan_causal_chunked_windows(dthip, oracle, torch_cuda):
    """Wan causal inference (Models/Wan.swift:104-127): the frames are attended in chunks; query chunk i (rows
    [i * frames, (i + 1) * frames)) sees the key / value prefix of min(hw, (i + 1) * frames + padFrames) rows.  Each
    chunk is one call on offset views of the same [1, hw, h, k] tensors, its output written into its slice of one
    buffer (the reference's Concat(axis: 1))."""
    torch = torch_cuda
    rng = np.random.default_rng(104)
    time_, per_frame, H, D = 7, 90, 3, 128       # 7 latent frames of 90 tokens
    causal, pad = 2, 1                            # chunks of 2 frames, one frame of look-ahead
    hw = time_ * per_frame
    frames, pad_frames = per_frame * causal, per_frame * pad
    q, k, v = rand_qkv(rng, 1, hw, hw, H, H, D)
    # the .scale1 convention: queries and keys pre-multiplied by 128^(-1/4), scale 1
    q *= np.float16(128 ** -0.25)
    k *= np.float16(128 ** -0.25)
    scale = 1.0
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    out = torch.full((1, hw, H, D), float("nan"), dtype=torch.float16, device="cuda")
    n_chunks = (time_ + causal - 1) // causal
    print("wan causal windows", n_chunks, "chunks", flush=True)
    for i in range(n_chunks):
        lo, hi = i * frames, min(hw, (i + 1) * frames)
        kv = min(hw, (i + 1) * frames + pad_frames)
        dthip.sdpa_segments([qd[:, lo:hi]], [kd[:, :kv]], [vd[:, :kv]], scale, out=out[:, lo:hi])
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.isfinite(got.astype(np.float32)).all()
    for i in range(n_chunks):
        lo, hi = i * frames, min(hw, (i + 1) * frames)
        kv = min(hw, (i + 1) * frames + pad_frames)
        want = oracle.C.sdpa(np.ascontiguousarray(q[:, lo:hi]), np.ascontiguousarray(k[:, :kv]),
                             np.ascontiguousarray(v[:, :kv]), scale)
        mx, rr = oracle.err_stats(got[:, lo:hi], want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)
    # the windows matter: the first chunk's rows differ from full (non-causal) attention over all frames
    full = oracle.C.sdpa(np.ascontiguousarray(q[:, :frames]), k, v, scale)
    assert float(np.abs(full.astype(np.float32) - got[:, :frames].astype(np.float32)).max()) > 1e-2


# ------------------------------------------------------------------ K3, key-split form

SPLIT_CASES = [
    # B, Sq, Skv, Hq, Hk, D, scale sign
    (1, 300, 1000, 2, 2, 128, 1),     # ragged queries and keys, tasks cut into up to 8 pieces
    (2, 256, 640, 3, 3, 128, 1),      # whole tiles; runs that span several tasks
    (1, 70, 777, 8, 8, 40, 1),        # head size 40 (padded to 64)
    (1, 130, 1900, 4, 2, 64, 1),      # grouped heads
    (1, 520, 2100, 1, 1, 128, -1),    # a scale the kernel folds into the scores first (negative)
    (1, 1, 300, 1, 1, 128, 1),        # one query row, five key tiles in two pieces
]


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hk,D,sign", SPLIT_CASES)
def test_sdpa_key_split_vs_oracle(dthip, oracle, torch_cuda, monkeypatch, B, Sq, Skv, Hq, Hk, D, sign):
    """The key-split form of the kernel (a task's key tiles shared out over several workgroups, partial results
    folded by the piece that finishes last), forced on small shapes: against the oracle, against the unsplit
    kernel, and twice in a row (the fold order is fixed, so the result may not depend on the order of arrival)."""
    torch = torch_cuda
    rng = np.random.default_rng(B * 1000 + Sq + Skv + D)
    q, k, v = rand_qkv(rng, B, Sq, Skv, Hq, Hk, D)
    scale = sign / np.sqrt(D)
    want = oracle.C.sdpa(q, k, v, scale)
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "always")
    assert dthip.lib().dt_sdpa_workspace_bytes(B, Hq, Hk, D, Sq, Skv, 0, 0) > 0  # the split is in force
    print("sdpa key split", B, Sq, Skv, Hq, Hk, D, sign, flush=True)
    got = dthip.sdpa_segments([qd], [kd], [vd], scale)
    again = dthip.sdpa_segments([qd], [kd], [vd], scale)
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "never")
    assert dthip.lib().dt_sdpa_workspace_bytes(B, Hq, Hk, D, Sq, Skv, 0, 0) == 0
    plain = dthip.sdpa_segments([qd], [kd], [vd], scale)
    torch.cuda.synchronize()
    mx, rr = oracle.err_stats(got.cpu().numpy(), want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    assert torch.equal(got, again)
    # same arithmetic up to the fp32 fold of the pieces: a rounding step of the fp16 result at most
    assert float((got.float() - plain.float()).abs().max()) <= 2e-3


def test_sdpa_key_split_joint_segments_fused_prep(dthip, oracle, torch_cuda, monkeypatch):
    """Key-split with text || image segments, fused per-head RMSNorm + RoPE staging and the static-scratch entry
    point: all three forms agree bit for bit with each other and with the oracle within the attention bar."""
    torch = torch_cuda
    rng = np.random.default_rng(431)
    T, h, w, H, D = 70, 24, 20, 3, 128
    HW = h * w
    segs = {n: (f16(rng.standard_normal((1, T, H, D))), f16(rng.standard_normal((1, HW, H, D)))) for n in "qkv"}
    gam = {n: (f16(1 + 0.05 * rng.standard_normal(D)), f16(1 + 0.05 * rng.standard_normal(D))) for n in "qk"}
    rot = f16(dthip.Flux1RotaryPositionEmbedding(h, w, T, channels=D))
    scale = 1 / np.sqrt(D)
    dev = lambda a: to_dev(torch, a)
    args = dict(q_segs=[dev(t) for t in segs["q"]], k_segs=[dev(t) for t in segs["k"]],
                v_segs=[dev(t) for t in segs["v"]], scale=scale, gamma_q=[dev(g) for g in gam["q"]],
                gamma_k=[dev(g) for g in gam["k"]], rot_q=dev(rot), rot_k=dev(rot))

    def prep(n):
        parts = [oracle.C.rmsnorm(segs[n][i][0], gam[n][i], 1e-6) for i in range(2)]
        return oracle.C.cmul(np.concatenate(parts, axis=0), rot)[None]

    want = oracle.C.sdpa(prep("q"), prep("k"), np.concatenate(segs["v"], axis=1), scale)
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "always")
    print("sdpa key split, joint segments with fused prep", flush=True)
    got = dthip.sdpa_segments(**args)
    got_static = dthip.sdpa_segments(**args, static_scratch=True)
    # without the staging pass: two segments straight into the split kernel
    plain_args = dict(q_segs=args["q_segs"], k_segs=args["k_segs"], v_segs=args["v_segs"], scale=scale)
    seg_split = dthip.sdpa_segments(**plain_args)
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "never")
    seg_plain = dthip.sdpa_segments(**plain_args)
    torch.cuda.synchronize()
    mx, rr = oracle.err_stats(got.cpu().numpy(), want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)
    assert torch.equal(got, got_static)
    assert float((seg_split.float() - seg_plain.float()).abs().max()) <= 2e-3


def test_sdpa_key_split_by_its_own_estimate(dthip, oracle, torch_cuda, monkeypatch):
    """A launch that fills a quarter of the card (4 heads x 4096 tokens: 64 workgroups of 64 key tiles) is split
    without being told to; sampled rows against the oracle."""
    torch = torch_cuda
    monkeypatch.delenv("DT_SDPA_KEY_SPLIT", raising=False)
    B, S, H, D = 1, 4096, 4, 128
    assert dthip.lib().dt_sdpa_workspace_bytes(B, H, H, D, S, S, 0, 0) > 0
    assert dthip.lib().dt_sdpa_workspace_bytes(1, 24, 24, D, 4608, 4608, 0, 0) == 0  # the Flux shape is not
    rng = np.random.default_rng(4096)
    q, k, v = rand_qkv(rng, B, S, S, H, H, D)
    scale = 1 / np.sqrt(D)
    print("sdpa key split by estimate", flush=True)
    got = dthip.sdpa_segments([to_dev(torch, q)], [to_dev(torch, k)], [to_dev(torch, v)], scale).cpu().numpy()
    rows = np.sort(rng.choice(S, size=40, replace=False))
    rows[0], rows[-1] = 0, S - 1
    want = oracle.C.sdpa(np.ascontiguousarray(q[:, rows]), k, v, scale)
    mx, rr = oracle.err_stats(got[:, rows], want)
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_quantized_level_flags_are_permissions(dthip, oracle, torch_cuda):
    """FlashAttentionLevel.quantized builds ScaledDotProductAttention(scale:, flags: [.Int8, .Float16])
    (Models/Flux1.swift:228-232): the flags permit lower precision, they do not ask for it, so the call is served by
    the fp16 kernel -- the same bits as with [.Float16], inside the attention bar of the oracle."""
    torch = torch_cuda
    rng = np.random.default_rng(229)
    q, k, v = rand_qkv(rng, 1, 300, 520, 3, 3, 128)
    scale = 1 / np.sqrt(128)
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    f16_only = dthip.ScaledDotProductAttention(scale=scale, flags=dthip.GEMMFlag.Float16)(qd, kd, vd)
    quantized = dthip.ScaledDotProductAttention(scale=scale, flags=dthip.GEMMFlag.Int8 | dthip.GEMMFlag.Float16)(qd, kd, vd)
    assert torch.equal(f16_only, quantized)
    mx, rr = oracle.err_stats(quantized.cpu().numpy(), oracle.C.sdpa(q, k, v, scale))
    assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_sdpa_key_split_replays_as_hip_graph(dthip, oracle, torch_cuda, monkeypatch):
    """A key-split attention launch (counter reset by a fill kernel, partial results through the workspace, fold by
    the last piece to arrive) captured in a HIP graph with fused query / key prep: every replay, with eager calls
    and synchronisations in between and the outputs cleared each time, gives the eager result bit for bit."""
    torch = torch_cuda
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "always")
    rng = np.random.default_rng(911)
    B, S, H, D = 1, 1500, 3, 128
    q, k, v = rand_qkv(rng, B, S, S, H, H, D)
    g = to_dev(torch, f16(1 + 0.05 * rng.standard_normal(D)))
    rot = to_dev(torch, f16(dthip.WanRotaryPositionEmbedding(1, S, 1, channels=D)))
    qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
    out = torch.zeros((B, S, H, D), dtype=torch.float16, device="cuda")
    call = lambda: dthip.sdpa_segments([qd], [kd], [vd], 1 / np.sqrt(D), gamma_q=[g], gamma_k=[g], rot_q=rot, rot_k=rot,
                                       out=out)
    print("key-split attention as hip graph", flush=True)
    call()
    torch.cuda.synchronize()
    want = out.clone()
    assert float(want.abs().max()) > 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for _ in range(4):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        call()  # eager work between the replays
        torch.cuda.synchronize()
