"""GPU parity on randomly drawn shapes: Dense (every index width, block size, ragged tiles, strided rows, several
weights per launch), attention (grouped heads, several segments on either side, ragged lengths, every head size) and
the norm / RoPE pass (aligned and unaligned views, every head size), each against the CPU oracle through the C ABI.
Seeded: the cases are the same on every run."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 2e-2, 1e-3
N_CASES = 40


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available()
    return torch


def f16(a):
    return np.asarray(a, dtype=np.float16)


def to_dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_dense_random_shapes(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(101)
    for i in range(N_CASES):
        q = int(rng.choice([4, 5, 6, 7, 8, 16]))
        nib = int(rng.choice([32, 64, 512, 1024, 4096, 16384]))
        K = int(rng.choice([64, 128, 192, 320, 512, 768, 1024, 1536]))
        if rng.random() < 0.15:
            K = int(rng.integers(1, 20)) * 8 + int(rng.choice([0, 4]))  # off the tiled kernel's granule
        M = int(rng.choice([1, 7, 64, 127, 128, 129, 255, 256, 300, 511, 1024, 1100, 2049]))
        Ns = [int(rng.choice([8, 70, 128, 129, 256, 320, 384, 520])) for _ in range(int(rng.choice([1, 1, 2, 3])))]
        ldx = K + int(rng.choice([0, 0, 8, 24]))
        print("dense", i, q, nib, M, K, Ns, ldx, flush=True)
        Xb = f16(rng.standard_normal((M, ldx)))
        X = np.ascontiguousarray(Xb[:, :K])
        ws, wants, biases = [], [], []
        for N in Ns:
            b = f16(rng.standard_normal(N) * 0.05) if rng.random() < 0.7 else None
            if q == 16:
                W = f16(rng.standard_normal((N, K)) * 0.05)
                ws.append(dthip.QxTensor.from_f16(W))
                wants.append(oracle.C.dense(X, W, b))
            else:
                packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 0.05)
                ws.append(dthip.QxTensor.from_packed(packed, q, nib, (N, K)))
                wants.append(oracle.C.dense_qx(X, packed, q, nib, N, b))
            biases.append(None if b is None else to_dev(torch, b))
        outs = dthip.dense_multi(to_dev(torch, Xb)[:, :K], ws, biases)
        for o, want in zip(outs, wants):
            mx, rr = oracle.err_stats(o.cpu().numpy(), want)
            assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)


def test_sdpa_random_shapes(dthip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(102)
    for i in range(N_CASES):
        D = int(rng.choice([40, 64, 128, 128, 32, 80]))
        Hk = int(rng.choice([1, 2, 3]))
        Hq = Hk * int(rng.choice([1, 1, 2, 4]))
        B = int(rng.choice([1, 1, 2]))
        ql = [int(rng.choice([1, 5, 64, 100, 256, 300, 700])) for _ in range(int(rng.choice([1, 1, 2, 3])))]
        kl = [int(rng.choice([1, 3, 63, 64, 65, 77, 128, 200, 513])) for _ in range(int(rng.choice([1, 1, 2, 3])))]
        print("sdpa", i, B, Hq, Hk, D, ql, kl, flush=True)
        q = f16(rng.standard_normal((B, sum(ql), Hq, D)) * rng.choice([1.0, 3.0]))
        k = f16(rng.standard_normal((B, sum(kl), Hk, D)))
        v = f16(rng.standard_normal((B, sum(kl), Hk, D)))
        scale = float(1 / np.sqrt(D))

        def split(t, lens):
            out, p = [], 0
            for n in lens:
                out.append(t[:, p:p + n])
                p += n
            return out

        qd, kd, vd = (to_dev(torch, t) for t in (q, k, v))
        got = dthip.sdpa_segments(split(qd, ql), split(kd, kl), split(vd, kl), scale).cpu().numpy()
        want = oracle.C.sdpa(q, np.repeat(k, Hq // Hk, axis=2), np.repeat(v, Hq // Hk, axis=2), scale)
        mx, rr = oracle.err_stats(got, want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (i, mx, rr)


def test_norm_rope_random_shapes(dthip, oracle, torch_cuda):
    """In place on a view that starts `off` elements into each row of a wider buffer.  A rotated pair is compared on
    the scale of the pair's magnitude (the rotation keeps it; a component can cancel to far less): one fp16 ulp per
    stage (norm, rotation)."""
    torch = torch_cuda
    rng = np.random.default_rng(103)
    for i in range(N_CASES):
        D = int(rng.choice([32, 40, 64, 128, 96, 2, 120]))
        H = int(rng.choice([1, 3, 8, 24]))
        S = int(rng.choice([1, 9, 64, 333]))
        B = int(rng.choice([1, 2]))
        off = int(rng.choice([0, 0, 2, 8]))
        use_g, use_r = rng.random() < 0.8, rng.random() < 0.8
        print("norm rope", i, B, S, H, D, off, use_g, use_r, flush=True)
        buf = f16(rng.standard_normal((B, S, H * D + off)))
        g = f16(1 + 0.05 * rng.standard_normal(D))
        th = rng.uniform(-3, 3, size=(S + 4, D // 2))
        rot = np.empty((S + 4, D), np.float16)
        rot[:, 0::2], rot[:, 1::2] = np.cos(th), np.sin(th)
        d = to_dev(torch, buf)
        dthip.qk_norm_rope_(d[:, :, off:].unflatten(2, (H, D)), to_dev(torch, g) if use_g else None, 1e-6, True,
                            rot=to_dev(torch, rot) if use_r else None, rot_pos0=3)
        got = d.cpu().numpy()
        assert np.array_equal(got[:, :, :off], buf[:, :, :off])
        x = np.ascontiguousarray(buf[:, :, off:]).reshape(B, S, H, D)
        for b in range(B):
            w = x[b]
            if use_g:
                w = oracle.C.rmsnorm(w, g, 1e-6)
            if use_r:
                w = oracle.C.cmul(w, rot[3:3 + S])
            wf = w.astype(np.float32)
            mag = np.sqrt(wf[..., 0::2] ** 2 + wf[..., 1::2] ** 2)
            # one fp16 ulp per stage: where the normalised value lies on a rounding tie (to within the fp32 evaluation)
            # the device and the oracle may round it apart, and the rotation carries that ulp into its result
            stages = 2.0 if (use_g and use_r) else 1.0
            tol = np.repeat(np.maximum(mag * 2.0 ** -10, 2.0 ** -14), 2, axis=-1) * stages
            diff = np.abs(got[b, :, off:].reshape(S, H, D).astype(np.float32) - wf)
            assert (diff <= tol).all(), (i, float((diff / tol).max()))


def _weight(dthip, oracle, rng, N, K, q, nib):
    if q == 16:
        return dthip.QxTensor.from_f16(f16(rng.standard_normal((N, K)) * 0.05))
    packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 0.05)
    return dthip.QxTensor.from_packed(packed, q, nib, (N, K))


def _ulps(a, b):
    ai, bi = a.view(np.int16).astype(np.int32), b.view(np.int16).astype(np.int32)
    ai = np.where(ai < 0, -32768 - ai, ai)
    bi = np.where(bi < 0, -32768 - bi, bi)
    return int(np.abs(ai - bi).max())


def test_dense_tails_random_shapes(dthip, oracle, torch_cuda):
    """Activation, gate and fp32 residual in the Dense epilogue on random shapes, against numpy on the device's own
    plain Dense result: the fp16 output within one ulp per rounded step that follows an activation (exact without
    one), the residual stream within the rounding of its addition."""
    torch = torch_cuda
    rng = np.random.default_rng(104)
    acts = {dthip.ACT_NONE: lambda y: y, dthip.ACT_GELU_TANH: oracle.np_gelu_tanh16, dthip.ACT_SWISH: oracle.np_swish16,
            dthip.ACT_GELU_ERF: oracle.np_gelu_erf16}
    for i in range(N_CASES):
        q = int(rng.choice([4, 5, 6, 8, 16]))
        nib = int(rng.choice([64, 512, 1024, 4096, 16384]))
        K = int(rng.choice([64, 128, 192, 320, 512, 1024]))
        M = int(rng.choice([1, 64, 127, 129, 256, 300, 1024, 1100, 2049]))
        N = int(rng.choice([8, 72, 128, 256, 384, 520]))
        act = int(rng.choice(list(acts)))
        use_gate, use_res = rng.random() < 0.5, rng.random() < 0.6
        keep = (rng.random() < 0.7) or not use_res
        print("dense tail", i, q, nib, M, K, N, act, use_gate, use_res, keep, flush=True)
        w = _weight(dthip, oracle, rng, N, K, q, nib)
        xd = to_dev(torch, f16(rng.standard_normal((M, K))))
        bd = to_dev(torch, f16(rng.standard_normal(N) * 0.1))
        gate = f16(1 + 0.3 * rng.standard_normal(N))
        res0 = rng.standard_normal((M, N)).astype(np.float32)
        plain = dthip.dense_multi(xd, [w], [bd])[0].cpu().numpy()
        res = torch.from_numpy(res0.copy()).cuda() if use_res else None
        o = dthip.dense_post(xd, [w], [bd], [dthip.DensePost(act, gate=to_dev(torch, gate) if use_gate else None,
                                                              residual=res, keep_output=keep)])[0]
        y = acts[act](plain)
        if use_gate:
            y = (y.astype(np.float32) * gate.astype(np.float32)[None, :]).astype(np.float16)
        if keep:
            allowed = 0 if act == dthip.ACT_NONE else (2 if use_gate else 1)
            assert _ulps(o.cpu().numpy(), y) <= allowed, i
        else:
            assert o is None
        if use_res:
            err = np.max(np.abs(res.cpu().numpy() - (res0 + y.astype(np.float32))))
            assert err <= 2.0 ** -9 * max(1.0, float(np.abs(y.astype(np.float32)).max())), (i, err)


def test_dense_fused_heads_random_shapes(dthip, oracle, torch_cuda):
    """Per-head RMSNorm + RoPE behind the projection (in the GEMM epilogue for 128-wide heads, as a pass after it
    otherwise) on random shapes, against the oracle's norm and rotation of the device's own plain Dense result.
    Two fp16 ulps of a pair's magnitude: one for a rounding of the normalised value that falls the other way (the
    sums of squares are added in another order), which the rotation then carries into both components."""
    torch = torch_cuda
    rng = np.random.default_rng(105)
    for i in range(N_CASES):
        q = int(rng.choice([4, 5, 6, 8, 16]))
        nib = int(rng.choice([64, 512, 1024, 4096, 16384]))
        K = int(rng.choice([64, 128, 192, 320, 512, 1024]))
        M = int(rng.choice([1, 64, 127, 129, 256, 300, 1024, 1100, 2049]))
        hd = int(rng.choice([128, 128, 64, 40]))
        H = int(rng.choice([1, 2, 3]))
        N, pos0 = H * hd, int(rng.choice([0, 5]))
        print("dense heads", i, q, nib, M, K, hd, H, flush=True)
        ws = [_weight(dthip, oracle, rng, N, K, q, nib) for _ in range(3)]
        bs = [to_dev(torch, f16(rng.standard_normal(N) * 0.05)) for _ in range(3)]
        gs = [f16(1 + 0.05 * rng.standard_normal(hd)) for _ in range(2)]
        th = rng.uniform(-3, 3, size=(pos0 + M, hd // 2))
        rot = np.empty((pos0 + M, hd), np.float16)
        rot[:, 0::2], rot[:, 1::2] = np.cos(th), np.sin(th)
        rd = to_dev(torch, rot)
        use = [(True, True), (rng.random() < 0.7, rng.random() < 0.8)]
        epi = [dthip.HeadEpilogue(to_dev(torch, gs[j]) if use[j][0] else None, rd if use[j][1] else None, pos0, 1e-6, hd)
               for j in range(2)] + [None]
        xd = to_dev(torch, f16(rng.standard_normal((M, K))))
        outs = dthip.dense_multi(xd, ws, bs, epilogues=epi)
        plain = dthip.dense_multi(xd, ws, bs)
        assert torch.equal(outs[2], plain[2])
        for j in range(2):
            y = plain[j].cpu().numpy().reshape(M, H, hd)
            if use[j][0]:
                y = oracle.C.rmsnorm(y, gs[j], 1e-6)
            if use[j][1]:
                y = oracle.C.cmul(y, rot[pos0:pos0 + M])
            wf = y.astype(np.float32)
            mag = np.sqrt(wf[..., 0::2] ** 2 + wf[..., 1::2] ** 2)
            tol = np.repeat(np.maximum(mag * 2.0 ** -9, 2.0 ** -14), 2, axis=-1)
            diff = np.abs(outs[j].cpu().numpy().reshape(M, H, hd).astype(np.float32) - wf)
            assert (diff <= tol).all(), (i, j, float((diff / tol).max()))


def test_sdpa_segments_prep_and_key_split_random(dthip, oracle, torch_cuda, monkeypatch):
    """Attention over random segment lists with every optional stage drawn at random -- per-segment norm weights on
    the query side (applied inside the kernel) and on the key side (staged), rotation tables on either side, grouped
    heads, head sizes from 8 to 128, positive and negative scales, the key-split form forced on, forced off or left
    to the library's estimate, the caller's workspace or the static scratch -- against the oracle's
    RMSNorm -> cmul -> attention chain."""
    torch = torch_cuda
    rng = np.random.default_rng(106)
    for i in range(60):
        D = int(rng.choice([40, 64, 128, 128, 128, 32, 16, 8, 24]))
        Hk = int(rng.integers(1, 4))
        Hq = Hk * int(rng.choice([1, 1, 2, 3]))
        B = int(rng.choice([1, 1, 2]))
        qlens = [int(rng.integers(1, 400)) for _ in range(int(rng.integers(1, 4)))]
        klens = [int(rng.integers(1, 900)) for _ in range(int(rng.integers(1, 4)))]
        Sq, Skv = sum(qlens), sum(klens)
        q = [f16(rng.standard_normal((B, n, Hq, D))) for n in qlens]
        k = [f16(rng.standard_normal((B, n, Hk, D))) for n in klens]
        v = [f16(rng.standard_normal((B, n, Hk, D))) for n in klens]
        use_gq, use_gk = rng.random() < 0.6, rng.random() < 0.4
        gq = [f16(1 + 0.05 * rng.standard_normal(D)) if use_gq and rng.random() < 0.8 else None for _ in qlens]
        gk = [f16(1 + 0.05 * rng.standard_normal(D)) if use_gk and rng.random() < 0.8 else None for _ in klens]
        rot = f16(dthip.WanRotaryPositionEmbedding(1, max(Sq, Skv), 1, channels=D)) if D % 16 == 0 and rng.random() < 0.6 else None
        rot_q = rot if rot is not None and rng.random() < 0.8 else None
        rot_k = rot if rot is not None and rng.random() < 0.6 else None
        scale = float(rng.choice([1 / np.sqrt(D), 0.07, -0.05]))
        mode = str(rng.choice(["always", "never", "auto"]))
        static = bool(rng.random() < 0.3)
        if mode == "auto":
            monkeypatch.delenv("DT_SDPA_KEY_SPLIT", raising=False)
        else:
            monkeypatch.setenv("DT_SDPA_KEY_SPLIT", mode)
        print("sdpa segments", i, B, qlens, klens, Hq, Hk, D, use_gq, use_gk, rot_q is not None, rot_k is not None,
              round(scale, 3), mode, static, flush=True)

        def prep(parts, gs, r, S):
            out = []
            for b in range(B):
                rows = np.concatenate([p[b] if g is None else oracle.C.rmsnorm(p[b], g, 1e-6) for p, g in zip(parts, gs)])
                out.append(rows if r is None else oracle.C.cmul(rows, r[:S]))
            return np.stack(out)

        want = oracle.C.sdpa(prep(q, gq, rot_q, Sq), prep(k, gk, rot_k, Skv), np.concatenate(v, axis=1), scale)
        dev = lambda a: None if a is None else to_dev(torch, a)
        got = dthip.sdpa_segments([dev(t) for t in q], [dev(t) for t in k], [dev(t) for t in v], scale,
                                  gamma_q=[dev(g) for g in gq] if any(g is not None for g in gq) else None,
                                  gamma_k=[dev(g) for g in gk] if any(g is not None for g in gk) else None,
                                  rot_q=dev(rot_q), rot_k=dev(rot_k), static_scratch=static)
        mx, rr = oracle.err_stats(got.cpu().numpy(), want)
        assert mx <= 2e-2 and rr <= 1e-3, (i, mx, rr)


def test_dense_large_palettes_tall_tile_random(dthip, oracle, torch_cuda):
    """128- and 256-entry palettes with small blocks on problems large enough for the 256-token x 128-feature tile
    (per-row palette tables, weight staging by one wave per SIMD): random ragged shapes against the oracle."""
    torch = torch_cuda
    rng = np.random.default_rng(107)
    for i in range(12):
        q = int(rng.choice([7, 8]))
        nib = int(rng.choice([64, 512, 1024, 4096]))
        K = int(rng.choice([128, 256, 512, 768]))
        M = int(rng.integers(2300, 3100))
        N = int(rng.integers(2200, 2600))
        print("dense tall tile", i, q, nib, M, K, N, flush=True)
        packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 0.05)
        w = dthip.QxTensor.from_packed(packed, q, nib, (N, K))
        x = f16(rng.standard_normal((M, K)))
        b = f16(rng.standard_normal(N) * 0.05) if rng.random() < 0.7 else None
        got = dthip.dense_multi(to_dev(torch, x), [w], [None if b is None else to_dev(torch, b)])[0].cpu().numpy()
        mx, rr = oracle.err_stats(got, oracle.C.dense_qx(x, packed, q, nib, N, b))
        assert mx <= 2e-2 and rr <= 1e-3, (i, mx, rr)
