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
    the scale of the pair's magnitude (the rotation keeps it; a component can cancel to far less): one fp16 ulp."""
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
            tol = np.repeat(np.maximum(mag * 2.0 ** -10, 2.0 ** -14), 2, axis=-1)
            diff = np.abs(got[b, :, off:].reshape(S, H, D).astype(np.float32) - wf)
            assert (diff <= tol).all(), (i, float((diff / tol).max()))
