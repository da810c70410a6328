"""The entry point that allocates nothing (dt_sdpa_f16_static: attention staged through the library's fixed per-GPU
array) against dt_sdpa_f16 with a caller's workspace, through the C ABI: two calls in a row, the second smaller, each
bit-identical to the existing entry point's output and within the attention bar of the oracle.  Collected last."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 2e-2, 1e-3


def _case(dthip, oracle, torch, rng, T, h, w, H, D, fused_out):
    """Joint text || image attention with fused per-head RMSNorm + RoPE (workspace: staged K), or SD 1.5 style
    attention with the fused unify-heads projection (workspace: staged attention output)."""
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    f16 = lambda a: np.asarray(a, dtype=np.float16)
    HW = h * w
    scale = 1 / np.sqrt(D)
    if fused_out:
        q = f16(rng.standard_normal((2, HW, H, D)))
        k = f16(rng.standard_normal((2, T, H, D)))
        v = f16(rng.standard_normal((2, T, H, D)))
        Wo = f16(rng.standard_normal((H * D, H * D)) * 0.05)
        bo = f16(rng.standard_normal(H * D) * 0.05)
        args = dict(q_segs=[dev(q)], k_segs=[dev(k)], v_segs=[dev(v)], scale=scale, Wo=dev(Wo), bo=dev(bo))
        att = oracle.C.sdpa(q, k, v, scale).reshape(2 * HW, H * D)
        want = oracle.C.dense(att, Wo, bo).reshape(2, HW, H * D)
        shape = (2, HW, H * D)
    else:
        segs = {n: (f16(rng.standard_normal((1, T, H, D))), f16(rng.standard_normal((1, HW, H, D)))) for n in "qkv"}
        gam = {n: (f16(1 + 0.05 * rng.standard_normal(D)), f16(1 + 0.05 * rng.standard_normal(D))) for n in "qk"}
        rot = f16(dthip.Flux1RotaryPositionEmbedding(h, w, T, channels=D))
        args = dict(q_segs=[dev(t) for t in segs["q"]], k_segs=[dev(t) for t in segs["k"]],
                    v_segs=[dev(t) for t in segs["v"]], scale=scale, gamma_q=[dev(g) for g in gam["q"]],
                    gamma_k=[dev(g) for g in gam["k"]], rot_q=dev(rot), rot_k=dev(rot))

        def prep(n):
            parts = [oracle.C.rmsnorm(segs[n][i][0], gam[n][i], 1e-6) for i in range(2)]
            return oracle.C.cmul(np.concatenate(parts, axis=0), rot)[None]

        want = oracle.C.sdpa(prep("q"), prep("k"), np.concatenate(segs["v"], axis=1), scale)
        shape = (1, T + HW, H, D)
    return args, want, shape


@pytest.mark.parametrize("fused_out", [False, True])
def test_static_scratch_entry_point_matches_workspace_entry_point(dthip, oracle, fused_out):
    import torch

    assert torch.cuda.is_available()
    assert dthip.lib().dt_init(0) == 0
    rng = np.random.default_rng(70 + int(fused_out))
    # two calls in a row on one stream; the second is smaller, so the array still holds the first call's bytes beyond it
    sizes = [(70, 24, 20, 3, 128), (33, 9, 10, 2, 64)] if not fused_out else [(77, 32, 32, 8, 40), (50, 12, 11, 4, 64)]
    cases = [_case(dthip, oracle, torch, rng, *sz, fused_out) for sz in sizes]
    outs = [torch.full(shape, float("nan"), dtype=torch.float16, device="cuda") for _, _, shape in cases]
    # the existing entry point first, workspace allocated by the caller (in a fresh process this is also what makes
    # the runtime load the kernels' code objects, which takes device memory once)
    refs = [dthip.sdpa_segments(**args) for args, _, _ in cases]
    torch.cuda.synchronize()
    # torch's own count sees its caching allocator only; the driver's free-byte count sees any hipMalloc / hipFree
    # that the library itself might make
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    for (args, _, _), out in zip(cases, outs):
        print("static scratch call", tuple(out.shape), "fused_out" if fused_out else "fused_prep", flush=True)
        dthip.sdpa_segments(**args, out=out, static_scratch=True)
    assert torch.cuda.memory_allocated() == before  # the host mirror allocated nothing either
    assert torch.cuda.mem_get_info()[0] == free_before  # nor did the library, behind torch's back
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for (args, want, _), out, ref in zip(cases, outs, refs):
        assert torch.equal(out, ref)
        mx, rr = oracle.err_stats(out.cpu().numpy(), want)
        assert mx <= MAX_ABS and rr <= REL_RMS, (mx, rr)


def test_static_scratch_rejects_requests_beyond_the_array(dthip):
    import torch

    B, S, H, D = 1, 12000, 24, 128   # staged K: 12000 * 24 * 128 * 2 B = 73.7 MB > 64 MiB
    q = torch.zeros((B, S, H, D), dtype=torch.float16, device="cuda")
    g = torch.ones(D, dtype=torch.float16, device="cuda")
    assert dthip.lib().dt_sdpa_workspace_bytes(B, H, H, D, S, S, 1, 0) > dthip.STATIC_SCRATCH_BYTES
    print("static scratch: request beyond the array", flush=True)
    with pytest.raises(dthip.DtError) as e:
        dthip.sdpa_segments([q], [q], [q], 1.0, gamma_q=[g], gamma_k=[g], static_scratch=True)
    assert e.value.status == dthip.DT_OOM
    # without staging the same shapes need no scratch at all and run
    o = dthip.sdpa_segments([q[:, :256]], [q[:, :256]], [q[:, :256]], 1.0, static_scratch=True)
    assert o.shape == (B, 256, H, D)


def test_static_scratch_at_the_documented_flux_shape(dthip):
    """The shape the array is sized for: 512 text + 64 x 64 image tokens, 24 heads x 128, fused per-head RMSNorm and
    RoPE (staged K: 28.3 MB of the 64 MiB array) -- bit for bit against dt_sdpa_f16."""
    import torch

    T, h, w, H, D = 512, 64, 64, 24, 128
    HW = h * w
    assert dthip.lib().dt_init(0) == 0  # (this is where a GPU's copy of the array is looked up, and loaded)
    assert dthip.lib().dt_sdpa_workspace_bytes(1, H, H, D, T + HW, T + HW, 1, 0) <= dthip.STATIC_SCRATCH_BYTES
    g = torch.Generator(device="cuda").manual_seed(72)
    rnd = lambda *s: torch.randn(s, device="cuda", generator=g).half()
    segs = {n: (rnd(1, T, H, D), rnd(1, HW, H, D)) for n in "qkv"}
    gam = {n: ((1 + 0.05 * rnd(D).float()).half(), (1 + 0.05 * rnd(D).float()).half()) for n in "qk"}
    rot = torch.from_numpy(dthip.Flux1RotaryPositionEmbedding(h, w, T, channels=D).astype(np.float16)).cuda()
    args = dict(q_segs=list(segs["q"]), k_segs=list(segs["k"]), v_segs=list(segs["v"]), scale=1 / np.sqrt(D),
                gamma_q=list(gam["q"]), gamma_k=list(gam["k"]), rot_q=rot, rot_k=rot)
    out = torch.full((1, T + HW, H, D), float("nan"), dtype=torch.float16, device="cuda")
    ref = dthip.sdpa_segments(**args)  # (first: in a fresh process this loads the kernels' code objects)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    print("static scratch call at the Flux shape", tuple(out.shape), flush=True)
    dthip.sdpa_segments(**args, out=out, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out, ref)
    assert bool(torch.isfinite(out.float()).all())


def test_static_scratch_validates_like_the_workspace_entry_point(dthip):
    """Bad arguments get the status dt_sdpa_f16 gives them, also when the shapes are beyond the array: the size of
    the request is looked at only after the argument checks."""
    import torch

    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
    g = torch.ones(128, dtype=torch.float16, device="cuda")
    big = 12000  # staged K beyond 64 MiB at 24 heads x 128
    cases = [
        (dict(q_segs=[z(1, big, 24, 128)], k_segs=[z(1, big, 5, 128)], v_segs=[z(1, big, 5, 128)]), dthip.DT_INVALID),  # 5 does not divide 24
        (dict(q_segs=[z(1, big, 24, 136)], k_segs=[z(1, big, 24, 136)], v_segs=[z(1, big, 24, 136)]), dthip.DT_NO_KERNEL),  # D > 128
        (dict(q_segs=[z(1, big, 24, 128)], k_segs=[z(1, big, 24, 128)], v_segs=[z(1, big - 8, 24, 128)]), dthip.DT_INVALID),  # k / v lengths differ
        (dict(q_segs=[z(1, 8, 2, 64)], k_segs=[z(1, 0, 2, 64)], v_segs=[z(1, 0, 2, 64)]), dthip.DT_INVALID),  # no keys
    ]
    for kw, want in cases:
        for static in (False, True):
            with pytest.raises(dthip.DtError) as e:
                gq = [g[:kw["q_segs"][0].shape[-1]]] if kw["q_segs"][0].shape[-1] <= 128 else None
                dthip.sdpa_segments(**kw, scale=1.0, gamma_q=gq, static_scratch=static)
            assert e.value.status == want, (static, want, e.value.status)
