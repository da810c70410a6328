"""GPU side of the `.ckpt` container reader: a palettized row read without `.jit` comes back dequantized (bit-exact
against the oracle), and a Dense whose weight and bias were filled by `read_model` computes what the oracle computes
from the same packed bytes."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_store_to_dense(tmp_path, dthip, oracle):
    import torch
    store_mod = importlib.import_module(dthip.__name__ + ".store")
    rng = np.random.default_rng(4)
    N, K, q, nib = 256, 320, 6, 4096
    packed, _, _ = oracle.synth_qx_weight(rng, N, K, q, nib, 0.05)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16)
    path = str(tmp_path / "m.ckpt")
    with store_mod.Store(path, mode="w") as st:
        st.write("__dit__[t-x_q-0-0]", dthip.QxTensor.from_packed(packed, q, nib, (N, K), device="cpu"))
        st.write("__dit__[t-x_q-0-1]", bias)
    print("store -> dense", flush=True)
    with store_mod.Store(path) as st:
        full = st.read("__dit__[t-x_q-0-0]", ("q6p",))          # no .jit: dequantized
        want = oracle.C.depalettize(q, nib, N * K, packed).reshape(N, K)
        assert np.array_equal(full.cpu().numpy().view(np.uint16), want.view(np.uint16))
        layer = dthip.Dense(N, name="x_q")
        assert st.read_model("dit", {"x_q": layer}) == []
    X = rng.standard_normal((70, K)).astype(np.float16)
    got = layer(torch.from_numpy(X).cuda()).cpu().numpy()
    mx, rr = oracle.err_stats(got, oracle.C.dense_qx(X, packed, q, nib, N, bias))
    assert mx <= 2e-2 and rr <= 1e-3

