"""The `.ckpt` container reader against files built here with sqlite3 directly: the table and column names, datatype
codes, the little-endian int32 `dim` array and the key scheme are the ones the reference's own script reads
(Scripts/qwen35_gguf_quant_csv.py:48-55, 113-135); palettized blobs come from the oracle's packer.  What a real file
would pin beyond that (how a row marks its codec, compressed blobs, the sidecar) is not covered: parity unpinned."""
import importlib
import os
import sqlite3
import struct

import numpy as np
import pytest


@pytest.fixture()
def store_mod(dthip):
    return importlib.import_module(dthip.__name__ + ".store")


def make_file(path, rows):
    db = sqlite3.connect(path)
    db.execute("CREATE TABLE tensors (name TEXT, type INTEGER, format INTEGER, datatype INTEGER, dim BLOB, data BLOB, "
               "PRIMARY KEY (name))")
    for name, code, shape, blob in rows:
        dims = list(shape) + [0] * (12 - len(shape))
        db.execute("INSERT INTO tensors VALUES (?, 0, 0, ?, ?, ?)", (name, code, struct.pack("<12i", *dims), blob))
    db.commit()
    db.close()


def test_palettized_lengths_are_distinct(store_mod, dthip, oracle):
    """The length formula equals the packer's output for every codec, ragged last blocks included, and no two codecs
    share a length for the shapes of the benchmark configurations (what recognising a blob by its length rests on)."""
    rng = np.random.default_rng(0)
    for name, (q, nib) in dthip.CODEC.items():
        for count in (1, 31, nib - 1, nib, nib + 1, 3 * nib + 77):
            packed, _, _ = oracle.synth_qx_weight(rng, 1, count, q, nib, 1.0)
            assert store_mod.palettized_bytes(q, nib, count) == packed.size == oracle.C.qx_bytes(q, nib, count)
    for count in (320 * 320, 320 * 768, 3072 * 3072, 3072 * 12288, 5120 * 5120, 5120 * 13824, 64 * 64, 128):
        sizes = [store_mod.palettized_bytes(q, nib, count) for q, nib in dthip.CODEC.values()] + [2 * count]
        assert len(set(sizes)) == len(sizes)


def test_store_reads_plain_and_palettized_rows(tmp_path, store_mod, dthip, oracle):
    rng = np.random.default_rng(1)
    N, K = 48, 160
    packed, pal, idx = oracle.synth_qx_weight(rng, N, K, 6, 4096, 0.05)
    bias = rng.standard_normal(N).astype(np.float16)
    pos = rng.standard_normal((1, 16, 8)).astype(np.float32)
    path = str(tmp_path / "model.ckpt")
    make_file(path, [
        ("__dit__[t-x_q-0-0]", 131072, (N, K), packed.tobytes()),
        ("__dit__[t-x_q-0-1]", 131072, (N,), bias.tobytes()),
        ("__dit__[t-pos_embed-0-0]", 16384, (1, 16, 8), pos.tobytes()),
        ("__dit__[t-odd-0-0]", (0x511 << 32) | 131072, (N, K), b"\\x00" * 100),   # some compressed blob
    ])
    with store_mod.Store(path) as st:
        assert st.keys == sorted(["__dit__[t-x_q-0-0]", "__dit__[t-x_q-0-1]", "__dit__[t-pos_embed-0-0]", "__dit__[t-odd-0-0]"])
        inf = st.info("__dit__[t-x_q-0-0]")
        assert (inf.datatype, inf.shape, inf.codec, inf.readable) == ("F16", (N, K), "q6p", True)
        assert st.info("__dit__[t-x_q-0-1]").codec is None and st.info("__dit__[t-pos_embed-0-0]").datatype == "F32"
        odd = st.info("__dit__[t-odd-0-0]")
        assert not odd.readable and odd.codec_id == 0x511
        assert st.info("missing") is None and st.read("missing", device="cpu") is None
        with pytest.raises(ValueError):
            st.read("__dit__[t-odd-0-0]", device="cpu")
        got_b = st.read("__dit__[t-x_q-0-1]", (), device="cpu")
        assert got_b.dtype.is_floating_point and np.array_equal(got_b.numpy(), bias)
        assert np.array_equal(st.read("__dit__[t-pos_embed-0-0]", (), device="cpu").numpy(), pos)
        w = st.read("__dit__[t-x_q-0-0]", ("jit", "q6p", "q8p"), device="cpu")
        assert isinstance(w, dthip.QxTensor) and (w.qbits, w.nib, w.shape) == (6, 4096, (N, K))
        assert np.array_equal(w.data.numpy()[: packed.size], packed)

        class Layer:
            weight = None
            bias = None

        layers = {"x_q": Layer(), "x_k": Layer()}
        assert st.read_model("dit", layers, device="cpu") == ["x_k"]
        assert layers["x_q"].weight.shape == (N, K) and np.array_equal(layers["x_q"].bias.numpy(), bias)


def test_store_write_round_trip(tmp_path, store_mod, dthip, oracle):
    rng = np.random.default_rng(2)
    packed, _, _ = oracle.synth_qx_weight(rng, 8, 64, 4, 512, 0.05)
    w = dthip.QxTensor.from_packed(packed, 4, 512, (8, 64), device="cpu")
    f32 = rng.standard_normal((3, 5)).astype(np.float32)
    path = str(tmp_path / "out.ckpt")
    with pytest.raises(FileNotFoundError):   # a reader never creates the file it was asked to read
        store_mod.Store(path)
    assert not os.path.exists(path)
    with store_mod.Store(path, mode="w") as st:
        st.write("a", w)
        st.write("b", f32)
    with store_mod.Store(path) as st:
        back = st.read("a", ("jit",), device="cpu")
        assert (back.qbits, back.nib, back.shape) == (4, 512, (8, 64))
        assert np.array_equal(back.data.numpy()[: packed.size], packed)
        assert np.array_equal(st.read("b", (), device="cpu").numpy(), f32)
        with pytest.raises(PermissionError):   # opened read-only
            st.write("c", f32)
    # the file is what the reference's own script expects: name, datatype, dim columns of table `tensors`
    rows = sqlite3.connect(path).execute("select name, datatype, dim from tensors order by name").fetchall()
    assert [r[0] for r in rows] == ["a", "b"] and rows[0][1] == 131072 and rows[1][1] == 16384
    assert struct.unpack("<12i", rows[0][2])[:3] == (8, 64, 0)
