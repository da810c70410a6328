"""Pins the oracle's palettized-layout code (integer / byte work: bit-exact).

Three independent statements of the MSB-first index stream are compared:
the C oracle, numpy's own bit packer, and the per-group byte formulas; plus
hand-computed byte vectors (tests/golden/pack_kat.json).
"""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "pack_kat.json")
QBITS = [4, 5, 6, 7, 8]


def formula_pack(q, i):
    """Per-group byte formulas of the codec (one group = lcm(q, 8) bits)."""
    i = [int(v) for v in i]
    if q == 8:
        return i
    if q == 4:
        return [((i[0] << 4) | i[1]) & 255]
    if q == 6:
        return [((i[0] << 2) | (i[1] >> 4)) & 255, ((i[1] << 4) | (i[2] >> 2)) & 255, ((i[2] << 6) | i[3]) & 255]
    if q == 5:
        return [
            ((i[0] << 3) | (i[1] >> 2)) & 255,
            ((i[1] << 6) | (i[2] << 1) | (i[3] >> 4)) & 255,
            ((i[3] << 4) | (i[4] >> 1)) & 255,
            ((i[4] << 7) | (i[5] << 2) | (i[6] >> 3)) & 255,
            ((i[6] << 5) | i[7]) & 255,
        ]
    if q == 7:
        return [
            ((i[0] << 1) | (i[1] >> 6)) & 255,
            ((i[1] << 2) | (i[2] >> 5)) & 255,
            ((i[2] << 3) | (i[3] >> 4)) & 255,
            ((i[3] << 4) | (i[4] >> 3)) & 255,
            ((i[4] << 5) | (i[5] >> 2)) & 255,
            ((i[5] << 6) | (i[6] >> 1)) & 255,
            ((i[6] << 7) | i[7]) & 255,
        ]
    raise AssertionError(q)


GROUP = {4: 2, 5: 8, 6: 4, 7: 8, 8: 1}


def test_golden_vectors(oracle):
    gold = json.load(open(GOLD))
    for case in gold["cases"]:
        q, idx, want = case["qbits"], case["idx"], case["bytes"]
        got = oracle.C.pack_indices(q, np.array(idx, np.uint8))
        assert got.tolist() == want, case
        assert oracle.np_pack_indices(q, idx).tolist() == want, case
        assert oracle.C.unpack_indices(q, np.array(want, np.uint8), len(idx)).tolist() == idx
        assert oracle.np_unpack_indices(q, want, len(idx)).tolist() == idx


def test_golden_block_case(oracle):
    bc = json.load(open(GOLD))["block_case"]
    q, nib, count = bc["qbits"], bc["nib"], bc["count"]
    pal = np.array([[(b + 1) + e / 16 for e in range(1 << q)] for b in range(2)], np.float16)
    packed = oracle.C.palettize_pack(q, nib, pal, np.array(bc["idx"], np.uint8))
    assert packed.size == bc["total_bytes"] == oracle.C.qx_bytes(q, nib, count)
    palbytes = 2 << q
    assert packed[palbytes:palbytes + 4].tolist() == bc["index_bytes"][0]
    off = palbytes + 4 + palbytes
    assert packed[off:off + 2].tolist() == bc["index_bytes"][1]
    assert np.array_equal(packed[:palbytes].view(np.float16), pal[0])
    assert oracle.C.depalettize(q, nib, count, packed).astype(np.float64).tolist() == bc["values"]
    assert oracle.np_depalettize(q, nib, count, packed).astype(np.float64).tolist() == bc["values"]


@pytest.mark.parametrize("q", QBITS)
def test_every_value_in_every_lane(oracle, q):
    """Exhaustive: each index value at each position of a group, others zero and others all-ones."""
    g = GROUP[q]
    for fill in (0, (1 << q) - 1):
        for pos in range(g):
            for val in range(1 << q):
                idx = np.full(g, fill, np.uint8)
                idx[pos] = val
                want = formula_pack(q, idx)
                assert oracle.C.pack_indices(q, idx).tolist() == want
                assert oracle.np_pack_indices(q, idx).tolist() == want
                assert oracle.C.unpack_indices(q, np.array(want, np.uint8), g).tolist() == idx.tolist()


@pytest.mark.parametrize("q", QBITS)
def test_ragged_roundtrip(oracle, q):
    rng = np.random.default_rng(q)
    for n in list(range(0, 70)) + [511, 512, 513, 4097]:
        idx = rng.integers(0, 1 << q, size=n, dtype=np.uint8)
        packed = oracle.C.pack_indices(q, idx)
        assert packed.size == (n * q + 7) // 8
        assert np.array_equal(packed, oracle.np_pack_indices(q, idx))
        assert np.array_equal(oracle.C.unpack_indices(q, packed, n), idx)
        assert np.array_equal(oracle.np_unpack_indices(q, packed, n), idx)


@pytest.mark.parametrize("q", QBITS)
@pytest.mark.parametrize("nib", [32, 512, 1024])
def test_depalettize_c_vs_numpy_and_closed_form(oracle, q, nib):
    rng = np.random.default_rng(100 * q + nib)
    for count in (0, 1, nib - 1, nib, nib + 1, 3 * nib + 17):
        nblocks = (count + nib - 1) // nib
        pal = (rng.standard_normal((nblocks, 1 << q)) * 0.02).astype(np.float16)
        idx = rng.integers(0, 1 << q, size=count, dtype=np.uint8)
        pc = oracle.C.palettize_pack(q, nib, pal, idx)
        pn = oracle.np_palettize_pack(q, nib, pal, idx)
        assert np.array_equal(pc, pn)
        assert pc.size == nblocks * (2 << q) + (count // nib) * (nib * q // 8) + ((count % nib) * q + 7) // 8
        want = pal[np.arange(count) // nib, idx] if count else np.zeros(0, np.float16)
        assert np.array_equal(oracle.C.depalettize(q, nib, count, pc).view(np.uint16), want.view(np.uint16))
        assert np.array_equal(oracle.np_depalettize(q, nib, count, pc).view(np.uint16), want.view(np.uint16))


def test_fp16_conversion_matches_numpy(oracle):
    """The C oracle carries its own fp16<->fp32 conversion: all 65536 patterns, and RNE rounding."""
    lib = oracle.C.lib
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        got = lib.dto_h2f(h)
        if np.isnan(f[h]):
            assert np.isnan(got)
        else:
            assert got == f[h]
            assert lib.dto_f2h(float(f[h])) == h
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 10,
        rng.standard_normal(2000).astype(np.float32) * 1e-5,
        rng.standard_normal(2000).astype(np.float32) * 1e-7,
        np.array([65504, 65519.9, 65520, 1e6, -1e6, 0.0, -0.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 3 * 2.0 ** -25], np.float32),
        (np.float32(1) + np.arange(0, 64, dtype=np.float32) * np.float32(2.0 ** -12)),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert lib.dto_f2h(float(x)) == int(w), (float(x), int(w))
