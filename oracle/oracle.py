"""CPU checker for the transformer-block hot path -- TEST INFRASTRUCTURE ONLY.

Two things live here:

* ``C`` -- ctypes bindings for ``libdtoracle.so`` (built from ``dt_oracle.c``,
  the C restatement whose header lists what each function follows in the
  reference and what pins it).
* ``np_*`` -- a second, independently written numpy restatement of the
  integer parts (index packing, palette lookup) and float64 versions of the
  floating-point parts.  The tests pin the C code against these, against
  hand-built byte vectors and against closed forms, so that a slip in either
  one (wrong bit order, wrong block stride, transposed operand) shows up.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  The product path never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libdtoracle.so")

_u8p = ctypes.POINTER(ctypes.c_uint8)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)
_i64 = ctypes.c_int64
_int = ctypes.c_int


def build(force: bool = False) -> str:
    """Compile libdtoracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(
        os.path.join(_HERE, "dt_oracle.c")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libdtoracle.so"], stdout=subprocess.DEVNULL)
    return _LIB


def _ptr(a: np.ndarray, typ):
    return a.ctypes.data_as(typ)


class _C:
    """Thin typed wrapper over the C oracle."""

    def __init__(self):
        self._lib = None

    @property
    def lib(self):
        if self._lib is None:
            if not os.path.exists(_LIB):
                build()
            lib = ctypes.CDLL(_LIB)
            lib.dto_qx_bytes.restype = _i64
            lib.dto_qx_bytes.argtypes = [_int, _int, _i64]
            lib.dto_pack_indices.argtypes = [_int, _u8p, _i64, _u8p]
            lib.dto_unpack_indices.argtypes = [_int, _u8p, _i64, _u8p]
            lib.dto_palettize_pack.argtypes = [_int, _int, _i64, _u16p, _u8p, _u8p]
            lib.dto_depalettize.argtypes = [_int, _int, _i64, _u8p, _u16p]
            lib.dto_dense.argtypes = [_i64, _i64, _i64, _u16p, _i64, _u16p, _u16p, _u16p, _i64]
            lib.dto_dense_qx.argtypes = [_i64, _i64, _i64, _u16p, _i64, _u8p, _int, _int, _u16p, _u16p, _i64]
            lib.dto_rmsnorm.restype = None
            lib.dto_rmsnorm.argtypes = [_i64, _i64, _u16p, _i64, _u16p, ctypes.c_float, _u16p, _i64]
            lib.dto_cmul.restype = None
            lib.dto_cmul.argtypes = [_i64, _i64, _i64, _u16p, _i64, _i64, _u16p, _i64, _u16p, _i64, _i64]
            lib.dto_rope_flux.argtypes = [_int, _int, _int, _int, _i32p, _int, _f32p]
            lib.dto_rope_wan.argtypes = [_int, _int, _int, _int, _f32p]
            lib.dto_sdpa.argtypes = (
                [_int, _int, _int, _int, _i64, _i64]
                + [_u16p, _i64, _i64, _i64] * 4
                + [ctypes.c_float, _int]
            )
            lib.dto_dense_instruction_count.restype = _i64
            lib.dto_dense_instruction_count.argtypes = [_i64, _i64, _i64]
            lib.dto_sdpa_instruction_count.restype = _i64
            lib.dto_sdpa_instruction_count.argtypes = [_i64] * 5
            lib.dto_h2f.restype = ctypes.c_float
            lib.dto_h2f.argtypes = [ctypes.c_uint16]
            lib.dto_f2h.restype = ctypes.c_uint16
            lib.dto_f2h.argtypes = [ctypes.c_float]
            self._lib = lib
        return self._lib

    # -- layout ---------------------------------------------------------
    def qx_bytes(self, qbits, nib, count):
        return int(self.lib.dto_qx_bytes(qbits, nib, count))

    def pack_indices(self, qbits, idx):
        idx = np.ascontiguousarray(idx, dtype=np.uint8)
        out = np.zeros((idx.size * qbits + 7) // 8, dtype=np.uint8)
        self.lib.dto_pack_indices(qbits, _ptr(idx, _u8p), idx.size, _ptr(out, _u8p))
        return out

    def unpack_indices(self, qbits, packed, n):
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        out = np.zeros(n, dtype=np.uint8)
        self.lib.dto_unpack_indices(qbits, _ptr(packed, _u8p), n, _ptr(out, _u8p))
        return out

    def palettize_pack(self, qbits, nib, palettes, idx):
        """palettes: float16 [nblocks, 2^q]; idx: uint8 [count] -> packed uint8 buffer."""
        idx = np.ascontiguousarray(idx, dtype=np.uint8).reshape(-1)
        count = idx.size
        palettes = np.ascontiguousarray(palettes, dtype=np.float16)
        nblocks = (count + nib - 1) // nib
        assert palettes.shape == (nblocks, 1 << qbits), palettes.shape
        out = np.zeros(self.qx_bytes(qbits, nib, count), dtype=np.uint8)
        rc = self.lib.dto_palettize_pack(
            qbits, nib, count, _ptr(palettes.view(np.uint16), _u16p), _ptr(idx, _u8p), _ptr(out, _u8p)
        )
        assert rc == 0
        return out

    def depalettize(self, qbits, nib, count, packed):
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        out = np.zeros(count, dtype=np.uint16)
        rc = self.lib.dto_depalettize(qbits, nib, count, _ptr(packed, _u8p), _ptr(out, _u16p))
        assert rc == 0
        return out.view(np.float16)

    # -- float ops ------------------------------------------------------
    def dense(self, X, W, bias=None):
        """X [M,K] f16 (rows may be strided), W [N,K] f16 -> Y [M,N] f16."""
        assert X.dtype == np.float16 and W.dtype == np.float16
        M, K = X.shape
        N = W.shape[0]
        assert W.shape == (N, K) and X.strides[1] == 2
        W = np.ascontiguousarray(W)
        Y = np.zeros((M, N), dtype=np.float16)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)
        rc = self.lib.dto_dense(
            M, N, K, _ptr(X.view(np.uint16), _u16p), X.strides[0] // 2 if M else K,
            _ptr(W.view(np.uint16), _u16p), None if b is None else _ptr(b.view(np.uint16), _u16p),
            _ptr(Y.view(np.uint16), _u16p), N,
        )
        assert rc == 0
        return Y

    def dense_qx(self, X, packed, qbits, nib, N, bias=None):
        assert X.dtype == np.float16
        X = np.ascontiguousarray(X)
        M, K = X.shape
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        Y = np.zeros((M, N), dtype=np.float16)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)
        rc = self.lib.dto_dense_qx(
            M, N, K, _ptr(X.view(np.uint16), _u16p), K, _ptr(packed, _u8p), qbits, nib,
            None if b is None else _ptr(b.view(np.uint16), _u16p), _ptr(Y.view(np.uint16), _u16p), N,
        )
        assert rc == 0
        return Y

    def rmsnorm(self, x, gamma, eps=1e-6):
        """x [..., width] f16 contiguous; normalises the last axis."""
        x = np.ascontiguousarray(x, dtype=np.float16)
        width = x.shape[-1]
        rows = x.size // width
        y = np.zeros_like(x)
        g = None if gamma is None else np.ascontiguousarray(gamma, dtype=np.float16)
        self.lib.dto_rmsnorm(
            rows, width, _ptr(x.view(np.uint16), _u16p), width,
            None if g is None else _ptr(g.view(np.uint16), _u16p), eps, _ptr(y.view(np.uint16), _u16p), width,
        )
        return y

    def cmul(self, x, rot):
        """x [S,H,D] f16, rot [S,D] f16 -> [S,H,D]."""
        x = np.ascontiguousarray(x, dtype=np.float16)
        rot = np.ascontiguousarray(rot, dtype=np.float16)
        S, H, D = x.shape
        assert rot.shape == (S, D)
        y = np.zeros_like(x)
        self.lib.dto_cmul(
            S, H, D, _ptr(x.view(np.uint16), _u16p), H * D, D, _ptr(rot.view(np.uint16), _u16p), D,
            _ptr(y.view(np.uint16), _u16p), H * D, D,
        )
        return y

    def rope_flux(self, height, width, token_length, channels=128, ref_sizes=()):
        n = token_length + height * width + sum(h * w for h, w in ref_sizes)
        out = np.zeros((n, channels), dtype=np.float32)
        ref = np.asarray([v for hw in ref_sizes for v in hw], dtype=np.int32)
        rc = self.lib.dto_rope_flux(
            height, width, token_length, len(ref_sizes), _ptr(ref, _i32p) if len(ref) else None, channels,
            _ptr(out, _f32p),
        )
        assert rc == 0
        return out

    def rope_wan(self, height, width, time, channels=128):
        out = np.zeros((time * height * width, channels), dtype=np.float32)
        rc = self.lib.dto_rope_wan(height, width, time, channels, _ptr(out, _f32p))
        assert rc == 0
        return out

    def sdpa(self, q, k, v, scale, round_mid=0):
        """q [B,Sq,Hq,D], k/v [B,Skv,Hk,D] f16 (any strides with D contiguous) -> [B,Sq,Hq,D]."""
        for t in (q, k, v):
            assert t.dtype == np.float16 and t.ndim == 4 and (t.shape[3] == 1 or t.strides[3] == 2)
        B, Sq, Hq, D = q.shape
        _, Skv, Hk, _ = k.shape
        o = np.zeros((B, Sq, Hq, D), dtype=np.float16)

        def st(t):
            return [t.strides[0] // 2, t.strides[1] // 2, t.strides[2] // 2]

        rc = self.lib.dto_sdpa(
            B, Hq, Hk, D, Sq, Skv,
            _ptr(q.view(np.uint16), _u16p), *st(q),
            _ptr(k.view(np.uint16), _u16p), *st(k),
            _ptr(v.view(np.uint16), _u16p), *st(v),
            _ptr(o.view(np.uint16), _u16p), *st(o),
            float(scale), int(round_mid),
        )
        assert rc == 0
        return o

    def dense_instruction_count(self, rows, inp, out):
        return int(self.lib.dto_dense_instruction_count(rows, inp, out))

    def sdpa_instruction_count(self, b, h, d, sa, sb):
        return int(self.lib.dto_sdpa_instruction_count(b, h, d, sa, sb))


C = _C()


# ----------------------------------------------------------------------------
# Independent numpy restatement (bit-level parts exact, float parts in float64)
# ----------------------------------------------------------------------------

def np_pack_indices(qbits: int, idx) -> np.ndarray:
    """MSB-first bit stream built with numpy's own bit packer."""
    idx = np.asarray(idx, dtype=np.uint8).reshape(-1)
    bits = np.unpackbits(idx[:, None], axis=1, bitorder="big")[:, 8 - qbits:]
    return np.packbits(bits.reshape(-1), bitorder="big")


def np_unpack_indices(qbits: int, packed, n: int) -> np.ndarray:
    bits = np.unpackbits(np.asarray(packed, dtype=np.uint8), bitorder="big")[: n * qbits]
    weights = (1 << np.arange(qbits - 1, -1, -1)).astype(np.uint16)
    return (bits.reshape(n, qbits).astype(np.uint16) * weights).sum(axis=1).astype(np.uint8)


def np_palettize_pack(qbits: int, nib: int, palettes, idx) -> np.ndarray:
    idx = np.asarray(idx, dtype=np.uint8).reshape(-1)
    palettes = np.asarray(palettes, dtype=np.float16)
    chunks = []
    for b in range((idx.size + nib - 1) // nib):
        chunks.append(palettes[b].view(np.uint8).reshape(-1))
        chunks.append(np_pack_indices(qbits, idx[b * nib:(b + 1) * nib]))
    return np.concatenate(chunks) if chunks else np.zeros(0, np.uint8)


def np_depalettize(qbits: int, nib: int, count: int, packed) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.zeros(count, dtype=np.float16)
    pos = 0
    palbytes = 2 << qbits
    for b in range((count + nib - 1) // nib):
        n = min(nib, count - b * nib)
        pal = packed[pos:pos + palbytes].view(np.float16)
        pos += palbytes
        nbytes = (n * qbits + 7) // 8
        out[b * nib:b * nib + n] = pal[np_unpack_indices(qbits, packed[pos:pos + nbytes], n)]
        pos += nbytes
    return out


def np_dense64(X, W, bias=None) -> np.ndarray:
    y = X.astype(np.float64) @ W.astype(np.float64).T
    if bias is not None:
        y = y + bias.astype(np.float64)
    return y


def np_rmsnorm64(x, gamma, eps=1e-6) -> np.ndarray:
    x = x.astype(np.float64)
    y = x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    return y if gamma is None else y * gamma.astype(np.float64)


def np_cmul64(x, rot) -> np.ndarray:
    """x [S,H,D], rot [S,D] interleaved (cos, sin) -> float64 [S,H,D]."""
    x = x.astype(np.float64)
    r = rot.astype(np.float64)[:, None, :]
    xc = x[..., 0::2] + 1j * x[..., 1::2]
    rc = r[..., 0::2] + 1j * r[..., 1::2]
    yc = xc * rc
    y = np.empty_like(x)
    y[..., 0::2] = yc.real
    y[..., 1::2] = yc.imag
    return y


def np_sdpa64(q, k, v, scale) -> np.ndarray:
    """Brute-force float64 attention, [B,S,H,D] layout, GQA by head grouping."""
    q = q.astype(np.float64)
    k = k.astype(np.float64)
    v = v.astype(np.float64)
    B, Sq, Hq, D = q.shape
    Hk = k.shape[2]
    g = Hq // Hk
    o = np.zeros((B, Sq, Hq, D))
    for b in range(B):
        for h in range(Hq):
            s = scale * (q[b, :, h] @ k[b, :, h // g].T)
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            o[b, :, h] = p @ v[b, :, h // g]
    return o


def err_stats(got, want):
    """(max-abs, rel-RMS) of got vs want, both computed in float64."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    d = got - want
    max_abs = float(np.abs(d).max()) if d.size else 0.0
    den = float(np.sqrt((want * want).mean())) if d.size else 1.0
    rel_rms = float(np.sqrt((d * d).mean()) / den) if den > 0 else float(np.sqrt((d * d).mean()))
    return max_abs, rel_rms


def synth_qx_weight(rng, N, K, qbits, nib, std=0.02):
    """Synthetic palettized weight of the benchmark kind: per-block N(0, std) fp16
    palettes and uniform indices.  Returns (packed uint8, palettes, idx)."""
    count = N * K
    nblocks = (count + nib - 1) // nib
    palettes = (rng.standard_normal((nblocks, 1 << qbits)) * std).astype(np.float16)
    idx = rng.integers(0, 1 << qbits, size=count, dtype=np.uint8)
    return C.palettize_pack(qbits, nib, palettes, idx), palettes, idx


# ---------------------------------------------------------------------------
# Elementwise tails of the feed-forward / residual paths (numpy; fp16 in, fp16 out; the activations are the
# mathematical functions, evaluated in float64 and rounded once).  Pinned in tests/test_oracle_ops.py by float64 closed forms (erf-GELU bound,
# gelu(x) - gelu(-x) = x, limits, sigmoid identity) and exact small cases of the residual update.  GELU(approximate: .tanh): Models/Flux1.swift:133-135; swish: :122-123;
# gated residual x + (y .* gate).to(of: x): :246-250, 275-283.
# ---------------------------------------------------------------------------

def np_gelu_tanh16(y16: np.ndarray) -> np.ndarray:
    """GELU(approximate: .tanh), 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))), evaluated in float64 and rounded
    once: the function itself.  (Evaluated in float32 as written, `1 + tanh(u)` cancels for x < -3: over all fp16
    inputs that form is up to 3 fp16 ulps -- 1.5e-7 in absolute terms -- off this one, on outputs below 2^-10.)"""
    x = y16.astype(np.float64)
    u = 0.7978845608028654 * (x + 0.044715 * x * x * x)
    return (0.5 * x * (1.0 + np.tanh(u))).astype(np.float32).astype(np.float16)


def np_gelu_erf16(y16: np.ndarray) -> np.ndarray:
    """GELU() in its erf form, 0.5 x (1 + erf(x / sqrt 2)) (GELU()(fc11(x)), Models/UNet.swift:513), fp16 in and out."""
    from scipy.special import erf
    x = y16.astype(np.float64)
    return (0.5 * x * (1 + erf(x / np.sqrt(2.0)))).astype(np.float32).astype(np.float16)


def np_mul16(a16: np.ndarray, b16: np.ndarray) -> np.ndarray:
    """fp16 elementwise product (out .* GELU()(fc11(x)), Models/UNet.swift:513): the float32 product of two fp16 values
    is exact, so one rounding."""
    return (a16.astype(np.float32) * b16.astype(np.float32)).astype(np.float16)


def np_layernorm16(x16: np.ndarray, gamma16=None, beta16=None, eps: float = 1e-5) -> np.ndarray:
    """LayerNorm(epsilon:, axis: [last]) with fp16 affine weight and bias on an fp16 tensor (Models/UNet.swift:530,
    544, 554): statistics (biased variance) and the affine step in float64, one rounding to fp16 at the end."""
    x = x16.astype(np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mean) / np.sqrt(var + eps)
    if gamma16 is not None:
        y = y * gamma16.astype(np.float64)
    if beta16 is not None:
        y = y + beta16.astype(np.float64)
    return y.astype(np.float32).astype(np.float16)


def np_swish16(y16: np.ndarray) -> np.ndarray:
    """x sigmoid(x) in float64, rounded once."""
    x = y16.astype(np.float64)
    with np.errstate(over="ignore"):
        return (x / (1.0 + np.exp(-x))).astype(np.float32).astype(np.float16)


def np_layernorm_modulate16(x32: np.ndarray, scale=None, shift=None, eps: float = 1e-6, mod: str = "f16") -> np.ndarray:
    """LayerNorm(epsilon:, axis: [last], elementwiseAffine: false) of an fp32 stream, then the adaLN modulation, fp16
    out.  mod "f16": fp16(fp16(fp16(norm) * scale) + shift) with fp16 scale / shift -- xNorm1(x).to(.Float16) .*
    xChunks[1] + xChunks[0] (Models/Flux1.swift:172-173, 281-282).  mod "f32": fp16(norm * (scale + 1) + shift) with
    fp32 scale / shift -- (xNorm2(out) .* (chunks[4] + 1) + chunks[3]).to(.Float16) (Models/Wan.swift:217-221).
    mod "affine": fp16(norm * scale + shift), the LayerNorm's own fp32 weight and bias (Models/Wan.swift:160-161).
    Statistics in float64 (biased variance), the normalised value rounded to float32 as the fp32 op leaves it."""
    x = x32.astype(np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    n = ((x - mean) / np.sqrt(var + eps)).astype(np.float32)
    if mod == "f16":
        y = n.astype(np.float16)
        if scale is not None:
            y = (y.astype(np.float32) * scale.astype(np.float16).astype(np.float32)).astype(np.float16)
        if shift is not None:
            y = (y.astype(np.float32) + shift.astype(np.float16).astype(np.float32)).astype(np.float16)
        return y
    if scale is not None:
        n = n * (scale.astype(np.float32) + np.float32(1) if mod == "f32" else scale.astype(np.float32))
    if shift is not None:
        n = n + shift.astype(np.float32)
    return n.astype(np.float16)


def np_lora_branch16(X16: np.ndarray, down16: np.ndarray, up16: np.ndarray, scale: float = 1.0) -> np.ndarray:
    """up(scale * down(x)) of a LoRADense, each op rounding to fp16 (Models/LoRA.swift:117-140): down [rank, in],
    up [count, rank], both without bias; the scalar multiply is its own op and only exists when scale != 1."""
    d = np_dense64(X16, down16).astype(np.float16)
    if scale != 1:
        d = (d.astype(np.float32) * np.float32(scale)).astype(np.float16)
    return np_dense64(d, up16).astype(np.float16)


def np_lora_branch32(X16: np.ndarray, down32: np.ndarray, up32: np.ndarray, scale: float = 1.0) -> np.ndarray:
    """The low-rank branch with highPrecision (Models/LoRA.swift:117-139): `denseDown(x.to(.Float32))`,
    `denseUp(scale * downX).to(of: x)` -- fp32 weights and intermediate, one rounding to fp16 at the end.  Evaluated in
    float64 and rounded to fp32 where the graph holds fp32 tensors (the fp32 GEMMs' own summation error, ~1e-6
    relative, is below what the final fp16 rounding keeps)."""
    t = (X16.astype(np.float64) @ down32.astype(np.float64).T).astype(np.float32)
    t = (np.float32(scale) * t).astype(np.float32)
    return (t.astype(np.float64) @ up32.astype(np.float64).T).astype(np.float32).astype(np.float16)


def np_add16(a16: np.ndarray, b16: np.ndarray) -> np.ndarray:
    """fp16 elementwise sum (out = dense(x) + up(...), Models/LoRA.swift:128-140); the float32 sum of two fp16 values
    is exact, so one rounding."""
    return (a16.astype(np.float32) + b16.astype(np.float32)).astype(np.float16)


def np_gated_residual32(res32: np.ndarray, y16: np.ndarray, gate32=None) -> np.ndarray:
    """res + float32(y) * gate32, the product formed in fp32 (x + out.to(of: x) .* chunks[2], Models/Wan.swift:159,
    220-221); gate broadcast over rows."""
    y = y16.astype(np.float32)
    if gate32 is not None:
        y = y * gate32.astype(np.float32)[None, :]
    return (res32.astype(np.float32) + y).astype(np.float32)


def np_gated_residual(res32: np.ndarray, y16: np.ndarray, gate16=None) -> np.ndarray:
    """res + float32(fp16(y * gate)); gate broadcast over rows."""
    y = y16 if gate16 is None else (y16.astype(np.float32) * gate16.astype(np.float32)[None, :]).astype(np.float16)
    return (res32.astype(np.float32) + y.astype(np.float32)).astype(np.float32)


def np_flux_joint_block(context32, x32, rot16, cch, xch, dense, bias, norm, k, h):
    """Flux.1 JointTransformerBlock op by op (Models/Flux1.swift:149-290; contextBlockPreOnly false, upcast false):
    LayerNorm + modulation (:160, 172-173), the six projections (:161-183), per-head RMSNorm of Q and K (:164-169,
    177-182), concat text || image and RoPE (:184-188), attention at scale 1 / sqrt(k) (:228-232), c_o / x_o and the
    gated residual additions (:236-250), the feed-forward with GELU(tanh) and its gated residual (:130-147, 251-283).
    `dense[name]` is a callable X16 -> Y16 (this module's Dense with that layer's weight and bias); `norm[name]` the
    fp16 RMSNorm weight; `cch` / `xch` the six fp16 modulation vectors of each stream.  fp32 streams in and out."""
    t, hw = context32.shape[0], x32.shape[0]
    c = np_layernorm_modulate16(context32, cch[1], cch[0], 1e-6, "f16")
    xx = np_layernorm_modulate16(x32, xch[1], xch[0], 1e-6, "f16")
    heads = lambda y, n: y.reshape(n, h, k)
    cK = C.rmsnorm(heads(dense["c_k"](c), t), norm["c_norm_k"], 1e-6)
    cQ = C.rmsnorm(heads(dense["c_q"](c), t), norm["c_norm_q"], 1e-6)
    cV = heads(dense["c_v"](c), t)
    xK = C.rmsnorm(heads(dense["x_k"](xx), hw), norm["x_norm_k"], 1e-6)
    xQ = C.rmsnorm(heads(dense["x_q"](xx), hw), norm["x_norm_q"], 1e-6)
    xV = heads(dense["x_v"](xx), hw)
    keys = C.cmul(np.concatenate([cK, xK], axis=0), rot16)
    queries = C.cmul(np.concatenate([cQ, xQ], axis=0), rot16)
    values = np.concatenate([cV, xV], axis=0)
    out = C.sdpa(queries[None], keys[None], values[None], 1.0 / np.sqrt(k))[0].reshape(t + hw, h * k)
    context = np_gated_residual(context32, dense["c_o"](np.ascontiguousarray(out[:t])), cch[2])
    x = np_gated_residual(x32, dense["x_o"](np.ascontiguousarray(out[t:])), xch[2])
    ff = lambda y, name: dense[name + "_out_proj"](np_gelu_tanh16(dense[name + "_linear1"](y)))
    context = np_gated_residual(context, ff(np_layernorm_modulate16(context, cch[4], cch[3], 1e-6, "f16"), "c"), cch[5])
    x = np_gated_residual(x, ff(np_layernorm_modulate16(x, xch[4], xch[3], 1e-6, "f16"), "x"), xch[5])
    return context, x


def np_wan_attention_block(x32, rot16, chunks32, cK16, cV16, dense, norm, norm3_w32, norm3_b32, k, h):
    """WanAttentionBlock op by op (Models/Wan.swift:68-277; batch 1, no causal inference, no injected image,
    self-attention at level .scale1): LayerNorm + fp32 modulation (:81-82), x_q / x_k / x_v with whole-row RMSNorm on Q
    and K (:83-92), RoPE (:93-94), the k^(-1/4) scale on both (:95-98), attention at scale 1 (:103, 129-131), x_o and
    the fp32-gated residual (:157-159), affine LayerNorm x_norm_3 (:160-161), x_c_q with whole-row RMSNorm (:162-167),
    cross-attention at 1 / sqrt(k) over the given context K / V (:169-174), c_o and its residual (:215-216), the
    feed-forward and its fp32-gated residual (:217-221).  `chunks32` = c + modulations, six fp32 vectors.
    `dense[name]`: callable X16 -> Y16; `norm[name]`: fp16 whole-row RMSNorm weights.  fp32 stream in and out."""
    hw = x32.shape[0]
    C_ = h * k
    xn = np_layernorm_modulate16(x32, chunks32[1], chunks32[0], 1e-6, "f32")
    xK = C.rmsnorm(dense["x_k"](xn), norm["x_norm_k"], 1e-6).reshape(hw, h, k)
    xQ = C.rmsnorm(dense["x_q"](xn), norm["x_norm_q"], 1e-6).reshape(hw, h, k)
    xV = dense["x_v"](xn).reshape(hw, h, k)
    quarter = np.float32(1.0 / np.sqrt(np.sqrt(k)))
    scale16 = lambda a: (a.astype(np.float32) * quarter).astype(np.float16)
    queries = scale16(C.cmul(xQ, rot16))
    keys = scale16(C.cmul(xK, rot16))
    att = C.sdpa(queries[None], keys[None], xV[None], 1.0)[0].reshape(hw, C_)
    out = np_gated_residual32(x32, dense["x_o"](att), chunks32[2])
    xn = np_layernorm_modulate16(out, norm3_w32, norm3_b32, 1e-6, "affine")
    cQ = C.rmsnorm(dense["x_c_q"](xn), norm["x_c_norm_q"], 1e-6).reshape(hw, h, k)
    cross = C.sdpa(cQ[None], cK16, cV16, 1.0 / np.sqrt(k))[0].reshape(hw, C_)
    out = np_gated_residual32(out, dense["c_o"](cross), None)
    xn = np_layernorm_modulate16(out, chunks32[4], chunks32[3], 1e-6, "f32")
    ff = dense["x_out_proj"](np_gelu_tanh16(dense["x_linear1"](xn)))
    return np_gated_residual32(out, ff, chunks32[5])


def np_flux_single_block(x32, rot16, xch, dense, norm, k, h):
    """Flux.1 SingleTransformerBlock op by op (Models/Flux1.swift:367-492; contextBlockPreOnly false): LayerNorm +
    modulation (:375-376), x_q / x_k / x_v with per-head RMSNorm (:377-386), RoPE (:390-391), attention at
    1 / sqrt(k) (:431-435), then x_o (no bias) + feed-forward of the same modulated input, summed in fp16, gated and
    added to the fp32 stream (:452-456).  `dense[name]`: callable X16 -> Y16; `xch`: shift, scale, gate (fp16)."""
    S = x32.shape[0]
    xn = np_layernorm_modulate16(x32, xch[1], xch[0], 1e-6, "f16")
    K_ = C.cmul(C.rmsnorm(dense["x_k"](xn).reshape(S, h, k), norm["x_norm_k"], 1e-6), rot16)
    Q_ = C.cmul(C.rmsnorm(dense["x_q"](xn).reshape(S, h, k), norm["x_norm_q"], 1e-6), rot16)
    V_ = dense["x_v"](xn).reshape(S, h, k)
    att = C.sdpa(Q_[None], K_[None], V_[None], 1.0 / np.sqrt(k))[0].reshape(S, h * k)
    ff = dense["x_out_proj"](np_gelu_tanh16(dense["x_linear1"](xn)))
    return np_gated_residual(x32, np_add16(dense["x_o"](att), ff), xch[2])


def np_unet_transformer_block(x16, c16, dense, norm, k, h):
    """BasicTransformerBlock of the SD 1.5 UNet op by op (Models/UNet.swift:519-565; fp16, no injected KV / IP
    adapters): LayerNorm(1e-5) with affine (:530, 538), self-attention q / k / v without bias and attention at
    1 / sqrt(k) with the unify-heads projection (:95-156), + x (:542), LayerNorm, cross-attention with keys and values
    from the text context (:269-320), + residual (:551), LayerNorm, fc10(x) .* GELU()(fc11(x)) -> fc2 (:506-517),
    + residual (:558).  x16 [b, hw, C], c16 [b, t, Cc]; `dense[name]`: callable X16 -> Y16; `norm[name]`: (weight,
    bias) fp16."""
    b, hw, C_ = x16.shape
    t = c16.shape[1]
    x2 = x16.reshape(b * hw, C_)
    c2 = c16.reshape(b * t, c16.shape[2])
    scale = 1.0 / np.sqrt(k)
    heads = lambda y, s: y.reshape(b, s, h, k)
    n1 = np_layernorm16(x2, *norm["layerNorm1"], 1e-5)
    att = C.sdpa(heads(dense["toqueries1"](n1), hw), heads(dense["tokeys1"](n1), hw), heads(dense["tovalues1"](n1), hw), scale)
    out = np_add16(dense["unifyheads1"](att.reshape(b * hw, C_)), x2)
    n2 = np_layernorm16(out, *norm["layerNorm2"], 1e-5)
    att = C.sdpa(heads(dense["toqueries2"](n2), hw), heads(dense["tokeys2"](c2), t), heads(dense["tovalues2"](c2), t), scale)
    out = np_add16(dense["unifyheads2"](att.reshape(b * hw, C_)), out)
    n3 = np_layernorm16(out, *norm["layerNorm3"], 1e-5)
    hid = np_mul16(dense["fc10"](n3), np_gelu_erf16(dense["fc11"](n3)))
    return np_add16(dense["fc2"](hid), out).reshape(b, hw, C_)

