"""Host side of the MI355X transformer-block hot path.

Mirrors the operator surface the reference's model builders use
(`Dense`, `RMSNorm`, `Functional.cmul`, `ScaledDotProductAttention`,
the rotary-table builders) on top of the C-ABI HIP library `libdthip.so`
declared in `include/dt_hip.h`.  torch is used for device memory and streams
only; every operator below runs a hand-written gfx950 kernel through ctypes
and raises if the library is missing or a call fails.  There is no CPU path.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdthip.so")
CSRC = os.path.join(_HERE, "csrc")

DT_OK, DT_INVALID, DT_NO_KERNEL, DT_OOM, DT_DEVICE_ERROR = 0, -1, -2, -3, -4
_STATUS = {0: "DT_OK", -1: "DT_INVALID", -2: "DT_NO_KERNEL", -3: "DT_OOM", -4: "DT_DEVICE_ERROR"}

# every symbol include/dt_hip.h declares
ABI_SYMBOLS = (
    "dt_version",
    "dt_init",
    "dt_qx_bytes",
    "dt_depalettize_f16",
    "dt_dense_qx_f16",
    "dt_dense_qx_heads_f16",
    "dt_dense_qx_grouped_f16",
    "dt_dense_qx_post_f16",
    "dt_qk_norm_rope_f16",
    "dt_layernorm_modulate_f16",
    "dt_layernorm_f16",
    "dt_sdpa_f16",
    "dt_sdpa_workspace_bytes",
    "dt_sdpa_f16_static",
    "dt_lora_branch_f32_f16",
)

STATIC_SCRATCH_BYTES = 64 << 20  # DT_SDPA_STATIC_SCRATCH_BYTES


class DtError(RuntimeError):
    def __init__(self, fn: str, status: int):
        super().__init__(f"{fn} failed: {_STATUS.get(status, status)}")
        self.status = status


class _QxWeight(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("qbits", ctypes.c_int32), ("nib", ctypes.c_int32), ("count", ctypes.c_int64)]


class _View4(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_s", ctypes.c_int64),
                ("stride_h", ctypes.c_int64)]


class _HeadEpilogue(ctypes.Structure):
    _fields_ = [("gamma", ctypes.c_void_p), ("rot", ctypes.c_void_p), ("rot_pos0", ctypes.c_int64),
                ("eps", ctypes.c_float), ("head_dim", ctypes.c_int32)]


class _DensePost(ctypes.Structure):
    _fields_ = [("activation", ctypes.c_int32), ("gate", ctypes.c_void_p), ("residual", ctypes.c_void_p),
                ("ld_residual", ctypes.c_int64), ("scale", ctypes.c_float), ("addend", ctypes.c_void_p),
                ("ld_addend", ctypes.c_int64), ("gate_f32", ctypes.c_void_p), ("multiplicand", ctypes.c_void_p),
                ("ld_multiplicand", ctypes.c_int64)]


class _DenseGroup(ctypes.Structure):
    _fields_ = [("M", ctypes.c_int64), ("K", ctypes.c_int64), ("X", ctypes.c_void_p), ("ldx", ctypes.c_int64),
                ("W", ctypes.c_void_p), ("n_weights", ctypes.c_int32), ("bias", ctypes.c_void_p),
                ("Y", ctypes.c_void_p), ("ldy", ctypes.c_void_p), ("epi", ctypes.c_void_p),
                ("post", ctypes.c_void_p)]


class _Segment(ctypes.Structure):
    _fields_ = [("view", _View4), ("len", ctypes.c_int64), ("gamma", ctypes.c_void_p)]


def build(verbose: bool = False) -> str:
    """Compile libdthip.so for gfx950 with the Makefile under csrc/ (always recompiles)."""
    cmd = ["make", "-C", CSRC, "-B", "-j8"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libdthip.so failed")
    return LIB_PATH


_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() or `make -C {CSRC}`; "
                "this package has no CPU or PyTorch fallback"
            )
        L = ctypes.CDLL(LIB_PATH)
        vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
        L.dt_version.restype = ctypes.c_char_p
        L.dt_version.argtypes = []
        L.dt_init.restype = i32
        L.dt_init.argtypes = [ctypes.c_int]
        L.dt_qx_bytes.restype = i64
        L.dt_qx_bytes.argtypes = [i32, i32, i64]
        L.dt_depalettize_f16.restype = i32
        L.dt_depalettize_f16.argtypes = [vp, ctypes.POINTER(_QxWeight), vp]
        L.dt_dense_qx_f16.restype = i32
        L.dt_dense_qx_f16.argtypes = [vp, i64, i64, vp, i64, ctypes.POINTER(_QxWeight), i32,
                                      ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(i64), ctypes.c_uint32]
        L.dt_dense_qx_heads_f16.restype = i32
        L.dt_dense_qx_heads_f16.argtypes = [vp, i64, i64, vp, i64, ctypes.POINTER(_QxWeight), i32,
                                            ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(i64),
                                            ctypes.POINTER(_HeadEpilogue), ctypes.c_uint32]
        L.dt_qk_norm_rope_f16.restype = i32
        L.dt_dense_qx_post_f16.restype = i32
        L.dt_dense_qx_post_f16.argtypes = [vp, i64, i64, vp, i64, ctypes.POINTER(_QxWeight), i32,
                                           ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(i64),
                                           ctypes.POINTER(_DensePost), ctypes.c_uint32]
        L.dt_dense_qx_grouped_f16.restype = i32
        L.dt_dense_qx_grouped_f16.argtypes = [vp, i32, ctypes.POINTER(_DenseGroup), ctypes.c_uint32]
        L.dt_qk_norm_rope_f16.argtypes = [vp, _View4, i32, i64, i32, i32, vp, f32, i32, vp, i64, f32]
        L.dt_layernorm_modulate_f16.restype = i32
        L.dt_layernorm_modulate_f16.argtypes = [vp, i64, i64, vp, i64, vp, vp, i32, f32, vp, i64]
        L.dt_layernorm_f16.restype = i32
        L.dt_layernorm_f16.argtypes = [vp, i64, i64, vp, i64, vp, vp, f32, vp, i64]
        L.dt_sdpa_f16.restype = i32
        L.dt_sdpa_f16.argtypes = [vp, i32, i32, i32, i32, i32, ctypes.POINTER(_Segment), i32,
                                  ctypes.POINTER(_Segment), ctypes.POINTER(_Segment), vp, vp, f32, _View4, f32,
                                  vp, vp, vp, ctypes.c_size_t]
        L.dt_sdpa_f16_static.restype = i32
        L.dt_sdpa_f16_static.argtypes = L.dt_sdpa_f16.argtypes[:-2]
        L.dt_lora_branch_f32_f16.restype = i32
        L.dt_lora_branch_f32_f16.argtypes = [vp, i64, i64, vp, i64, vp, i32, vp, i64, f32, vp, vp, i64]
        L.dt_sdpa_workspace_bytes.restype = ctypes.c_size_t
        L.dt_sdpa_workspace_bytes.argtypes = [i32, i32, i32, i32, i64, i64, i32, i32]
        _lib = L
    return _lib


def _check(fn: str, status: int):
    if status != DT_OK:
        raise DtError(fn, status)


def _torch():
    import torch

    return torch


def _stream_ptr(stream=None):
    torch = _torch()
    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


class _on:
    """Makes `stream` torch's current stream for the body of an operator, so that the tensors the operator
    allocates, the copies it makes (`clone`, `contiguous`) and the kernels it launches are all ordered on that one
    stream, and torch's allocator ties every temporary's reuse to it.  None = leave the current stream alone."""

    def __init__(self, stream):
        self.ctx = None if stream is None else _torch().cuda.stream(stream)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


def _stream_scoped(fn):
    """Runs an operator with its `stream=` argument as torch's current stream (see _on)."""
    import functools
    import inspect

    sig = inspect.signature(fn)

    @functools.wraps(fn)
    def wrapped(*args, **kwargs):
        stream = sig.bind(*args, **kwargs).arguments.get("stream")
        with _on(stream):
            return fn(*args, **kwargs)

    return wrapped


def _f16_cuda(t, name):
    torch = _torch()
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float16):
        raise TypeError(f"{name} must be a CUDA float16 tensor")
    return t


# --------------------------------------------------------------------------
# palettized weights
# --------------------------------------------------------------------------

# Elements per palette block for each codec.  Derived from the shipped model
# sizes (about 0.25 bit/weight of palette overhead for q6p/q8p, 0.5 for
# q4p/q5p); the library itself takes (qbits, nib) at run time.
CODEC = {"q4p": (4, 512), "q5p": (5, 1024), "q6p": (6, 4096), "q7p": (7, 8192), "q8p": (8, 16384)}


def qx_bytes(qbits: int, nib: int, count: int) -> int:
    return int(lib().dt_qx_bytes(qbits, nib, count))


def pack_indices(qbits: int, idx: np.ndarray) -> np.ndarray:
    """MSB-first bit stream of `qbits`-wide indices (host-side producer of the format).
    Eight indices always fill exactly `qbits` bytes: build each group as one 64-bit
    big-endian number and cut it into bytes."""
    idx = np.asarray(idx, dtype=np.uint8).reshape(-1)
    n = idx.size
    nbytes = (n * qbits + 7) // 8
    if qbits == 8:
        return idx.copy()
    groups = (n + 7) // 8
    padded = np.zeros(groups * 8, dtype=np.uint64)
    padded[:n] = idx & ((1 << qbits) - 1)
    padded = padded.reshape(groups, 8)
    val = np.zeros(groups, dtype=np.uint64)
    for j in range(8):
        val |= padded[:, j] << np.uint64(qbits * (7 - j))
    out = np.empty((groups, qbits), dtype=np.uint8)
    for i in range(qbits):
        out[:, i] = (val >> np.uint64(8 * (qbits - 1 - i))).astype(np.uint8)
    return out.reshape(-1)[:nbytes].copy()


def pack_qx(qbits: int, nib: int, palettes: np.ndarray, idx: np.ndarray) -> np.ndarray:
    """Packed buffer from per-block fp16 palettes [nblocks, 2^q] and indices [count]."""
    idx = np.asarray(idx, dtype=np.uint8).reshape(-1)
    palettes = np.ascontiguousarray(palettes, dtype=np.float16)
    count = idx.size
    nblocks = (count + nib - 1) // nib
    if palettes.shape != (nblocks, 1 << qbits):
        raise ValueError(f"palettes must be [{nblocks}, {1 << qbits}]")
    full = count // nib
    pal_bytes = 2 << qbits
    blk_bytes = nib * qbits // 8 if (nib * qbits) % 8 == 0 else None
    chunks = []
    if blk_bytes is not None and full > 0:
        # all full blocks at once
        packed = pack_indices(qbits, idx[: full * nib]).reshape(full, blk_bytes)
        body = np.empty((full, pal_bytes + blk_bytes), dtype=np.uint8)
        body[:, :pal_bytes] = palettes[:full].view(np.uint8).reshape(full, pal_bytes)
        body[:, pal_bytes:] = packed
        chunks.append(body.reshape(-1))
        start = full
    else:
        start = 0
    for b in range(start, nblocks):
        chunks.append(palettes[b].view(np.uint8).reshape(-1))
        chunks.append(pack_indices(qbits, idx[b * nib:(b + 1) * nib]))
    return np.concatenate(chunks) if chunks else np.zeros(0, np.uint8)


@dataclass
class QxTensor:
    """A weight as `store.read(codec: [.jit, .q?p])` leaves it: packed, on the device.

    qbits == 16 means a plain fp16 [out, in] tensor (data is then a float16 tensor)."""

    data: "object"  # torch uint8 (packed) or float16 tensor on the GPU
    qbits: int
    nib: int
    shape: tuple  # (out, in)

    @property
    def count(self) -> int:
        return int(self.shape[0]) * int(self.shape[1])

    def _c(self) -> _QxWeight:
        return _QxWeight(self.data.data_ptr(), self.qbits, self.nib, self.count)

    @staticmethod
    def from_packed(packed: np.ndarray, qbits: int, nib: int, shape, device="cuda") -> "QxTensor":
        torch = _torch()
        want = qx_bytes(qbits, nib, int(shape[0]) * int(shape[1]))
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        if packed.size != want:
            raise ValueError(f"packed buffer has {packed.size} bytes, layout needs {want}")
        # pad so the device buffer is a whole number of dwords
        buf = np.zeros((packed.size + 15) // 16 * 16, dtype=np.uint8)
        buf[: packed.size] = packed
        return QxTensor(torch.from_numpy(buf).to(device), qbits, nib, (int(shape[0]), int(shape[1])))

    @staticmethod
    def from_f16(w, device="cuda") -> "QxTensor":
        torch = _torch()
        if isinstance(w, np.ndarray):
            w = torch.from_numpy(np.ascontiguousarray(w, dtype=np.float16))
        w = w.to(device).contiguous()
        return QxTensor(w, 16, 0, tuple(w.shape))

    def dequantize(self, stream=None, out=None):
        """fp16 [out, in] tensor (K0): what a CPU read of the same key followed by Tensor<Float16>(from:) holds.
        `out`: a contiguous fp16 tensor of that shape to fill instead of a new one."""
        torch = _torch()
        if out is not None and (out.dtype != torch.float16 or tuple(out.shape) != tuple(self.shape)
                                or not out.is_contiguous() or out.device != self.data.device):
            raise ValueError("out must be a contiguous fp16 tensor of the weight's shape on its device")
        with _on(stream):
            if self.qbits == 16:
                return self.data.clone() if out is None else out.copy_(self.data)
            if out is None:
                out = torch.empty(self.shape, dtype=torch.float16, device=self.data.device)
            w = self._c()
            _check("dt_depalettize_f16", lib().dt_depalettize_f16(_stream_ptr(stream), ctypes.byref(w), out.data_ptr()))
            return out


# --------------------------------------------------------------------------
# operators (names and argument meaning follow the reference's Model DSL)
# --------------------------------------------------------------------------

class GEMMFlag:
    """Functional.GEMMFlag: permissions to compute at a given precision, not requests (Models/Flux1.swift:134, 162,
    229-231).  `Int8` is what FlashAttentionLevel.quantized adds to an attention's flags (`[.Int8, .Float16]`,
    Models/UNetProtocol.swift:14-19): this library computes such calls with its fp16 kernel (fp16 operands, fp32
    accumulation and statistics), which every combination of these flags permits."""
    Float16 = 1
    Float32 = 2
    Int8 = 4


@dataclass
class HeadEpilogue:
    """Per-head RMSNorm and RoPE fused behind a Dense: gamma [head_dim] or None, rot [>= rot_pos0 + M, head_dim] or None."""

    gamma: "object" = None
    rot: "object" = None
    rot_pos0: int = 0
    eps: float = 1e-6
    head_dim: int = 128


def _marshal_dense(x, weights, biases, outs, epilogues):
    """ctypes arguments of one Dense problem; returns (keepalive, fields, outs, M, x2)."""
    torch = _torch()
    _f16_cuda(x, "x")
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    n = len(weights)
    W = (_QxWeight * n)(*[w._c() for w in weights])
    for w in weights:
        if w.shape[1] != K:
            raise ValueError(f"weight {w.shape} does not match input width {K}")
    if outs is None:
        outs = [torch.empty((M, w.shape[0]), dtype=torch.float16, device=x.device) for w in weights]
    vp = ctypes.c_void_p
    B = (vp * n)(*[None if b is None else _f16_cuda(b, "bias").data_ptr() for b in biases])
    Y = (vp * n)(*[o.data_ptr() for o in outs])
    LDY = (ctypes.c_int64 * n)(*[o.stride(0) for o in outs])
    E = None
    if epilogues is not None:
        E = (_HeadEpilogue * n)()
        for i, e in enumerate(epilogues):
            if e is None:
                E[i] = _HeadEpilogue(None, None, 0, 0.0, 128)
                continue
            if e.rot is not None:
                _f16_cuda(e.rot, "rot")
                if e.rot.dim() != 2 or e.rot.shape[1] != e.head_dim or not e.rot.is_contiguous() \
                        or e.rot.shape[0] < e.rot_pos0 + M:
                    raise ValueError("rot must be a contiguous [>= rot_pos0 + M, head_dim] table")
            if e.gamma is not None and (_f16_cuda(e.gamma, "gamma").numel() != e.head_dim or not e.gamma.is_contiguous()):
                raise ValueError("gamma must hold head_dim elements")
            E[i] = _HeadEpilogue(None if e.gamma is None else e.gamma.data_ptr(),
                                 None if e.rot is None else e.rot.data_ptr(), e.rot_pos0, e.eps, e.head_dim)
    return (x2, M, K, n, W, B, Y, LDY, E, outs)


def _shape_outs(x, M, outs):
    lead = tuple(x.shape[:-1])
    return [o.reshape(lead + (o.shape[-1],)) if o.shape[0] == M and o.is_contiguous() else o for o in outs]


def dense_multi(x, weights: Sequence[QxTensor], biases: Sequence[Optional[object]], outs=None, flags: int = 0,
                stream=None, epilogues: Optional[Sequence[Optional[HeadEpilogue]]] = None):
    """Several Dense ops that share the input, one launch (x_q / x_k / x_v).  `epilogues[i]` (optional) fuses the
    per-head RMSNorm / RoPE that follows projection i."""
    with _on(stream):
        x2, M, K, n, W, B, Y, LDY, E, outs = _marshal_dense(x, weights, biases, outs, epilogues)
        if E is None:
            st = lib().dt_dense_qx_f16(_stream_ptr(stream), M, K, x2.data_ptr(), x2.stride(0), W, n, B, Y, LDY, flags)
            _check("dt_dense_qx_f16", st)
        else:
            st = lib().dt_dense_qx_heads_f16(_stream_ptr(stream), M, K, x2.data_ptr(), x2.stride(0), W, n, B, Y, LDY, E, flags)
            _check("dt_dense_qx_heads_f16", st)
        return _shape_outs(x, M, outs)


ACT_NONE, ACT_GELU_TANH, ACT_SWISH, ACT_GELU_ERF = 0, 1, 2, 3


class DensePost:
    """Elementwise tail of one projection, in this order: scalar `scale`, fp16 `addend` [M, N] (the low-rank branch of a
    LoRADense, Models/LoRA.swift:117-140; a residual of an fp16 stream), fp16 `multiplicand` [M, N] (the gated
    feed-forward `fc10(x) .* GELU()(fc11(x))`, Models/UNet.swift:510-513), activation (ACT_*), per-feature fp16 gate [N], fp32 residual [M, N] that the
    result is accumulated into (`x + (y .* gate).to(of: x)`, Models/Flux1.swift:250).  A float32 gate multiplies in
    fp32 on the way into the residual instead (`x + out.to(of: x) .* chunks[2]`, Models/Wan.swift:159).  With
    `residual` given and `keep_output=False` the fp16 result itself is not written."""

    def __init__(self, activation: int = ACT_NONE, gate=None, residual=None, keep_output: bool = True,
                 scale: float = 1.0, addend=None, multiplicand=None):
        self.activation, self.gate, self.residual, self.keep_output = activation, gate, residual, keep_output
        self.scale, self.addend, self.multiplicand = scale, addend, multiplicand


def _marshal_posts(posts, weights, M, Y, outs):
    """dt_dense_post array for the DensePost tails of one problem; clears Y / outs entries that only accumulate."""
    torch = _torch()
    n = len(weights)
    P = (_DensePost * n)()
    for i, p in enumerate(posts):
        if p is None:
            P[i] = _DensePost(ACT_NONE, None, None, 0, 1.0, None, 0, None, None, 0)
            continue
        N = weights[i].shape[0]
        if float(p.scale) == 0.0:
            # dt_dense_post.scale == 0 means "no scale" in the C ABI (a zero-initialised struct is a plain Dense)
            raise ValueError("DensePost.scale must not be 0 (the library reads 0 as 'no scale'); a zero result "
                             "needs no Dense")
        g16 = g32 = None
        if p.gate is not None:
            if isinstance(p.gate, torch.Tensor) and p.gate.dtype == torch.float32:  # product formed in fp32 (Wan)
                if not p.gate.is_cuda:
                    raise TypeError("gate must be a CUDA tensor")
                g32 = p.gate
            else:
                g16 = _f16_cuda(p.gate, "gate")
            if p.gate.numel() != N or not p.gate.is_contiguous():
                raise ValueError("gate must hold one value per output feature")
        rp, ldr = None, 0
        if p.residual is not None:
            r = p.residual
            if not (isinstance(r, torch.Tensor) and r.is_cuda and r.dtype == torch.float32):
                raise TypeError("residual must be a float32 CUDA tensor")
            r2 = r.reshape(-1, N) if r.dim() != 2 else r
            if r2.shape != (M, N) or r2.stride(1) != 1 or r2.data_ptr() != r.data_ptr():
                raise ValueError("residual must be an [M, N] view with contiguous rows")
            rp, ldr = r2.data_ptr(), r2.stride(0)
            if not p.keep_output:
                Y[i] = None
                outs[i] = None
        ap, lda = None, 0
        if p.addend is not None:
            a2 = _f16_cuda(p.addend, "addend")
            a2 = a2.reshape(-1, N) if a2.dim() != 2 else a2
            if a2.shape != (M, N) or a2.stride(1) != 1 or a2.data_ptr() != p.addend.data_ptr():
                raise ValueError("addend must be an [M, N] view with contiguous rows")
            ap, lda = a2.data_ptr(), a2.stride(0)
        mp, ldm = None, 0
        if p.multiplicand is not None:
            m2 = _f16_cuda(p.multiplicand, "multiplicand")
            m2 = m2.reshape(-1, N) if m2.dim() != 2 else m2
            if m2.shape != (M, N) or m2.stride(1) != 1 or m2.data_ptr() != p.multiplicand.data_ptr():
                raise ValueError("multiplicand must be an [M, N] view with contiguous rows")
            mp, ldm = m2.data_ptr(), m2.stride(0)
        P[i] = _DensePost(p.activation, None if g16 is None else g16.data_ptr(), rp, ldr, float(p.scale), ap, lda,
                          None if g32 is None else g32.data_ptr(), mp, ldm)
    return P


def dense_post(x, weights: Sequence[QxTensor], biases: Sequence[Optional[object]], posts: Sequence[Optional[DensePost]],
               outs=None, flags: int = 0, stream=None):
    """Dense ops sharing `x`, each followed by its DensePost tail inside the GEMM epilogue (the feed-forward's
    linear1 -> GELU and the gated residual additions of a transformer block).  Returns the fp16 outputs (None where
    a projection only accumulates into its residual)."""
    with _on(stream):
        x2, M, K, n, W, B, Y, LDY, _, outs = _marshal_dense(x, weights, biases, outs, None)
        P = _marshal_posts(posts, weights, M, Y, outs)
        st = lib().dt_dense_qx_post_f16(_stream_ptr(stream), M, K, x2.data_ptr(), x2.stride(0), W, n, B, Y, LDY, P, flags)
        _check("dt_dense_qx_post_f16", st)
    lead = tuple(x.shape[:-1])
    return [None if o is None else (o.reshape(lead + (o.shape[-1],)) if o.shape[0] == M and o.is_contiguous() else o)
            for o in outs]


def dense_grouped(problems: Sequence[dict], flags: int = 0, stream=None):
    """Independent Dense problems enqueued together (the context and image projections of a joint block).  Each
    problem is a dict with the arguments of dense_multi or dense_post: x, weights, biases, and optionally outs and
    either epilogues or posts.  Returns one list of outputs per problem (None where a projection only accumulates
    into its residual)."""
    with _on(stream):
        return _dense_grouped(problems, flags, stream)


def _dense_grouped(problems, flags, stream):
    keep = [_marshal_dense(p["x"], p["weights"], p["biases"], p.get("outs"), p.get("epilogues")) for p in problems]
    G = (_DenseGroup * len(keep))()
    cast = lambda a: None if a is None else ctypes.addressof(a)  # the arrays stay alive in `keep` until the call returns
    posts = []
    for i, (x2, M, K, n, W, B, Y, LDY, E, outs) in enumerate(keep):
        P = None
        if problems[i].get("posts") is not None:
            P = _marshal_posts(problems[i]["posts"], problems[i]["weights"], M, Y, outs)
        posts.append(P)
        G[i] = _DenseGroup(M, K, x2.data_ptr(), x2.stride(0), cast(W), n, cast(B), cast(Y), cast(LDY), cast(E), cast(P))
    st = lib().dt_dense_qx_grouped_f16(_stream_ptr(stream), len(keep), G, flags)
    _check("dt_dense_qx_grouped_f16", st)
    return [[None if o is None else _shape_outs(p["x"], k[1], [o])[0] for o in k[9]] for p, k in zip(problems, keep)]


class Dense:
    """Dense(count:noBias:flags:name:) -- y = x W^T + b with W [count, in] (Models/Flux1.swift:161-176)."""

    def __init__(self, count: int, noBias: bool = False, flags: int = 0, name: str = ""):
        self.count, self.noBias, self.flags, self.name = count, noBias, flags, name
        self.weight: Optional[QxTensor] = None
        self.bias = None

    def __call__(self, x, stream=None):
        if self.weight is None:
            raise RuntimeError(f"Dense {self.name!r}: weight not loaded")
        if self.weight.shape[0] != self.count:
            raise ValueError(f"Dense {self.name!r}: weight has {self.weight.shape[0]} rows, count is {self.count}")
        b = None if self.noBias else self.bias
        return dense_multi(x, [self.weight], [b], flags=self.flags, stream=stream)[0]


class LoRANetworkConfiguration:
    """rank / scale / highPrecision of the low-rank branch (Models/LoRA.swift:4-22)."""

    def __init__(self, rank: int, scale: float = 1.0, highPrecision: bool = False):
        self.rank, self.scale, self.highPrecision = rank, scale, highPrecision


class LoRADense:
    """LoRADense(count:configuration:noBias:flags:name:) -- dense(x) + up(scale * down(x)) with the palettized base
    left packed and the fp16 low-rank pair applied beside it (Models/LoRA.swift:85-142; running the LoRA separately
    is the preferred mode for quantized models, Models/UNetProtocol.swift:696-697).  Three launches of the Dense
    kernel: down (with the scale in its epilogue) beside the base projection, then up, whose epilogue adds the base
    projection's result; every intermediate is rounded to fp16 as the reference's separate ops round.  With
    `highPrecision` the pair is fp32 (`down.data` / `up.data` float32 tensors): the branch is computed as
    fp16(up(scale * down(float(x)))) in fp32 throughout (Models/LoRA.swift:117-139) by dt_lora_branch_f32_f16 and added
    in the base projection's epilogue."""

    def __init__(self, count: int, configuration: LoRANetworkConfiguration, noBias: bool = False, flags: int = 0,
                 name: str = ""):
        self.count, self.configuration, self.noBias, self.flags, self.name = count, configuration, noBias, flags, name
        self.weight: Optional[QxTensor] = None
        self.bias = None
        self.down: Optional[QxTensor] = None  # [rank, in] fp16
        self.up: Optional[QxTensor] = None    # [count, rank] fp16

    def _padded(self):
        """The pair with the rank padded by zero rows / columns to the tiled kernel's K granule (64): the zeros add
        nothing, so the results are the same bit for bit, and the up projection avoids the slow any-shape kernel."""
        # keyed on the identity of the pair's tensors (held here, so that their addresses cannot be handed to other
        # tensors while the cache lives), their in-place modification counters, the rank and the count
        src = (self.down.data, self.up.data)
        key = (self.down.data._version, self.up.data._version, self.configuration.rank, self.count,
               tuple(self.down.shape), tuple(self.up.shape))
        held = getattr(self, "_pad_src", None)
        if held is None or held[0] is not src[0] or held[1] is not src[1] or getattr(self, "_pad_key", None) != key:
            self._pad_src = src
            r = self.configuration.rank
            rp = (r + 63) // 64 * 64
            dn, up = self.down, self.up
            if rp != r and self.down.qbits == 16 and self.up.qbits == 16:
                torch = _torch()
                d = torch.zeros((rp, dn.shape[1]), dtype=torch.float16, device=dn.data.device)
                d[:r] = dn.data
                u = torch.zeros((self.count, rp), dtype=torch.float16, device=up.data.device)
                u[:, :r] = up.data
                dn, up = QxTensor(d, 16, 0, tuple(d.shape)), QxTensor(u, 16, 0, tuple(u.shape))
            self._pad_key, self._pad = key, (dn, up)
        return self._pad

    def __call__(self, x, post: Optional[DensePost] = None, stream=None):
        if self.weight is None:
            raise RuntimeError(f"LoRADense {self.name!r}: weight not loaded")
        b = None if self.noBias else self.bias
        # no matching LoRA keys: plain Dense.  A scale of zero makes the branch up(0 * down(x)) = 0 exactly, and
        # adding zero changes nothing: the same plain Dense
        if self.configuration.rank <= 0 or self.down is None or self.up is None or self.configuration.scale == 0:
            if post is None:
                return dense_multi(x, [self.weight], [b], flags=self.flags, stream=stream)[0]
            return dense_post(x, [self.weight], [b], [post], flags=self.flags, stream=stream)[0]
        if self.down.shape[0] != self.configuration.rank or self.up.shape != (self.count, self.configuration.rank):
            raise ValueError(f"LoRADense {self.name!r}: down / up shapes do not match rank and count")
        p = post or DensePost()
        if p.scale != 1.0 or p.addend is not None or p.multiplicand is not None:
            raise ValueError(f"LoRADense {self.name!r}: the tail may carry an activation, a gate and a residual only")
        if self.configuration.highPrecision:
            return self._high_precision(x, b, p, stream)
        dn, up = self._padded()
        # The down projection is a few dozen workgroups that wait on memory; the base projection does not depend on
        # it.  They go out side by side on two streams, and the up projection, whose epilogue adds the base
        # projection's result and then runs the tail, follows both.  (fp16(base) + fp16(branch) rounds the same
        # whichever of the two is the addend.)
        torch = _torch()
        main = stream if stream is not None else torch.cuda.current_stream(x.device)
        side = _side_stream(x.device)
        side.wait_stream(main)
        down = dense_post(x, [dn], [None], [DensePost(scale=self.configuration.scale)], stream=side)[0]
        base = dense_multi(x, [self.weight], [b], flags=self.flags, stream=main)[0]
        main.wait_stream(side)  # every use of x and `down` on the side stream is ordered before what follows on `main`
        # `down` came from the side stream's pool and is read on `main`: its memory must not go back to that pool's
        # next user before `main` has passed this point
        down.record_stream(main)
        tail = DensePost(p.activation, p.gate, p.residual, p.keep_output, addend=base.reshape(-1, self.count))
        out = dense_post(down, [up], [None], [tail], stream=main)[0]
        return None if out is None else out.reshape(*x.shape[:-1], self.count)


def _lora_high_precision(self, x, b, p, stream):
    """out = dense(x) + fp16(up32(scale * down32(float(x)))), then the tail: the fp32 branch beside the base projection
    on a second stream, the sum in the base projection's epilogue."""
    torch = _torch()
    dn, up = self.down.data, self.up.data
    if dn.dtype != torch.float32 or up.dtype != torch.float32 or not dn.is_contiguous() or not up.is_contiguous():
        raise TypeError(f"LoRADense {self.name!r}: highPrecision takes contiguous float32 down / up weights")
    _f16_cuda(x, "x")
    K, r = x.shape[-1], self.configuration.rank
    main = stream if stream is not None else torch.cuda.current_stream(x.device)
    with _on(main):  # a copy, if the view needs one, belongs on the caller's stream
        x2 = x.reshape(-1, K)
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
    M = x2.shape[0]
    side = _side_stream(x.device)
    side.wait_stream(main)
    with torch.cuda.stream(side):
        T = torch.empty((M, r), dtype=torch.float32, device=x.device)
        branch = torch.empty((M, self.count), dtype=torch.float16, device=x.device)
        st = lib().dt_lora_branch_f32_f16(_stream_ptr(side), M, K, x2.data_ptr(), x2.stride(0), dn.data_ptr(), r,
                                          up.data_ptr(), self.count, float(self.configuration.scale), T.data_ptr(),
                                          branch.data_ptr(), branch.stride(0))
        _check("dt_lora_branch_f32_f16", st)
    main.wait_stream(side)
    T.record_stream(main)
    branch.record_stream(main)
    tail = DensePost(p.activation, p.gate, p.residual, p.keep_output, addend=branch)
    out = dense_post(x2, [self.weight], [b], [tail], flags=self.flags, stream=main)[0]
    return None if out is None else out.reshape(*x.shape[:-1], self.count)


LoRADense._high_precision = _lora_high_precision

_SIDE_STREAMS = {}


def _side_stream(device):
    """One extra stream per device (default priority) for work that may run beside the caller's stream."""
    torch = _torch()
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


def _view4(t) -> _View4:
    if t.dim() != 4 or t.stride(3) != 1:
        raise ValueError("expected a [B, S, H, D] tensor with contiguous D")
    return _View4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def qk_norm_rope_(x, gamma=None, eps: float = 1e-6, norm_per_head: bool = True, rot=None, rot_pos0: int = 0,
                  post_scale: float = 1.0, stream=None):
    """In place on [B, S, H, D]: RMSNorm (per head, or over the whole row), then cmul with `rot`, then a scale."""
    _f16_cuda(x, "x")
    B, S, H, D = x.shape
    if rot is not None:
        _f16_cuda(rot, "rot")
        if rot.dim() != 2 or rot.shape[1] != D or not rot.is_contiguous() or rot.shape[0] < rot_pos0 + S:
            raise ValueError("rot must be a contiguous [>= rot_pos0 + S, D] table")
    if gamma is not None:
        _f16_cuda(gamma, "gamma")
        want = D if norm_per_head else H * D
        if gamma.numel() != want or not gamma.is_contiguous():
            raise ValueError(f"gamma must hold {want} elements")
    st = lib().dt_qk_norm_rope_f16(
        _stream_ptr(stream), _view4(x), B, S, H, D, None if gamma is None else gamma.data_ptr(), eps,
        1 if norm_per_head else 0, None if rot is None else rot.data_ptr(), rot_pos0, post_scale)
    _check("dt_qk_norm_rope_f16", st)
    return x


class RMSNorm:
    """RMSNorm(epsilon:axis:name:) on [B, S, H, D] (axis [3], per head) or [B, S, C] (axis [2], whole row)."""

    def __init__(self, epsilon: float, axis: Sequence[int], name: str = ""):
        self.epsilon, self.axis, self.name = epsilon, list(axis), name
        self.weight = None

    def __call__(self, x, stream=None):
        with _on(stream):
            y = x.clone()
            if x.dim() == 4 and self.axis == [3]:
                return qk_norm_rope_(y, self.weight, self.epsilon, True, stream=stream)
            if x.dim() == 3 and self.axis == [2]:
                qk_norm_rope_(_as_heads(y), self.weight, self.epsilon, False, stream=stream)
                return y
            raise DtError("RMSNorm", DT_NO_KERNEL)


MOD_F16, MOD_F32, MOD_AFFINE_F32 = 0, 1, 2


@_stream_scoped
def layernorm_modulate(x, scale=None, shift=None, epsilon: float = 1e-6, out=None, stream=None, affine: bool = False):
    """LayerNorm(epsilon:, axis: [last], elementwiseAffine: false) of the fp32 stream `x` [..., C], then the adaLN
    modulation, fp16 out.  fp16 `scale` / `shift` [C]: `norm(x).to(.Float16) .* scale + shift` (Models/Flux1.swift:
    172-173); fp32 ones: `(norm(x) .* (scale + 1) + shift).to(.Float16)` (Models/Wan.swift:217-221), or with
    `affine=True` the LayerNorm's own fp32 weight and bias, `norm(x) * scale + shift` (Models/Wan.swift:160-161)."""
    torch = _torch()
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == torch.float32):
        raise TypeError("x must be a float32 CUDA tensor")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    mods = [t for t in (scale, shift) if t is not None]
    dtypes = {t.dtype for t in mods}
    if len(dtypes) > 1 or not dtypes <= {torch.float16, torch.float32}:
        raise TypeError("scale and shift must both be float16 or both be float32")
    for t in mods:
        if not t.is_cuda or t.numel() != C or not t.is_contiguous():
            raise ValueError("scale / shift must be contiguous CUDA vectors of C elements")
    mod = MOD_F32 if dtypes == {torch.float32} else MOD_F16
    if affine:
        if mod != MOD_F32:
            raise TypeError("affine LayerNorm takes float32 weight and bias")
        mod = MOD_AFFINE_F32
    if out is None:
        out = torch.empty((M, C), dtype=torch.float16, device=x.device)
    elif out.dtype != torch.float16 or out.shape != (M, C) or out.stride(1) != 1:
        raise ValueError("out must be an [M, C] float16 view with contiguous rows")
    st = lib().dt_layernorm_modulate_f16(_stream_ptr(stream), M, C, x2.data_ptr(), x2.stride(0),
                                         None if scale is None else scale.data_ptr(),
                                         None if shift is None else shift.data_ptr(), mod, float(epsilon),
                                         out.data_ptr(), out.stride(0))
    _check("dt_layernorm_modulate_f16", st)
    return out.reshape(tuple(x.shape[:-1]) + (C,)) if out.is_contiguous() else out


@_stream_scoped
def layernorm16(x, weight=None, bias=None, epsilon: float = 1e-5, out=None, stream=None):
    """LayerNorm(epsilon:, axis: [last]) with fp16 affine `weight` / `bias` [C] on an fp16 tensor [..., C], fp16 out
    (the norms of a UNet transformer block, Models/UNet.swift:530, 544, 554)."""
    torch = _torch()
    _f16_cuda(x, "x")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    for t in (weight, bias):
        if t is not None and (_f16_cuda(t, "weight / bias").numel() != C or not t.is_contiguous()):
            raise ValueError("weight / bias must be contiguous vectors of C elements")
    if out is None:
        out = torch.empty((M, C), dtype=torch.float16, device=x.device)
    elif out.dtype != torch.float16 or out.shape != (M, C) or out.stride(1) != 1:
        raise ValueError("out must be an [M, C] float16 view with contiguous rows")
    st = lib().dt_layernorm_f16(_stream_ptr(stream), M, C, x2.data_ptr(), x2.stride(0),
                                None if weight is None else weight.data_ptr(), None if bias is None else bias.data_ptr(),
                                float(epsilon), out.data_ptr(), out.stride(0))
    _check("dt_layernorm_f16", st)
    return out.reshape(tuple(x.shape[:-1]) + (C,)) if out.is_contiguous() else out


class LayerNorm:
    """LayerNorm(epsilon:axis:elementwiseAffine:) on the last axis.  Of an fp32 tensor, result cast to fp16
    (`xNorm1(x).to(.Float16)`, Models/Flux1.swift:172-173; with fp32 `weight` / `bias` `xNorm3(out).to(.Float16)`,
    Models/Wan.swift:160-161); of an fp16 tensor with fp16 `weight` / `bias` (Models/UNet.swift:530)."""

    def __init__(self, epsilon: float, axis: Sequence[int], elementwiseAffine: bool = True, name: str = ""):
        self.epsilon, self.axis, self.elementwiseAffine, self.name = epsilon, list(axis), elementwiseAffine, name
        self.weight = None
        self.bias = None

    def __call__(self, x, stream=None):
        if self.axis != [x.dim() - 1]:
            raise ValueError("LayerNorm: only the last axis is supported")
        if x.dtype == _torch().float16:
            if self.elementwiseAffine and (self.weight is None or self.bias is None):
                raise RuntimeError(f"LayerNorm {self.name!r}: weight / bias not loaded")
            return layernorm16(x, self.weight if self.elementwiseAffine else None,
                               self.bias if self.elementwiseAffine else None, self.epsilon, stream=stream)
        if not self.elementwiseAffine:
            return layernorm_modulate(x, None, None, self.epsilon, stream=stream)
        if self.weight is None or self.bias is None:
            raise RuntimeError(f"LayerNorm {self.name!r}: weight / bias not loaded")
        return layernorm_modulate(x, self.weight, self.bias, self.epsilon, stream=stream, affine=True)


def _as_heads(y):
    B, S, C = y.shape
    for d in (128, 64, 32, 16, 8, 2):
        if C % d == 0:
            return y.view(B, S, C // d, d)
    raise DtError("RMSNorm", DT_NO_KERNEL)


class Functional:
    @staticmethod
    def cmul(left, right, stream=None):
        """Complex multiply on adjacent pairs; `right` is the [1, S, 1, D] (or [S, D]) rotary table."""
        with _on(stream):
            y = left.clone()
            rot = right.reshape(-1, right.shape[-1]).contiguous()
            return qk_norm_rope_(y, None, 0.0, True, rot=rot, stream=stream)


class ScaledDotProductAttention:
    """ScaledDotProductAttention(scale:isCausal:hasAttentionMask:flags:multiHeadOutputProjectionFused:name:)
    (Models/Flux1.swift:228-232, Models/UNet.swift:122-155).  Inputs [B, S, H, D]; returns [B, Sq, Hq, D], or
    [B, Sq, Hq*D] when the unify-heads projection is fused (then `.weight` [HD, HD] fp16 and `.bias`)."""

    def __init__(self, scale: float, isCausal: bool = False, hasAttentionMask: bool = False, flags: int = 0,
                 multiHeadOutputProjectionFused: bool = False, name: str = ""):
        if isCausal or hasAttentionMask:
            raise DtError("ScaledDotProductAttention(isCausal/hasAttentionMask)", DT_NO_KERNEL)
        self.scale, self.flags, self.fused, self.name = float(scale), flags, multiHeadOutputProjectionFused, name
        self.weight = None
        self.bias = None

    def __call__(self, queries, keys, values, stream=None):
        return sdpa_segments([queries], [keys], [values], self.scale,
                             Wo=self.weight if self.fused else None, bo=self.bias if self.fused else None,
                             stream=stream)


@_stream_scoped
def sdpa_segments(q_segs, k_segs, v_segs, scale, gamma_q=None, gamma_k=None, rot_q=None, rot_k=None,
                  eps: float = 1e-6, Wo=None, bo=None, out=None, stream=None, static_scratch: bool = False):
    """Attention over a joint sequence given as segments (text || image without a concat).
    gamma_q / gamma_k: per-segment per-head RMSNorm weights (or None); rot_*: [S, D] tables.
    static_scratch: stage through the library's fixed per-GPU array (dt_sdpa_f16_static) instead of a workspace
    allocated here; with `out` given the call then allocates nothing.  Requests beyond STATIC_SCRATCH_BYTES raise
    DtError(DT_OOM); calls that may overlap on one GPU must not both use it."""
    torch = _torch()
    L = lib()
    for t in list(q_segs) + list(k_segs) + list(v_segs):
        _f16_cuda(t, "q/k/v")
    B, _, Hq, D = q_segs[0].shape
    Hk = k_segs[0].shape[2]
    Sq = sum(t.shape[1] for t in q_segs)
    Skv = sum(t.shape[1] for t in k_segs)
    nq, nk = len(q_segs), len(k_segs)
    gq = gamma_q or [None] * nq
    gk = gamma_k or [None] * nk

    def segs(ts, gs):
        arr = (_Segment * len(ts))()
        for i, (t, g) in enumerate(zip(ts, gs)):
            arr[i] = _Segment(_view4(t), t.shape[1], None if g is None else _f16_cuda(g, "gamma").data_ptr())
        return arr

    qa, ka, va = segs(q_segs, gq), segs(k_segs, gk), segs(v_segs, [None] * nk)
    # only K is staged for a fused norm / rotation (the queries are handled inside the attention kernel)
    prep = any(g is not None for g in gk) or rot_k is not None
    fused = Wo is not None
    if out is None:
        shape = (B, Sq, Hq * D) if fused else (B, Sq, Hq, D)
        out = torch.empty(shape, dtype=torch.float16, device=q_segs[0].device)
    if fused:
        ov = _View4(out.data_ptr(), out.stride(0), out.stride(1), 0)
    else:
        ov = _view4(out)
    rq = None if rot_q is None else _f16_cuda(rot_q, "rot_q").data_ptr()
    rk = None if rot_k is None else _f16_cuda(rot_k, "rot_k").data_ptr()
    wo = None if Wo is None else _f16_cuda(Wo, "Wo").data_ptr()
    bo_p = None if bo is None else _f16_cuda(bo, "bo").data_ptr()
    if static_scratch:
        st = L.dt_sdpa_f16_static(_stream_ptr(stream), B, Hq, Hk, D, nq, qa, nk, ka, va, rq, rk, eps, ov, scale, wo, bo_p)
        _check("dt_sdpa_f16_static", st)
        return out
    need = L.dt_sdpa_workspace_bytes(B, Hq, Hk, D, Sq, Skv, int(prep), int(fused))
    ws = torch.empty(max(need, 256) + 256, dtype=torch.uint8, device=out.device) if need else None
    ws_ptr = None
    if ws is not None:
        ws_ptr = (ws.data_ptr() + 255) & ~255
    st = L.dt_sdpa_f16(
        _stream_ptr(stream), B, Hq, Hk, D, nq, qa, nk, ka, va, rq, rk, eps, ov, scale, wo, bo_p, ws_ptr, need)
    _check("dt_sdpa_f16", st)
    return out


# --------------------------------------------------------------------------
# rotary tables (host side, as in the reference: computed on the CPU in double,
# stored as float, cast to fp16 on upload)
# --------------------------------------------------------------------------

def _axis_table(pos: np.ndarray, dim: int) -> np.ndarray:
    k = np.arange(dim // 2, dtype=np.float64)
    theta = pos.astype(np.float64)[:, None] * 1.0 / np.power(10000.0, k * 2 / dim)
    out = np.empty((pos.size, dim), dtype=np.float32)
    out[:, 0::2] = np.cos(theta)
    out[:, 1::2] = np.sin(theta)
    return out


def Flux1RotaryPositionEmbedding(height: int, width: int, tokenLength: int, referenceSizes=(), channels: int = 128):
    """[tokenLength + height*width + sum(ref), channels] float32 table (Models/Flux1.swift:5-119), heads = 1."""
    assert channels % 16 == 0
    dim0, dim1 = channels // 8, channels * 7 // 16
    pos0 = [np.zeros(tokenLength + height * width)]
    ys, xs = np.divmod(np.arange(height * width), width)
    pos1 = [np.zeros(tokenLength), ys]
    pos2 = [np.zeros(tokenLength), xs]
    h = w = 0
    for (rh, rw) in referenceSizes:
        hoff = woff = 0
        if rh + h > rw + w:
            woff = w
        else:
            hoff = h
        ys, xs = np.divmod(np.arange(rh * rw), rw)
        pos0.append(np.ones(rh * rw))
        pos1.append(ys + hoff)
        pos2.append(xs + woff)
        h, w = max(h, rh + hoff), max(w, rw + woff)
    p0, p1, p2 = (np.concatenate(p) for p in (pos0, pos1, pos2))
    return np.concatenate([_axis_table(p0, dim0), _axis_table(p1, dim1), _axis_table(p2, dim1)], axis=1)


def WanRotaryPositionEmbedding(height: int, width: int, time: int, channels: int = 128):
    """[time*height*width, channels] float32 table (Models/Wan.swift:5-46), heads = 1."""
    assert channels % 16 == 0
    dim1 = (channels // 6) * 2
    dim0 = channels - 2 * dim1
    i = np.arange(time * height * width)
    t, rem = np.divmod(i, height * width)
    y, x = np.divmod(rem, width)
    return np.concatenate([_axis_table(t, dim0), _axis_table(y, dim1), _axis_table(x, dim1)], axis=1)


# --------------------------------------------------------------------------
# work units (Models/InstructionCount/InstructionCount.swift:4-17)
# --------------------------------------------------------------------------

def DenseInstructionCount(rows: int, input: int, output: int) -> int:
    assert rows >= 0 and input >= 0 and output >= 0
    return rows * output * input


def ScaledDotProductAttentionInstructionCount(batchSize, heads, headDimension, sequenceDimensionA,
                                              sequenceDimensionB) -> int:
    return batchSize * heads * (2 * headDimension + 5) * sequenceDimensionA * sequenceDimensionB
