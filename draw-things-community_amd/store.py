"""Reader (and a small writer, for tests) of the `.ckpt` tensor container the reference stores weights in.

What the reference tree itself shows of the container (Scripts/qwen35_gguf_quant_csv.py:48-55, 113-135): an SQLite
file with a table `tensors` whose rows carry `name`, `datatype` and `dim` (a little-endian int32 array, unused axes
zero); datatype codes 16384 = F32, 131072 = F16, 262144 = F64, 524288 = BF16, 4 = I32, 8 = I64.  Keys look like
`__dit__[t-x_q-0-0]`; the last number is 0 for a layer's weight and 1 for its bias (Models/UNetProtocol.swift:995,
2067, 2245).  Large models keep their blobs in a sidecar `<file>-tensordata` (SwiftLLM/Sources/TensorData.swift:5-7).

What the tree does not show, and this module therefore takes as a working assumption that only a real file can
confirm: the `data` column holds the tensor's bytes; a palettized tensor's bytes are the per-block `palette, packed
indices` stream this library consumes; how the row marks its codec (here: any bits of `datatype` above the low 32 are
kept as `codec_id` and otherwise ignored).  Instead of trusting a marker, `read` recognises a palettized blob by its
length: the layout fixes `blocks * 2^q * 2 + ceil(count * q / 8)` bytes for each codec's (bits, block size), and no
two of the codecs give the same length for one element count.  Blobs that match neither the plain nor a palettized
length (the reference also compresses small tensors with its `ezm7` coder) and blobs kept in the sidecar are reported
as unreadable rather than guessed at.
"""
import os
import sqlite3
import struct
import urllib.parse
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import CODEC, QxTensor

DATATYPES = {16384: ("F32", np.float32), 131072: ("F16", np.float16), 262144: ("F64", np.float64),
             524288: ("BF16", None), 4: ("I32", np.int32), 8: ("I64", np.int64)}
_CODE_OF = {"F32": 16384, "F16": 131072, "F64": 262144, "I32": 4, "I64": 8}
_ELEMENT_BYTES = {"F32": 4, "F16": 2, "F64": 8, "BF16": 2, "I32": 4, "I64": 8}


def palettized_bytes(qbits: int, nib: int, count: int) -> int:
    """Length of a palettized fp16 tensor of `count` elements: per block of `nib` elements 2^q fp16 palette entries,
    then the block's indices, MSB first, padded to a byte at the end of each block."""
    total, left = 0, count
    while left > 0:
        n = min(nib, left)
        total += (2 << qbits) + (n * qbits + 7) // 8
        left -= n
    return total


@dataclass
class TensorInfo:
    name: str
    datatype: str            # "F16", "F32", ...
    shape: Tuple[int, ...]
    nbytes: int              # length of the stored blob
    codec: Optional[str]     # "q6p", ... when the blob has a palettized length; None for plain storage
    codec_id: int            # bits of the datatype column above the low 32 (as stored; not interpreted)
    readable: bool           # plain or palettized length; False for anything else


class Store:
    """`graph.openStore(path)`: `keys`, `read(key, codec:)`, `write(key, tensor:)` over the container's SQLite file."""

    def __init__(self, path: str, codecs: Optional[Dict[str, Tuple[int, int]]] = None, mode: str = "r"):
        """mode "r" (default): the file must exist and is opened read-only, as the reference's own reader checks
        first (Scripts/qwen35_gguf_quant_csv.py:113-121); "w": opened read-write, created with an empty `tensors`
        table if missing."""
        if mode not in ("r", "w"):
            raise ValueError("mode must be 'r' or 'w'")
        self.path, self.mode = path, mode
        self.codecs = dict(CODEC if codecs is None else codecs)
        if mode == "r":
            if not os.path.isfile(path):
                raise FileNotFoundError(path)
            self.db = sqlite3.connect("file:" + urllib.parse.quote(os.path.abspath(path)) + "?mode=ro", uri=True)
        else:
            self.db = sqlite3.connect(path)
            self.db.execute("CREATE TABLE IF NOT EXISTS tensors (name TEXT, type INTEGER, format INTEGER, datatype INTEGER, "
                            "dim BLOB, data BLOB, PRIMARY KEY (name))")

    def close(self):
        if self.mode == "w":
            self.db.commit()
        self.db.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def keys(self) -> List[str]:
        return [r[0] for r in self.db.execute("SELECT name FROM tensors ORDER BY name")]

    @staticmethod
    def _shape(dim: bytes) -> Tuple[int, ...]:
        dims = struct.unpack("<" + "i" * (len(dim) // 4), dim) if dim else ()
        return tuple(int(d) for d in dims if d > 0)

    def _classify(self, datatype: str, count: int, nbytes: int) -> Tuple[Optional[str], bool]:
        if nbytes == count * _ELEMENT_BYTES[datatype]:
            return None, True
        if datatype == "F16":
            hits = [n for n, (q, nib) in self.codecs.items() if palettized_bytes(q, nib, count) == nbytes]
            if len(hits) == 1:
                return hits[0], True
        return None, False

    def info(self, key: str) -> Optional[TensorInfo]:
        row = self.db.execute("SELECT datatype, dim, length(data) FROM tensors WHERE name = ?", (key,)).fetchone()
        if row is None:
            return None
        code, dim, nbytes = int(row[0]), row[1], int(row[2] or 0)
        name = DATATYPES.get(code & 0xffffffff, (str(code & 0xffffffff), None))[0]
        shape = self._shape(dim)
        count = int(np.prod(shape)) if shape else 0
        codec, ok = self._classify(name, count, nbytes) if name in _ELEMENT_BYTES else (None, False)
        return TensorInfo(key, name, shape, nbytes, codec, code >> 32, ok)

    def read(self, key: str, codec: Sequence[str] = ("jit",), device: str = "cuda"):
        """`store.read(key, codec: [.jit, .q6p, ...])` (Models/UNetProtocol.swift:2230-2233).  A palettized 2-D tensor
        comes back as the packed QxTensor when "jit" is among the codecs (the weight stays packed on the device) and
        dequantized to fp16 otherwise; plain tensors come back as torch tensors.  None if the key is missing; ValueError
        if the blob's length matches no known storage."""
        import torch
        inf = self.info(key)
        if inf is None:
            return None
        if not inf.readable:
            raise ValueError(f"{key}: {inf.nbytes} bytes for {inf.datatype}{list(inf.shape)} is neither plain nor a known "
                             "palettized length (compressed, or kept in the -tensordata sidecar)")
        blob = self.db.execute("SELECT data FROM tensors WHERE name = ?", (key,)).fetchone()[0]
        raw = np.frombuffer(blob, dtype=np.uint8)
        if inf.codec is None:
            dt = DATATYPES[_CODE_OF[inf.datatype]][1] if inf.datatype in _CODE_OF else None
            if dt is None:
                raise ValueError(f"{key}: {inf.datatype} tensors are not supported")
            return torch.from_numpy(raw.view(dt).reshape(inf.shape).copy()).to(device)
        q, nib = self.codecs[inf.codec]
        rows = inf.shape[0] if len(inf.shape) > 1 else 1
        shape2 = (rows, int(np.prod(inf.shape)) // rows)
        w = QxTensor.from_packed(raw, q, nib, shape2, device=device)
        if "jit" in codec and len(inf.shape) >= 2:
            return w
        return w.dequantize().reshape(inf.shape)

    def write(self, key: str, tensor, datatype: Optional[str] = None):
        """Stores a numpy array / torch tensor as plain bytes, or a QxTensor's packed stream as it is (the palette
        fitting of the reference's quantizer is not part of this library).  Needs a store opened with mode "w"."""
        if self.mode != "w":
            raise PermissionError(f"{self.path} was opened read-only")
        if isinstance(tensor, QxTensor):
            if tensor.qbits == 16:
                return self.write(key, tensor.data.cpu().numpy())
            n = palettized_bytes(tensor.qbits, tensor.nib, tensor.count)
            blob = tensor.data.cpu().numpy().tobytes()[:n]
            code, shape = _CODE_OF["F16"], tensor.shape
        else:
            arr = tensor.detach().cpu().numpy() if hasattr(tensor, "detach") else np.asarray(tensor)
            names = {np.dtype(np.float32): "F32", np.dtype(np.float16): "F16", np.dtype(np.float64): "F64",
                     np.dtype(np.int32): "I32", np.dtype(np.int64): "I64"}
            name = datatype or names[arr.dtype]
            blob, code, shape = np.ascontiguousarray(arr).tobytes(), _CODE_OF[name], arr.shape
        dims = list(shape) + [0] * (12 - len(shape))
        self.db.execute("INSERT OR REPLACE INTO tensors (name, type, format, datatype, dim, data) VALUES (?, 0, 0, ?, ?, ?)",
                        (key, code, struct.pack("<12i", *dims), blob))

    def read_model(self, model_key: str, layers: Dict[str, object], codec: Sequence[str] = ("jit",), device: str = "cuda"):
        """Fills `.weight` / `.bias` of the given layers (host mirrors with those attributes, keyed by the layer's
        name) from `__<model_key>__[t-<name>-0-0]` and `...-0-1]`; returns the names that had no weight in the file."""
        missing = []
        for name, layer in layers.items():
            w = self.read(f"__{model_key}__[t-{name}-0-0]", codec, device)
            if w is None:
                missing.append(name)
                continue
            if not isinstance(w, QxTensor):
                w = QxTensor.from_f16(w.half(), device=device)
            layer.weight = w
            b = self.read(f"__{model_key}__[t-{name}-0-1]", (), device)
            if b is not None and hasattr(layer, "bias"):
                layer.bias = b.half()
        return missing
