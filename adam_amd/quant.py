"""Host-side packers for the block-quantised weight formats the decode path consumes.

GGUF Q4_0 / Q8_0 blocks (32 weights, fp16 scale ``d``) are turned into what the ADAMAH op
surface uploads: linear codes plus per-group ``(scale, zero_point)`` --
``scale = d, zp = -8 d`` for Q4_0 and ``scale = d, zp = -128 d`` with ``u8 = int8 + 128`` for
Q8_0 (reference: adam/models/engine.py:998-1011, :1149-1154; block layouts
adam/loaders/gguf.py:282-299).  The library recognises exactly these qparams and keeps
such maps as fp16-scale planes internally.
"""
from dataclasses import dataclass
import numpy as np

QK = 32


@dataclass
class QTensor:
    """A block-quantised matrix [N, K] in map form.

    kind   'q4_0' (codes = packed nibble bytes, even element low) or 'q8_0' (codes = uint8 = int8+128)
    d      float16 block scales, row-major over blocks of 32 along K
    """
    kind: str
    shape: tuple
    d: np.ndarray
    codes: np.ndarray

    @property
    def size(self):
        return int(self.shape[0]) * int(self.shape[1])

    def qparams(self):
        s = self.d.astype(np.float32)
        off = np.float32(-8.0 if self.kind == 'q4_0' else -128.0)
        return s, (off * s).astype(np.float32)

    def dequant(self):
        """float32 [N, K]; (code - offset) * d, exact in float32."""
        s = self.d.astype(np.float32)
        if self.kind == 'q4_0':
            c = np.empty(self.size, np.uint8)
            c[0::2] = self.codes & 0x0F
            c[1::2] = self.codes >> 4
            v = c.reshape(-1, QK).astype(np.float32) - np.float32(8.0)
        else:
            v = self.codes.reshape(-1, QK).astype(np.float32) - np.float32(128.0)
        return (v * s[:, None]).reshape(self.shape)


def _scales(x, div):
    amax = np.abs(x).max(axis=1)
    d32 = (amax / np.float32(div)).astype(np.float16).astype(np.float32)
    d32 = np.where(d32 > 0, d32, np.float32(1.0))
    return d32


def quantize_q4_0(w):
    """fp16 absmax/8 scale, codes = clip(rint(x/d) + 8, 0, 15), packed two per byte."""
    shape = tuple(w.shape)
    x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, QK)
    d32 = _scales(x, 8.0)
    c = np.clip(np.rint(x / d32[:, None]) + 8.0, 0, 15).astype(np.uint8).reshape(-1)
    return QTensor('q4_0', shape, d32.astype(np.float16), (c[0::2] | (c[1::2] << 4)).astype(np.uint8))


def quantize_q8_0(w):
    """fp16 absmax/127 scale, int8 codes stored as uint8 = q + 128."""
    shape = tuple(w.shape)
    x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, QK)
    d32 = _scales(x, 127.0)
    q = np.clip(np.rint(x / d32[:, None]), -127, 127).astype(np.int16)
    return QTensor('q8_0', shape, d32.astype(np.float16), (q + 128).astype(np.uint8).reshape(-1))


def from_gguf_q4_0(raw, shape):
    """GGUF Q4_0 bytes (18 B/block: d, 16 nibble bytes; low nibbles = elems 0..15) -> QTensor."""
    n = int(shape[0]) * int(shape[1])
    nb = n // QK
    blk = np.frombuffer(raw, dtype=np.uint8)[:nb * 18].reshape(nb, 18)
    d = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).copy()
    nib = blk[:, 2:18]
    c = np.concatenate([nib & 0x0F, nib >> 4], axis=1).reshape(-1)
    return QTensor('q4_0', tuple(shape), d, (c[0::2] | (c[1::2] << 4)).astype(np.uint8))


def from_gguf_q8_0(raw, shape):
    """GGUF Q8_0 bytes (34 B/block: d, 32 int8) -> QTensor."""
    n = int(shape[0]) * int(shape[1])
    nb = n // QK
    blk = np.frombuffer(raw, dtype=np.uint8)[:nb * 34].reshape(nb, 34)
    d = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).copy()
    q = np.ascontiguousarray(blk[:, 2:34]).view(np.int8).astype(np.int16)
    return QTensor('q8_0', tuple(shape), d, (q + 128).astype(np.uint8).reshape(-1))
