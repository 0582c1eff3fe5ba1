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

    kind   'q4_0' (codes = packed nibble bytes, even element low), 'q8_0' (codes = uint8 = int8+128)
           or 'q4_aff' (nibble codes with an explicit float32 scale and zero point per 32 weights:
           w = scale * code + zp, e.g. the sub-blocks of GGUF Q4_K)
    d      float16 block scales, row-major over blocks of 32 along K (None for 'q4_aff')
    """
    kind: str
    shape: tuple
    d: np.ndarray
    codes: np.ndarray
    scale: np.ndarray = None
    zp: np.ndarray = None

    @property
    def size(self):
        return int(self.shape[0]) * int(self.shape[1])

    def qparams(self):
        if self.kind == 'q4_aff':
            return self.scale, self.zp
        s = self.d.astype(np.float32)
        off = np.float32(-8.0 if self.kind == 'q4_0' else -128.0)
        return s, (off * s).astype(np.float32)

    def dequant_rows(self, row, n):
        """float32 [n, K] of rows row .. row + n - 1."""
        k = int(self.shape[1])
        lo, cnt = row * k, n * k
        g0, g1 = lo // QK, (lo + cnt) // QK
        if self.kind == 'q8_0':
            sub = QTensor(self.kind, (n, k), self.d[g0:g1], self.codes[lo:lo + cnt])
        else:
            sub = QTensor(self.kind, (n, k), None if self.d is None else self.d[g0:g1], self.codes[lo // 2:(lo + cnt) // 2],
                          None if self.scale is None else self.scale[g0:g1], None if self.zp is None else self.zp[g0:g1])
        return sub.dequant()

    def dequant(self):
        """float32 [N, K]; (code - offset) * d, exact in float32 ('q4_aff': scale * code + zp, one rounding each)."""
        if self.kind == 'q4_aff':
            c = np.empty(self.size, np.uint8)
            c[0::2] = self.codes & 0x0F
            c[1::2] = self.codes >> 4
            v = c.reshape(-1, QK).astype(np.float32) * self.scale[:, None] + self.zp[:, None]
            return v.reshape(self.shape)
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


def from_gguf_q4_k(raw, shape):
    """GGUF Q4_K bytes (144 B / 256 weights: fp16 d, fp16 dmin, 12 bytes of 6-bit scales and minima of
    the 8 sub-blocks, 128 nibble bytes; per 64 weights the low nibbles are the first 32) -> QTensor
    'q4_aff' with scale = d * sc and zero point = -dmin * m per sub-block (the values the reference
    extracts, adam/models/engine.py:1022-1043); nibbles re-ordered to map order, nothing re-quantised."""
    n = int(shape[0]) * int(shape[1])
    nb = n // 256
    b = np.frombuffer(raw, dtype=np.uint8)[:nb * 144].reshape(nb, 144)
    d = np.ascontiguousarray(b[:, 0:2]).view(np.float16).reshape(nb).astype(np.float32)
    dmin = np.ascontiguousarray(b[:, 2:4]).view(np.float16).reshape(nb).astype(np.float32)
    s = b[:, 4:16]
    sc = np.empty((nb, 8), np.uint8)
    mn = np.empty((nb, 8), np.uint8)
    sc[:, 0:4] = s[:, 0:4] & 63
    mn[:, 0:4] = s[:, 4:8] & 63
    sc[:, 4:8] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:8] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    scale = (d[:, None] * sc.astype(np.float32)).reshape(-1)
    zp = (-(dmin[:, None] * mn.astype(np.float32))).reshape(-1)
    q = b[:, 16:144].reshape(nb, 4, 32)
    c = np.stack([q & 0x0F, q >> 4], axis=2).reshape(-1)          # per 64 weights: low nibbles, then high
    return QTensor('q4_aff', tuple(shape), None, (c[0::2] | (c[1::2] << 4)).astype(np.uint8), scale, zp)
