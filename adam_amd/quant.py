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

    kind   'q4_0' (codes = packed nibble bytes, even element low), 'q8_0' (codes = uint8 = int8+128),
           'q4_aff' (nibble codes with an explicit float32 scale and zero point per 32 weights:
           w = scale * code + zp, e.g. the sub-blocks of GGUF Q4_K)
           or 'q4_req' (float32 values in `data` that the device's own quantiser turns into 4-bit codes
           when they are scattered into the map, with `scale`, `zp` from each group's minimum and
           maximum: what the reference does with every weight type it has no direct form for)
    d      float16 block scales, row-major over blocks of 32 along K (None for 'q4_aff' / 'q4_req')
    """
    kind: str
    shape: tuple
    d: np.ndarray
    codes: np.ndarray
    scale: np.ndarray = None
    zp: np.ndarray = None
    data: np.ndarray = None

    @property
    def size(self):
        return int(self.shape[0]) * int(self.shape[1])

    def qparams(self):
        if self.kind in ('q4_aff', 'q4_req'):
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
        elif self.kind == 'q4_req':
            sub = QTensor(self.kind, (n, k), None, None, self.scale[g0:g1], self.zp[g0:g1], self.data[lo:lo + cnt])
        else:
            sub = QTensor(self.kind, (n, k), None if self.d is None else self.d[g0:g1], self.codes[lo // 2:(lo + cnt) // 2],
                          None if self.scale is None else self.scale[g0:g1], None if self.zp is None else self.zp[g0:g1])
        return sub.dequant()

    def dequant(self):
        """float32 [N, K]; (code - offset) * d, exact in float32 ('q4_aff': scale * code + zp, one rounding each;
        'q4_req': the same over the codes the device quantiser makes, code = clamp(round((x - zp) / max(scale,
        1e-10)), 0, 15) in float32 with ties to even -- shaders/src/q4/map_scatter.comp:26-31)."""
        if self.kind == 'q4_req':
            x = self.data.reshape(-1, QK)
            qf = (x - self.zp[:, None]) / np.maximum(self.scale, np.float32(1e-10))[:, None]
            c = np.clip(np.rint(qf), 0, 15).astype(np.float32)
            return (c * self.scale[:, None] + self.zp[:, None]).astype(np.float32).reshape(self.shape)
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


def from_gguf_q5_0(raw, shape, clip=True):
    """GGUF Q5_0 bytes (22 B/block: fp16 d, 32 high bits, 16 nibble bytes; w = d (q - 16), q = nibble | bit << 4)
    -> QTensor 'q8_0': the reference keeps such tensors in the 8-bit map with scale |d| and, as code, the signed
    5-bit value times the sign of d.  Its default path gets there by rounding w / |d| and clipping to [-16, 15]
    (adam/models/engine.py:1171-1179): exact except for q = 0 in a block with d < 0, whose value +16 is stored as
    15.  `clip=True` (default) gives those codes; `clip=False` keeps +16, which is what the reference's raw decode
    stores (engine.py:1155-1169, taken on one device family only) and is exact for every block.  A block with d = 0
    gets scale 1 and codes 0, as there."""
    n = int(shape[0]) * int(shape[1])
    nb = n // QK
    blk = np.frombuffer(raw, dtype=np.uint8)[:nb * 22].reshape(nb, 22)
    d = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).astype(np.float32)
    qh = np.ascontiguousarray(blk[:, 2:6]).view(np.uint32).reshape(nb)
    ql = blk[:, 6:22]
    lo = np.concatenate([ql & 0x0F, ql >> 4], axis=1).astype(np.int16)
    hi = ((qh[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(np.int16)
    q = (lo | (hi << 4)) - 16
    q = q * np.where(d < 0, -1, 1).astype(np.int16)[:, None]
    if clip:
        q = q.clip(-16, 15)
    q[d == 0] = 0
    scale = np.where(d != 0, np.abs(d), np.float32(1.0)).astype(np.float16)
    return QTensor('q8_0', tuple(shape), scale, (q + 128).astype(np.uint8).reshape(-1))


def decode_gguf_q6_k(raw, n):
    """GGUF Q6_K bytes (210 B / 256 weights: 128 bytes of low nibbles, 64 bytes of high bit pairs, 16 int8
    sub-block scales, fp16 d; w = d * sc * (q - 32)) -> float32[n], products taken in that order in float32
    (the reference's decoder, adam/loaders/gguf.py:339-364)."""
    nb = n // 256
    b = np.frombuffer(raw, dtype=np.uint8)[:nb * 210].reshape(nb, 210)
    ql = b[:, 0:128].reshape(nb, 2, 64)
    qh = b[:, 128:192].reshape(nb, 2, 32)
    sc = np.ascontiguousarray(b[:, 192:208]).view(np.int8).reshape(nb, 2, 8).astype(np.float32)
    d = np.ascontiguousarray(b[:, 208:210]).view(np.float16).reshape(nb).astype(np.float32)
    la, lb = ql[:, :, 0:32], ql[:, :, 32:64]
    q = np.stack([(la & 0x0F) | ((qh & 3) << 4), (lb & 0x0F) | (((qh >> 2) & 3) << 4),
                  (la >> 4) | (((qh >> 4) & 3) << 4), (lb >> 4) | (((qh >> 6) & 3) << 4)], axis=2)   # [nb, 2, 4, 32]
    q = q.astype(np.float32) - np.float32(32.0)
    # weight l of quarter j in half h uses sub-block scale 8 h + 2 j + l // 16
    idx = 2 * np.arange(4)[:, None] + (np.arange(32)[None, :] // 16)                              # [4, 32]
    s = sc[:, :, idx]                                                                            # [nb, 2, 4, 32]
    ds = (d[:, None, None, None] * s).astype(np.float32)
    return (ds * q).astype(np.float32).reshape(-1)[:n]


def decode_bf16(raw, n):
    """bfloat16 -> float32: the 16 bits are the upper half of the float."""
    return (np.frombuffer(raw, dtype=np.uint16)[:n].astype(np.uint32) << 16).view(np.float32)


def requantize_q4(w):
    """A float matrix as the reference uploads it when the file's type has no direct map form (Q6_K, F16, BF16,
    F32 matrices; adam/models/engine.py:1063-1071, :1086-1096): per 32 weights scale = (max - min) / 15 (1 when
    they are all equal), zero point = min, and the values themselves, which the device quantises on arrival."""
    shape = tuple(w.shape)
    x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, QK)
    mn = x.min(axis=1).astype(np.float64)
    mx = x.max(axis=1).astype(np.float64)
    scale = np.where(mx > mn, (mx - mn) / 15.0, 1.0).astype(np.float32)
    return QTensor('q4_req', shape, None, None, scale, mn.astype(np.float32), x.reshape(-1))
