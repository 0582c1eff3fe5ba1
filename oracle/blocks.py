"""Block-quantised weight formats used by the decode path (oracle side; test infrastructure).

Two views of the same data are needed:

* the GGUF on-disk block layouts (Q4_0: fp16 ``d`` + 16 nibble bytes, low nibbles are
  elements 0..15 and high nibbles 16..31; Q8_0: fp16 ``d`` + 32 int8), restated from the
  reference loader's decoders ``adam/loaders/gguf.py:282-299`` (block sizes ``:24-33``);
* the ADAMAH map form the reference engine uploads: linear codes (Q4: element ``i`` is
  nibble ``i % 8`` of little-endian word ``i // 8``, i.e. even element = low nibble of
  byte ``i // 2`` -- ``adam/models/engine.py:998-1011``; Q8: one byte per element holding
  ``int8 + 128`` -- ``engine.py:1149-1154``) plus per-32-group ``(scale, zero_point)`` with
  ``scale = d`` and ``zero_point = -8 d`` (Q4_0) or ``-128 d`` (Q8_0).

The reference tree holds no Q4_0/Q8_0 *quantiser*; the one here follows the benchmark
config's wording ("fp16 absmax/8 scale, 4-bit codes offset 8").  It runs on the host for
both the oracle and the HIP path, so parity never depends on its rounding choices.
"""
import numpy as np

QK = 32  # weights per block for both formats


def quantize_q4_0(w):
    """Quantise a float array (size divisible by 32, blocks along the last axis).

    d = fp16(max|x| / 8) per block (1.0 if that is zero), code = clip(rint(x / d) + 8, 0, 15).
    Returns (d as float16 [n_blocks], codes as uint8 [n] in 0..15), both flattened row-major.
    """
    x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, QK)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(8.0)).astype(np.float16)
    d32 = d.astype(np.float32)
    d32 = np.where(d32 > 0, d32, np.float32(1.0))
    d = d32.astype(np.float16)
    q = np.rint(x / d32[:, None]) + 8.0
    codes = np.clip(q, 0, 15).astype(np.uint8).reshape(-1)
    return d, codes


def quantize_q8_0(w):
    """d = fp16(max|x| / 127) per block (1.0 if zero), q = clip(rint(x / d), -127, 127).

    Returns (d float16 [n_blocks], q int8 [n]).
    """
    x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, QK)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float16)
    d32 = d.astype(np.float32)
    d32 = np.where(d32 > 0, d32, np.float32(1.0))
    d = d32.astype(np.float16)
    q = np.clip(np.rint(x / d32[:, None]), -127, 127).astype(np.int8).reshape(-1)
    return d, q


def dequant_q4_0(d, codes):
    """(code - 8) * d in float32 -- the value every layout below must reproduce bit-exactly."""
    d32 = np.asarray(d, dtype=np.float16).astype(np.float32)
    c = np.asarray(codes, dtype=np.uint8).reshape(-1, QK).astype(np.float32)
    return ((c - np.float32(8.0)) * d32[:, None]).reshape(-1)


def dequant_q8_0(d, q):
    d32 = np.asarray(d, dtype=np.float16).astype(np.float32)
    c = np.asarray(q, dtype=np.int8).reshape(-1, QK).astype(np.float32)
    return (c * d32[:, None]).reshape(-1)


# ---- ADAMAH map form -------------------------------------------------------------------

def pack_linear_nibbles(codes):
    """Codes 0..15 -> bytes, even element in the low nibble (engine.py:1003-1011)."""
    c = np.asarray(codes, dtype=np.uint8).reshape(-1)
    if c.size & 1:
        c = np.concatenate([c, np.zeros(1, np.uint8)])
    return (c[0::2] | (c[1::2] << 4)).astype(np.uint8)


def unpack_linear_nibbles(packed, n):
    p = np.asarray(packed, dtype=np.uint8).reshape(-1)
    out = np.empty(p.size * 2, np.uint8)
    out[0::2] = p & 0x0F
    out[1::2] = p >> 4
    return out[:n]


def q4_0_qparams(d):
    """ADAMAH per-group (scale, zero_point) equivalent to a Q4_0 block: (d, -8 d)."""
    s = np.asarray(d, dtype=np.float16).astype(np.float32)
    return s, (np.float32(-8.0) * s).astype(np.float32)


def q8_0_qparams(d):
    """(d, -128 d); codes are stored as uint8 = int8 + 128 (engine.py:1149-1154, 1192-1194)."""
    s = np.asarray(d, dtype=np.float16).astype(np.float32)
    return s, (np.float32(-128.0) * s).astype(np.float32)


def q8_to_u8(q):
    return (np.asarray(q, dtype=np.int8).astype(np.int16) + 128).astype(np.uint8)


# ---- GGUF on-disk blocks ---------------------------------------------------------------

def gguf_q4_0_bytes(d, codes):
    """Serialise to GGUF Q4_0 blocks: 2 B fp16 d, then 16 B with elems 0..15 low / 16..31 high."""
    d = np.asarray(d, dtype=np.float16)
    c = np.asarray(codes, dtype=np.uint8).reshape(-1, QK)
    nb = c.shape[0]
    blk = np.empty((nb, 18), np.uint8)
    blk[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    blk[:, 2:18] = c[:, :16] | (c[:, 16:] << 4)
    return blk.reshape(-1).tobytes()


def decode_gguf_q4_0(data, ne):
    """Restates GGUFLoader._dq4_0 (adam/loaders/gguf.py:290-299), vectorised."""
    nb = ne // QK
    blk = np.frombuffer(data, dtype=np.uint8)[:nb * 18].reshape(nb, 18)
    s = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).astype(np.float32)
    nib = blk[:, 2:18]
    out = np.empty((nb, QK), np.float32)
    out[:, :16] = ((nib & 0x0F).astype(np.float32) - 8) * s[:, None]
    out[:, 16:] = (((nib >> 4) & 0x0F).astype(np.float32) - 8) * s[:, None]
    return out.reshape(-1)


def gguf_q4_0_to_codes(data, ne):
    """GGUF Q4_0 bytes -> (d float16, linear codes) without touching the values."""
    nb = ne // QK
    blk = np.frombuffer(data, dtype=np.uint8)[:nb * 18].reshape(nb, 18)
    d = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).copy()
    nib = blk[:, 2:18]
    codes = np.concatenate([nib & 0x0F, nib >> 4], axis=1).astype(np.uint8).reshape(-1)
    return d, codes


def gguf_q8_0_bytes(d, q):
    d = np.asarray(d, dtype=np.float16)
    c = np.asarray(q, dtype=np.int8).reshape(-1, QK)
    nb = c.shape[0]
    blk = np.empty((nb, 34), np.uint8)
    blk[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    blk[:, 2:34] = c.view(np.uint8)
    return blk.reshape(-1).tobytes()


def decode_gguf_q8_0(data, ne):
    """Restates GGUFLoader._dq8 (adam/loaders/gguf.py:282-288), vectorised."""
    nb = ne // QK
    blk = np.frombuffer(data, dtype=np.uint8)[:nb * 34].reshape(nb, 34)
    s = np.ascontiguousarray(blk[:, 0:2]).view(np.float16).reshape(nb).astype(np.float32)
    q = np.ascontiguousarray(blk[:, 2:34]).view(np.int8).astype(np.float32)
    return (q * s[:, None]).reshape(-1)
