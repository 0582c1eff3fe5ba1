"""GGUF files -> the block form the decode path uploads, without re-quantisation.

A GGUF file holds little-endian metadata (key / typed value pairs), tensor descriptors (name,
dimensions, ggml type, offset) and an aligned data section of ggml blocks.  The reference reads it
in adam/loaders/gguf.py:97-150 and decodes the blocks to float32 in :282-337; its engine then
turns Q4_0 / Q8_0 / Q4_K blocks back into map form -- linear codes plus one (scale, zero point)
per 32 weights -- at adam/models/engine.py:998-1043 and :1149-1154.  Here the blocks go straight
to that form:

  Q4_0  18 B / 32 weights: fp16 d, 16 bytes (low nibbles = weights 0..15, high = 16..31);
        w = d (q - 8)            -> scale d, zero point -8 d, nibbles re-ordered to map order
  Q8_0  34 B / 32 weights: fp16 d, 32 int8;  w = d q   -> code q + 128, scale d, zero point -128 d
  Q4_K  144 B / 256 weights: fp16 d, fp16 dmin, 12 bytes of 6-bit (sc, m) for 8 sub-blocks of 32,
        128 bytes of nibbles (per 64 weights: low nibbles = first 32, high = next 32);
        w = d sc q - dmin m      -> scale d sc, zero point -dmin m per sub-block

  Q5_0  22 B / 32 weights: fp16 d, 32 high bits, 16 nibble bytes; w = d (q - 16)
        -> 8-bit map: code sign(d) (q - 16) + 128, scale |d|, zero point -128 |d| (exact; reference
        engine.py:1171-1179 keeps Q5_0 with Q8_0 in its 8-bit map)

For these, only the ORDER of the codes changes (the map keeps weight i in nibble i % 2 of byte i / 2); codes,
scales and minima are the file's own, so the device computes with exactly the values a ggml decoder yields.

Types without a map form of their own -- Q6_K (210 B / 256 weights: w = d sc (q - 32), 6-bit q in low nibbles
plus bit pairs, 16 int8 sub-block scales), F16, BF16 and F32 matrices -- are decoded to float32 and take the route
the reference gives "all other types" (engine.py:585-589, :1063-1096): into the 4-bit map with scale =
(max - min) / 15 and zero point = min per 32 weights, the codes made by the map's own quantiser when the floats
are scattered into it.  That step loses precision by the reference's design; the parity target is the reference,
so it is kept.  One-dimensional tensors (norm weights) stay float32.  Any other ggml type raises
NotImplementedError naming the tensor.
"""
import mmap
import struct

import numpy as np

from .quant import (from_gguf_q4_0, from_gguf_q8_0, from_gguf_q4_k, from_gguf_q5_0, decode_gguf_q6_k, decode_bf16,
                    requantize_q4)

GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q5_0, GGML_Q8_0, GGML_Q4_K, GGML_Q6_K, GGML_BF16 = 0, 1, 2, 6, 8, 12, 14, 30
# weights, bytes per block
_BLOCK = {GGML_Q4_0: (32, 18), GGML_Q5_0: (32, 22), GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144), GGML_Q6_K: (256, 210)}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_T_STRING, _T_ARRAY = 8, 9


class GGUFFile:
    """Parsed header of one file; tensor data stays memory-mapped until asked for."""

    def __init__(self, path):
        self.path = path
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self._pos = 0
        if self._take(4) != b"GGUF":
            raise ValueError(f"{path}: not a GGUF file")
        self.version = self._scalar(4)
        if self.version not in (2, 3):
            raise ValueError(f"{path}: GGUF version {self.version} is not supported")
        n_tensors, n_kv = self._scalar(10), self._scalar(10)
        self.metadata = {}
        for _ in range(n_kv):
            key = self._string()
            self.metadata[key] = self._value(self._scalar(4))
        self.tensors = {}                      # name -> (shape rows-first, ggml type, offset in the data section)
        for _ in range(n_tensors):
            name = self._string()
            dims = [self._scalar(10) for _ in range(self._scalar(4))]
            gtype, off = self._scalar(4), self._scalar(10)
            self.tensors[name] = (tuple(reversed(dims)), gtype, off)
        align = int(self.metadata.get("general.alignment", 32))
        self.data_start = (self._pos + align - 1) // align * align

    def close(self):
        try:
            self._mm.close()
        except BufferError:      # a caller still holds a view of the mapping
            pass
        self._f.close()

    # ---- header primitives
    def _take(self, n):
        b = self._mm[self._pos:self._pos + n]
        if len(b) != n:
            raise ValueError(f"{self.path}: truncated header")
        self._pos += n
        return b

    def _scalar(self, t):
        fmt = _SCALAR[t]
        return struct.unpack(fmt, self._take(struct.calcsize(fmt)))[0]

    def _string(self):
        return self._take(self._scalar(10)).decode("utf-8", errors="replace")

    def _value(self, t):
        if t == _T_STRING:
            return self._string()
        if t == _T_ARRAY:
            et, n = self._scalar(4), self._scalar(10)
            if et in _SCALAR and et != 7:
                fmt = _SCALAR[et]
                a = np.frombuffer(self._take(n * struct.calcsize(fmt)), dtype=np.dtype(fmt)).tolist()
                return a
            return [self._value(et) for _ in range(n)]
        if t not in _SCALAR:
            raise ValueError(f"{self.path}: unknown metadata type {t}")
        return self._scalar(t)

    # ---- tensors
    def numel(self, name):
        return int(np.prod(self.tensors[name][0], dtype=np.int64))

    def raw(self, name):
        """The tensor's bytes as a uint8 view of the mapping."""
        shape, gtype, off = self.tensors[name]
        n = self.numel(name)
        if gtype in _BLOCK:
            per, size = _BLOCK[gtype]
            if shape[-1] % per:
                raise ValueError(f"{name}: row length {shape[-1]} is not a multiple of {per}")
            nbytes = n // per * size
        elif gtype == GGML_F32:
            nbytes = 4 * n
        elif gtype in (GGML_F16, GGML_BF16):
            nbytes = 2 * n
        else:
            raise NotImplementedError(f"{name}: ggml type {gtype} is not supported")
        lo = self.data_start + off
        if lo + nbytes > len(self._mm):
            raise ValueError(f"{name}: data runs past the end of the file")
        return np.frombuffer(self._mm, dtype=np.uint8, count=nbytes, offset=lo)

    def tensor(self, name):
        """float32 array (F32 / F16 / BF16 / Q6_K, decoded) or QTensor in map form (Q4_0, Q8_0, Q4_K blocks as
        they are; Q5_0 as signed 8-bit codes, adam/models/engine.py:1171-1179)."""
        shape, gtype, _ = self.tensors[name]
        raw = self.raw(name)
        if gtype == GGML_F32:
            return raw.view(np.float32).reshape(shape).copy()
        if gtype == GGML_F16:
            return raw.view(np.float16).astype(np.float32).reshape(shape)
        if gtype == GGML_BF16:
            return decode_bf16(raw, self.numel(name)).reshape(shape)
        if gtype == GGML_Q6_K:
            return decode_gguf_q6_k(raw, self.numel(name)).reshape(shape)
        if len(shape) != 2:
            shape = (int(np.prod(shape[:-1], dtype=np.int64)), shape[-1])
        if gtype == GGML_Q4_0:
            return from_gguf_q4_0(raw, shape)
        if gtype == GGML_Q8_0:
            return from_gguf_q8_0(raw, shape)
        if gtype == GGML_Q5_0:
            return from_gguf_q5_0(raw, shape)
        return from_gguf_q4_k(raw, shape)


class RowLookup:
    """Embedding rows of an untied model, decoded on the host one row at a time (the reference looks
    them up on the host as well, adam/models/engine.py:2986-2992)."""

    def __init__(self, source):
        self._t = source                       # QTensor or float32 [V, E]
        self.shape = tuple(source.shape)

    def row(self, tok):
        t, k = self._t, self.shape[1]
        if isinstance(t, np.ndarray):
            return np.ascontiguousarray(t[int(tok)], np.float32)
        return t.dequant_rows(int(tok), 1).reshape(k)

    def rows(self, lo, hi):
        """Rows lo .. hi-1 as one float32 [hi - lo, E] array (what a device-side table is filled from)."""
        t, k = self._t, self.shape[1]
        if isinstance(t, np.ndarray):
            return np.ascontiguousarray(t[lo:hi], np.float32)
        return t.dequant_rows(int(lo), int(hi - lo)).reshape(hi - lo, k)


def config_from_metadata(md, tensors):
    """ModelConfig from the file's metadata, with the reference's defaults
    (adam/models/engine.py:57-111); head sizes come from attention.key_length / value_length when
    present, else from the Q and K projection shapes."""
    from .engine import ModelConfig
    arch = md.get("general.architecture", "llama")
    g = lambda key, default: md.get(f"{arch}.{key}", md.get(key, default))
    c = ModelConfig(arch=arch)
    c.n_ctx = int(g("context_length", 4096))
    c.n_layer = int(g("block_count", 32))
    c.n_embd = int(g("embedding_length", 4096))
    c.n_ff = int(g("feed_forward_length", c.n_embd * 4))
    c.n_head = int(g("attention.head_count", 32))
    c.n_head_kv = int(g("attention.head_count_kv", c.n_head))
    c.norm_eps = float(g("attention.layer_norm_rms_epsilon", 1e-6))
    vocab = g("vocab_size", md.get("tokenizer.ggml.tokens"))
    if isinstance(vocab, list):
        vocab = len(vocab)
    if vocab is None and "token_embd.weight" in tensors:
        vocab = tensors["token_embd.weight"][0][0]
    c.n_vocab = int(vocab)
    q_rows = tensors.get("blk.0.attn_q.weight", ((c.n_embd,),))[0][0]
    k_rows = tensors.get("blk.0.attn_k.weight", ((c.n_embd // max(c.n_head, 1) * c.n_head_kv,),))[0][0]
    c.head_dim = int(g("attention.key_length", q_rows // max(c.n_head, 1)))
    c.head_dim_kv = int(g("attention.value_length", k_rows // max(c.n_head_kv, 1)))
    if arch == "gemma3":
        c.sliding_window = int(g("attention.sliding_window", 512))
        c.rope_base_global = float(g("rope.freq_base", 1e6))
        c.rope_base_local = float(g("rope.local_freq_base", c.rope_base_global))
    else:
        c.sliding_window = int(g("attention.sliding_window", 0))
        c.rope_base_global = float(g("rope.freq_base", 10000.0))
        c.rope_base_local = c.rope_base_global
    act = g("feed_forward.activation_type", None)
    gelu_archs = {"gemma", "gemma2", "gemma3", "gpt2", "gptj", "gptneox", "falcon", "starcoder", "starcoder2", "refact"}
    c.ffn_act = {8: "gelu", 9: "gelu", 10: "silu", 6: "relu"}.get(act, "silu") if act is not None else \
        ("gelu" if arch in gelu_archs else "silu")
    c.emb_scale = float(np.sqrt(float(c.n_embd))) if arch.startswith("gemma") else 1.0
    c.attn_softcap = float(g("attention.logit_softcapping", 0.0))
    c.final_softcap = float(g("logit_softcapping", 0.0))
    if arch == "gemma3":
        c.attn_softcap = c.attn_softcap or 50.0
        c.final_softcap = c.final_softcap or 30.0
    return c


def load_model(path):
    """(ModelConfig, dict name -> QTensor / float32 array / RowLookup) for DecodeEngine.

    With an `output.weight` tensor the model is untied: the embedding matrix stays on the host and is
    read row by row; without one the embedding matrix is also the LM head and goes to the device."""
    f = GGUFFile(path)
    cfg = config_from_metadata(f.metadata, f.tensors)
    out = {}
    for name in f.tensors:
        if name.startswith("rope_freqs") or not name.endswith(".weight"):
            continue
        out[name] = f.tensor(name)
    untied = "output.weight" in out
    for name, t in list(out.items()):
        # Weight matrices whose type has no map form of its own (Q6_K, F16, BF16, F32) go to the 4-bit map as the
        # reference sends them (adam/models/engine.py:585-589, :1063-1096): group minimum / maximum as qparams, the
        # float values quantised by the device on arrival.  Row length must fill whole groups of 32.
        if isinstance(t, np.ndarray) and t.ndim == 2 and not (untied and name == "token_embd.weight"):
            if t.shape[1] % 32:
                raise NotImplementedError(f"{name}: float matrix rows of {t.shape[1]} weights do not fill groups of 32")
            out[name] = requantize_q4(t)
    if untied:
        out["token_embd.weight"] = RowLookup(out["token_embd.weight"])
    f.close()
    return cfg, out
