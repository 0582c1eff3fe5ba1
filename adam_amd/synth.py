"""Random-init models of the benchmark's architectures, already in uploadable block form.

Weights are N(0, sigma) float32 drawn per tensor from a seeded generator and quantised on the
host to Q4_0 (body; tied LM head) or Q8_0 (untied LM head), norm weights are 1.  Tensor
names follow GGUF (`blk.N.attn_q.weight`, ...), which is what the reference engine keys on
(adam/models/engine.py:518-609).
"""
import zlib
import numpy as np

from .engine import ModelConfig
from .quant import quantize_q4_0, quantize_q8_0


def gemma3_1b_config():
    """Gemma-3-1B shape: 26 layers, E=1152, 4 q / 1 kv heads of 256, GeGLU 6912, tied vocab 262144."""
    return ModelConfig(arch="gemma3", n_vocab=262144, n_ctx=32768, n_embd=1152, n_head=4, n_head_kv=1,
                       n_layer=26, n_ff=6912, head_dim=256, head_dim_kv=256, norm_eps=1e-6,
                       rope_base_global=1e6, rope_base_local=1e4, sliding_window=512, ffn_act='gelu',
                       emb_scale=float(np.sqrt(1152.0)), attn_softcap=50.0, final_softcap=30.0)


def llama3_8b_config():
    """Llama-3-8B shape: 32 layers, E=4096, 32 q / 8 kv heads of 128, SwiGLU 14336, vocab 128256."""
    return ModelConfig(arch="llama", n_vocab=128256, n_ctx=8192, n_embd=4096, n_head=32, n_head_kv=8,
                       n_layer=32, n_ff=14336, head_dim=128, head_dim_kv=128, norm_eps=1e-5,
                       rope_base_global=500000.0, rope_base_local=500000.0, ffn_act='silu')


def tiny_config(arch="gemma3", n_layer=2, n_embd=128, n_head=4, n_head_kv=1, head_dim=64, n_ff=256,
                n_vocab=512):
    """Small model of either family for CPU-sized parity tests."""
    if arch == "gemma3":
        return ModelConfig(arch="gemma3", n_vocab=n_vocab, n_ctx=4096, n_embd=n_embd, n_head=n_head,
                           n_head_kv=n_head_kv, n_layer=n_layer, n_ff=n_ff, head_dim=head_dim,
                           head_dim_kv=head_dim, norm_eps=1e-6, rope_base_global=1e6, rope_base_local=1e4,
                           ffn_act='gelu', emb_scale=float(np.sqrt(float(n_embd))), attn_softcap=50.0,
                           final_softcap=30.0)
    return ModelConfig(arch="llama", n_vocab=n_vocab, n_ctx=4096, n_embd=n_embd, n_head=n_head,
                       n_head_kv=n_head_kv, n_layer=n_layer, n_ff=n_ff, head_dim=head_dim,
                       head_dim_kv=head_dim, norm_eps=1e-5, rope_base_global=500000.0,
                       rope_base_local=500000.0, ffn_act='silu')


class SyntheticEmbedding:
    """Untied token embedding (the reference looks untied embeddings up on the host, engine.py:2986-2992: a row
    copy out of a float32 table).  A [V, E] float32 table of a large vocabulary would take gigabytes of host
    memory for numbers that carry no information, so the rows come from a pool of at most POOL generated rows,
    made on first use: a lookup is a copy, as in a real model, and tokens POOL apart (after a fixed scramble)
    share a row."""

    POOL = 4096

    def __init__(self, n_vocab, n_embd, seed, sigma):
        self.shape = (n_vocab, n_embd)
        self.seed, self.sigma = seed, sigma
        self._pool = None

    def _rows_of(self, toks):
        if self._pool is None:
            rng = np.random.default_rng([self.seed, 0x0E3B])
            n = min(self.shape[0], self.POOL)
            self._pool = rng.standard_normal((n, self.shape[1]), dtype=np.float32) * np.float32(self.sigma)
        n = self._pool.shape[0]
        return self._pool[toks if self.shape[0] <= n else (toks * 40503 + 11) % n]

    def row(self, tok):
        return self._rows_of(int(tok))

    def rows(self, lo, hi):
        """Rows lo .. hi-1 as one [hi - lo, E] array (what a device-side table is filled from)."""
        return self._rows_of(np.arange(lo, hi, dtype=np.int64))


def _gen(name, shape, seed, sigma, quant, rows_per_chunk=8192):
    rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
    n, k = shape
    if n <= rows_per_chunk:
        return quant(rng.standard_normal((n, k), dtype=np.float32) * np.float32(sigma))
    parts = []
    for r in range(0, n, rows_per_chunk):
        m = min(rows_per_chunk, n - r)
        parts.append(quant(rng.standard_normal((m, k), dtype=np.float32) * np.float32(sigma)))
    out = parts[0]
    out.shape = (n, k)
    out.d = np.concatenate([p.d for p in parts])
    out.codes = np.concatenate([p.codes for p in parts])
    return out


def make_model(cfg, seed=0, sigma=0.02, workers=None):
    """dict name -> QTensor (matrices) / float32 array (norms) / SyntheticEmbedding (untied embd).

    Every tensor has its own generator seeded by (seed, crc32(name)), so the result does not
    depend on `workers` (threads used to draw and quantise tensors in parallel)."""
    import os
    from concurrent.futures import ThreadPoolExecutor
    c = cfg
    q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
    t, jobs = {}, []
    gemma = c.arch.startswith("gemma")
    for L in range(c.n_layer):
        p = f"blk.{L}"
        mats = {"attn_q": (q_dim, c.n_embd), "attn_k": (k_dim, c.n_embd), "attn_v": (k_dim, c.n_embd),
                "attn_output": (c.n_embd, c.n_head * c.head_dim_kv), "ffn_gate": (c.n_ff, c.n_embd),
                "ffn_up": (c.n_ff, c.n_embd), "ffn_down": (c.n_embd, c.n_ff)}
        for nm, sh in mats.items():
            jobs.append((f"{p}.{nm}.weight", sh, quantize_q4_0))
        t[f"{p}.attn_norm.weight"] = np.ones(c.n_embd, np.float32)
        t[f"{p}.ffn_norm.weight"] = np.ones(c.n_embd, np.float32)
        if gemma:
            t[f"{p}.attn_q_norm.weight"] = np.ones(c.head_dim, np.float32)
            t[f"{p}.attn_k_norm.weight"] = np.ones(c.head_dim_kv, np.float32)
            t[f"{p}.post_attention_norm.weight"] = np.ones(c.n_embd, np.float32)
            t[f"{p}.post_ffw_norm.weight"] = np.ones(c.n_embd, np.float32)
    t["output_norm.weight"] = np.ones(c.n_embd, np.float32)
    if gemma:   # tied: the embedding matrix is also the LM head (Q4_0)
        jobs.append(("token_embd.weight", (c.n_vocab, c.n_embd), quantize_q4_0))
    else:       # untied: Q8_0 output head, host-side embedding rows
        jobs.append(("output.weight", (c.n_vocab, c.n_embd), quantize_q8_0))
        t["token_embd.weight"] = SyntheticEmbedding(c.n_vocab, c.n_embd, seed, sigma)
    workers = workers or min(16, os.cpu_count() or 1)
    jobs.sort(key=lambda j: -j[1][0] * j[1][1])
    with ThreadPoolExecutor(max_workers=workers) as ex:
        for (name, _, _), qt in zip(jobs, ex.map(lambda j: _gen(j[0], j[1], seed, sigma, j[2]), jobs)):
            t[name] = qt
    return t
