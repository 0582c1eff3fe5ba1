"""NumPy float32 decode forward pass (oracle; test infrastructure, never shipped).

Restates the reference's own CPU statement of one decode step,
`check_cpu_generation.forward_cpu` (tests/diagnostics/diag_inference.py:973-1037, helpers
:934-956) and `_cpu_attention_step` (adam/models/engine.py:2419-2445): RMSNorm, per-head
QK-norm (Gemma), half-split RoPE on every architecture, GQA with kv head = h // (Hq/Hkv),
full-prefix causal attention with optional tanh soft-cap, GeGLU(tanh-GELU)/SwiGLU FFN,
post-norms when present, tied or untied LM head, optional final soft-cap.

Differences from the reference text, on purpose: (1) weights come dequantised from the same
Q4_0/Q8_0 blocks the device holds; (2) `kv_fp16=True` rounds K and V to fp16 when they enter
the cache, matching the device KV format; (3) the fused Gemma QK-norm uses eps = 1e-6 like the
device op (shaders/src/f32/map_qk_norm_rope_x.comp:64) instead of `norm_eps`.
It is independent of `adamah_np.NumpyAdamah`: it never goes through the op surface, which is
what makes "harness on the op surface == this function" a meaningful wiring check.
"""
import numpy as np

f32 = np.float32


class CpuModel:
    def __init__(self, cfg, tensors, kv_cap, kv_fp16=False, acc64=True):
        """tensors: name -> float32 ndarray ([N,K] matrices, 1-D norms); the untied embedding may be
        an object with .row(tok).  acc64=False keeps every matrix product (attention included) in float32
        BLAS, which is how the reference's forward_cpu runs (used when this model is timed as the CPU baseline)."""
        self.c = cfg
        self.acc64 = acc64
        self.t = tensors
        self.kv_fp16 = kv_fp16
        c = cfg
        self.k_cache = np.zeros((c.n_layer, c.n_head_kv, kv_cap, c.head_dim_kv), np.float32)
        self.v_cache = np.zeros((c.n_layer, c.n_head_kv, kv_cap, c.head_dim_kv), np.float32)

    @staticmethod
    def rms(x, w, eps):
        rms = np.sqrt(np.mean(x.astype(np.float64) ** 2) + eps)
        return ((x / f32(rms)) * w).astype(np.float32)

    @staticmethod
    def gelu(x):
        return f32(0.5) * x * (f32(1.0) + np.tanh(f32(0.797884583) * (x + f32(0.0447149985) * x * x * x)))

    @staticmethod
    def silu(x):
        return x / (f32(1.0) + np.exp(-x))

    @staticmethod
    def rope_half(x, pos, base):
        n, d = x.shape
        half = d // 2
        e = (2 * np.arange(half)).astype(np.float32) / f32(d)
        p = np.power(np.float64(f32(base)), e.astype(np.float64)).astype(np.float32)
        theta = (f32(pos) * (f32(1.0) / p)).astype(np.float32)
        ct = np.cos(theta.astype(np.float64)).astype(np.float32)
        st = np.sin(theta.astype(np.float64)).astype(np.float32)
        x0, x1 = x[:, :half], x[:, half:]
        return np.concatenate([x0 * ct - x1 * st, x0 * st + x1 * ct], axis=1).astype(np.float32)

    def mv(self, name, x):
        if not self.acc64:
            return self.t[name] @ x
        return (self.t[name].astype(np.float64) @ x.astype(np.float64)).astype(np.float32)

    def embed(self, tok):
        e = self.t['token_embd.weight']
        row = e.row(tok) if hasattr(e, 'row') else e[tok]
        h = np.array(row, dtype=np.float32)
        if self.c.emb_scale != 1.0:
            h = h * f32(self.c.emb_scale)
        return h

    def forward(self, tok, pos):
        c, t = self.c, self.t
        gs = max(1, c.n_head // c.n_head_kv)
        seq = pos + 1
        hidden = self.embed(tok)
        for L in range(c.n_layer):
            p = f'blk.{L}'
            freq = c.rope_base_global if c.is_global(L) else c.rope_base_local
            normed = self.rms(hidden, t[f'{p}.attn_norm.weight'], c.norm_eps)
            q = self.mv(f'{p}.attn_q.weight', normed).reshape(c.n_head, c.head_dim)
            k = self.mv(f'{p}.attn_k.weight', normed).reshape(c.n_head_kv, c.head_dim_kv)
            v = self.mv(f'{p}.attn_v.weight', normed).reshape(c.n_head_kv, c.head_dim_kv)
            qnn = f'{p}.attn_q_norm.weight'
            if qnn in t:
                qw, kw = t[qnn], t[f'{p}.attn_k_norm.weight']
                q = np.stack([self.rms(q[i], qw, 1e-6) for i in range(c.n_head)])
                k = np.stack([self.rms(k[i], kw, 1e-6) for i in range(c.n_head_kv)])
            q = self.rope_half(q, pos, freq)
            k = self.rope_half(k, pos, freq)
            if self.kv_fp16:
                k = k.astype(np.float16).astype(np.float32)
                v = v.astype(np.float16).astype(np.float32)
            self.k_cache[L, :, pos, :] = k
            self.v_cache[L, :, pos, :] = v
            scale = f32(1.0 / np.sqrt(c.head_dim))
            attn = np.zeros((c.n_head, c.head_dim_kv), np.float32)
            for h in range(c.n_head):
                Kh = self.k_cache[L, h // gs, :seq]
                Vh = self.v_cache[L, h // gs, :seq]
                if self.acc64:
                    sc = ((Kh.astype(np.float64) @ q[h].astype(np.float64)).astype(np.float32) * scale).astype(np.float32)
                else:                                   # the timed baseline: float32 BLAS here too, no conversions
                    sc = ((Kh @ q[h]) * scale).astype(np.float32)
                if c.attn_softcap > 0:
                    cap = f32(c.attn_softcap)
                    sc = (np.tanh(sc / cap) * cap).astype(np.float32)
                if self.acc64:
                    w_ = np.exp((sc - sc.max()).astype(np.float64))
                    w_ /= w_.sum()
                    attn[h] = (w_ @ Vh.astype(np.float64)).astype(np.float32)
                else:
                    w_ = np.exp(sc - sc.max())
                    attn[h] = (w_ @ Vh) / w_.sum()
            o = self.mv(f'{p}.attn_output.weight', attn.reshape(-1))
            pan = f'{p}.post_attention_norm.weight'
            if pan in t:
                o = self.rms(o, t[pan], c.norm_eps)
            hidden = (hidden + o).astype(np.float32)
            n2 = self.rms(hidden, t[f'{p}.ffn_norm.weight'], c.norm_eps)
            gate = self.mv(f'{p}.ffn_gate.weight', n2)
            up = self.mv(f'{p}.ffn_up.weight', n2)
            with np.errstate(over='ignore'):
                act = (self.gelu(gate) if c.ffn_act == 'gelu' else self.silu(gate)).astype(np.float32) * up
            ffn = self.mv(f'{p}.ffn_down.weight', act.astype(np.float32))
            pfn = f'{p}.post_ffw_norm.weight'
            if pfn in t:
                ffn = self.rms(ffn, t[pfn], c.norm_eps)
            hidden = (hidden + ffn).astype(np.float32)
        self.last_hidden = hidden
        nf = self.rms(hidden, t['output_norm.weight'], c.norm_eps)
        lm = 'output.weight' if 'output.weight' in t else 'token_embd.weight'
        logits = self.mv(lm, nf)
        self.last_raw_logits = logits          # before the final soft-cap: what the LM-head product alone gives
        if c.final_softcap > 0:
            cap = f32(c.final_softcap)
            logits = (np.tanh(logits / cap) * cap).astype(np.float32)
        return logits

    def generate(self, prompt, n_tokens, forced=None):
        """Greedy; np.argmax takes the first maximum = lowest index, the device tie rule."""
        logits = None
        for i, tk in enumerate(prompt):
            logits = self.forward(int(tk), i)
        out, margins = [], []
        pos = len(prompt)
        for step in range(n_tokens):
            nt = int(np.argmax(logits))
            top2 = np.partition(logits, -2)[-2:]
            margins.append(float(top2[1] - top2[0]))
            out.append(nt)
            feed = nt if forced is None else int(forced[step])
            logits = self.forward(feed, pos)
            pos += 1
        return out, margins
