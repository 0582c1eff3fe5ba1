"""Decode harness: issues the reference model engine's op sequence through the ADAMAH op surface.

This is the caller side of the drop-in boundary.  It reproduces, for block-quantised
(Q4_0 / Q8_0) models, what `ADAMEngine` does in the reference (adam/models/engine.py):

* `_build_layout`      :518-609   tensors sorted with Q,K,V adjacent, packed back to back into the
                                   Q4 map (and the Q8 map for Q8_0 tensors), norms into the workspace
* `_alloc_workspace`   :1213-1576 slot order, score rows at element 0, per-head-contiguous KV cache
                                   `[K|V][Hkv][kv_cap][d]` at the end of map 0, all loc handles
* `_upload_all`        :929-1211  qparams + packed nibble upload (Q4), uint8+128 upload (Q8)
* `_upload_locs`       :1601-1725 one base handle per weight, merged QKV / gate-up detection
* `_forward`           :2971-3706 the per-token op order (default, non-Broadcom path)
* `generate`           :3810-3944 token-by-token prefill, greedy decode loop, `decode_tps`

It talks only to an object with the binding's methods, so the same harness runs on the HIP
library and on any other implementation of the surface.  Two extensions beyond the
reference, both optional: weights may be spread over several Q4 maps when they exceed the
32-bit element range of one map, and the KV region may be declared fp16 (`kv_fp16`).
"""
import time
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .quant import QTensor


@dataclass
class GenerationConfig:
    """Field names of the reference's GenerationConfig (adam/models/engine.py:24-29).  The defaults here are
    greedy decoding with no stop token (what the parity tests and the benchmark want); `reference_defaults()`
    gives the reference's own (temperature 0.8, top-k 40, top-p 0.95, repeat penalty 1.1, stop token 1)."""
    max_tokens: int = 128
    temperature: float = 0.0
    top_k: int = 1
    top_p: float = 1.0
    repeat_penalty: float = 1.0
    seed: Optional[int] = None
    repeat_on_prompt: bool = False
    eos_token_ids: tuple = ()

    @classmethod
    def reference_defaults(cls, **kw):
        return cls(**{**dict(temperature=0.8, top_k=40, top_p=0.95, repeat_penalty=1.1, eos_token_ids=(1,)), **kw})


@dataclass
class ModelConfig:
    arch: str = "llama"
    n_vocab: int = 32000
    n_ctx: int = 4096
    n_embd: int = 4096
    n_head: int = 32
    n_head_kv: int = 32
    n_layer: int = 32
    n_ff: int = 11008
    head_dim: int = 128
    head_dim_kv: int = 128
    norm_eps: float = 1e-6
    rope_base_global: float = 10000.0
    rope_base_local: float = 10000.0
    sliding_window: int = 0
    ffn_act: str = 'silu'
    emb_scale: float = 1.0
    attn_softcap: float = 0.0
    final_softcap: float = 0.0

    def is_global(self, L):
        # reference engine.py:52-54
        if self.arch == "gemma3":
            return (L + 1) % 6 == 0
        return True


class DecodeEngine:
    WS_MAP = 0
    Q8_MAP = 2
    EMB_MAP = 15          # float32 copy of an untied embedding table, made when the greedy loops run ahead
    Q4_GROUP = 32
    SAMPLE_TOPK_MAX = 64       # reference engine.py:118
    SAMPLE_REPEAT_MAX = 64     # reference engine.py:120
    SAMPLE_APPROX_SHORTLIST_MAX = 256

    def __init__(self, gpu, cfg, tensors, A=None, kv_cap=1024, kv_fp16=False,
                 fusion_scheduler_mode='legacy', gpu_fused_rows_per_group=256,
                 q4_map_elem_limit=(1 << 32) - 64, verbose=False, decode_plan=True, plan_id=0,
                 prefill_chunk=0, batch=1, lookahead=True, gpu_fused_topk=True, gpu_approx_rerank=False,
                 gpu_approx_partial_k=None, sampling_mode=None):
        """`gpu_fused_topk`, `gpu_approx_rerank`, `gpu_approx_partial_k`: the reference engine's switches of the
        same names (engine.py:333-338), which decide among the LM-head / sampling modes (`_select_sampling_mode`).
        `sampling_mode` names one of them outright ('gpu_matvec_argmax', 'gpu_fused_topk', 'gpu_argmax',
        'gpu_approx_rerank', 'gpu_topk', 'cpu'); a mode the configuration cannot serve raises at generate()."""
        if A is None:
            from . import adamah as A
        self.gpu, self.cfg, self.A = gpu, cfg, A
        self.tensors = tensors = dict(tensors)
        self._gpu_fused_topk = bool(gpu_fused_topk)
        self._gpu_approx_rerank = bool(gpu_approx_rerank)
        self._gpu_approx_partial_k = max(1, min(self.SAMPLE_TOPK_MAX, int(gpu_approx_partial_k or self.SAMPLE_TOPK_MAX)))
        self._force_mode = sampling_mode
        self._lm_q4_approx_name = None
        head = tensors.get('output.weight')
        if self._gpu_approx_rerank and isinstance(head, QTensor) and head.kind == 'q8_0':
            # a 4-bit copy of the 8-bit LM head for the shortlist pass, made as the reference makes it: the
            # dequantised matrix through the 4-bit map's own quantiser with min / max qparams (engine.py:578-583,
            # :1077-1085, :1100-1110)
            from .quant import requantize_q4
            self._lm_q4_approx_name = 'output.weight.q4_approx'
            tensors[self._lm_q4_approx_name] = requantize_q4(head.dequant())
        self.verbose = verbose
        self._kv_cap = int(kv_cap)
        self._kv_fp16 = bool(kv_fp16)
        self._rows_per_group = max(1, int(gpu_fused_rows_per_group))
        self._q4_limit = int(q4_map_elem_limit)
        self._batch = max(1, int(batch))
        self._chunk = max(0, int(prefill_chunk))
        if self._batch > 1:                       # the rows of a batched decode step use the chunk slots
            self._chunk = max(self._chunk, self._batch)
        self._build_layout()
        self._alloc_workspace()
        self._upload_all()
        self._alloc_kv_cache()
        self._upload_locs()
        self._sched = str(fusion_scheduler_mode).strip().lower()
        gpu.fusion_set_scheduler_mode(self._sched)
        gpu.fusion_enable(True)
        self._sample_token_ready = False
        self.n_ops_last_forward = 0
        # One step of lookahead in the greedy loops (embedding rows gathered on the device from the token the
        # previous step left there, tokens handed to the host through the library's ring): set up on first use.
        self._lookahead = bool(lookahead) and getattr(gpu, '_has_token_feed', False)
        self._feed = None
        self.feed_table_bytes = 0          # device bytes of the float32 embedding table of an untied model's token feed
        self.feed_table_upload_s = 0.0
        self._feed_ticket = 0
        # The per-token op list is the same every step except for pos / seq_len, so it is registered
        # once as a native decode plan (reference API adamah.c:10341-10398) and replayed with one call.
        self._plan_id = None
        if decode_plan and getattr(gpu, '_has_decode_plan', False):
            ops = self._plan_ops()
            if len(ops) <= 4096:
                gpu.register_decode_plan(plan_id, ops)
                self._plan_id = plan_id
        # A lockstep step of the full batch is also the same op list every step: a second plan (one native
        # call per step instead of ~47 Python calls per layer, which would otherwise bound the step).
        self._ls_plan_id = None
        if decode_plan and self._batch > 1 and getattr(gpu, '_has_decode_plan', False):
            ops = self._lockstep_plan_ops(self._batch)
            if len(ops) <= 4096:
                gpu.register_decode_plan(plan_id + 1, ops)
                self._ls_plan_id = plan_id + 1

    # ------------------------------------------------------------------ layout
    @staticmethod
    def _qkv_sort_key(n):
        for a, b in (('.attn_q.', '.attn_z0.'), ('.attn_k.', '.attn_z1.'), ('.attn_v.', '.attn_z2.')):
            if a in n:
                return n.replace(a, b)
        return n

    def _build_layout(self):
        t = self.tensors
        self._tied = 'output.weight' not in t
        self._off, self._map_of, self._kind = {}, {}, {}
        self._norm_names = []
        q4_maps = [1] + [i for i in range(3, 16)]
        mi, q4_pos, q8_pos = 0, 0, 0
        self._q4_sizes = {}
        for name in sorted(t.keys(), key=self._qkv_sort_key):
            v = t[name]
            if isinstance(v, QTensor):
                if v.kind == 'q8_0':
                    self._off[name], self._map_of[name], self._kind[name] = q8_pos, self.Q8_MAP, 'q8'
                    q8_pos += v.size
                else:
                    if q4_pos and q4_pos + v.size > self._q4_limit:
                        self._q4_sizes[q4_maps[mi]] = q4_pos
                        mi += 1; q4_pos = 0
                    self._off[name], self._map_of[name], self._kind[name] = q4_pos, q4_maps[mi], 'q4'
                    q4_pos += v.size
            elif isinstance(v, np.ndarray) and v.ndim == 1:
                self._norm_names.append(name)
        if q4_pos:
            self._q4_sizes[q4_maps[mi]] = q4_pos
        self._q8_total = q8_pos
        self._lm_name = 'token_embd.weight' if self._tied else 'output.weight'

    # ------------------------------------------------------------------ workspace
    def _up(self, arr):
        h, _ = self.gpu.upload_dev(np.ascontiguousarray(arr, dtype=np.uint32))
        if h == 0:
            raise RuntimeError("upload_dev failed")
        return h

    def _alloc_workspace(self):
        c, g = self.cfg, self.gpu
        kv_cap = self._kv_cap
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        gs = c.n_head // c.n_head_kv
        self._ws = {}
        self._fused_groups = (c.n_vocab + self._rows_per_group - 1) // self._rows_per_group

        def span(name, sz, pos):
            h = self._up(np.arange(pos, pos + sz))
            self._ws[name] = (h, sz, pos)
            g.register_loc_span(h, 0, pos, sz)

        pos = 0
        sc_sz = c.n_head * kv_cap
        span('scores', sc_sz, 0)
        self._scores_row_h = self._up(np.arange(0, sc_sz, kv_cap))
        g.register_row_base_span(self._scores_row_h, 0, 0, c.n_head, kv_cap, kv_cap)
        pos += sc_sz
        self._pos_scale = pos; pos += 1
        if c.emb_scale != 1.0:
            h = self._up(np.full(c.n_embd, pos))
            self._ws['emb_scale'] = (h, c.n_embd, pos)
            g.register_loc_span(h, 0, pos, 1)
            self._pos_emb_scale = pos; pos += 1
        if c.attn_softcap > 0:
            self._pos_attn_cap = pos; pos += 1
        if c.final_softcap > 0:
            self._pos_final_cap = pos
            # one entry per logit: the broadcast ops take a location per element (reference engine.py:1282-1287)
            self._final_cap_h = self._up(np.full(c.n_vocab, pos))
            g.register_loc_span(self._final_cap_h, 0, pos, 1)
            pos += 1

        slots = [('hidden', c.n_embd), ('normed', c.n_embd), ('q', q_dim), ('k', k_dim), ('v', k_dim),
                 ('attn_out', c.n_head * c.head_dim_kv), ('o_proj', c.n_embd), ('gate', c.n_ff),
                 ('up', c.n_ff), ('act', c.n_ff), ('ffn_out', c.n_embd), ('logits', c.n_vocab),
                 ('sample_token', 1), ('sample_rand', 1),
                 ('sample_fused_idx', self._fused_groups * self.SAMPLE_TOPK_MAX),
                 ('sample_fused_val', self._fused_groups * self.SAMPLE_TOPK_MAX),
                 ('sample_topk_idx', self.SAMPLE_TOPK_MAX), ('sample_topk_val', self.SAMPLE_TOPK_MAX),
                 ('sample_topk_prob', self.SAMPLE_TOPK_MAX), ('sample_short_sel', self.SAMPLE_APPROX_SHORTLIST_MAX),
                 ('sample_exact_idx', self.SAMPLE_APPROX_SHORTLIST_MAX),
                 ('sample_exact_val', self.SAMPLE_APPROX_SHORTLIST_MAX),
                 ('normed2', c.n_embd)]
        for name, sz in slots:
            span(name, sz, pos); pos += sz

        for name in self._norm_names:
            self._off[name] = pos; self._map_of[name] = 0
            pos += self.tensors[name].size

        if self._chunk:
            pos = self._alloc_chunk_slots(pos)

        pos_q, pos_k, pos_v = self._ws['q'][2], self._ws['k'][2], self._ws['v'][2]
        self._q_rows_h = self._up(pos_q + np.arange(c.n_head) * c.head_dim)
        g.register_row_base_span(self._q_rows_h, 0, pos_q, c.n_head, c.head_dim, c.head_dim)
        self._k_rows_h = self._up(pos_k + np.arange(c.n_head_kv) * c.head_dim_kv)
        g.register_row_base_span(self._k_rows_h, 0, pos_k, c.n_head_kv, c.head_dim_kv, c.head_dim_kv)
        # separate source handles for RoPE (same positions as the q / k slots)
        self._q_rope_src_h = self._up(np.arange(pos_q, pos_q + q_dim))
        self._k_rope_src_h = self._up(np.arange(pos_k, pos_k + k_dim))
        g.register_loc_span(self._q_rope_src_h, 0, pos_q, q_dim)
        g.register_loc_span(self._k_rope_src_h, 0, pos_k, k_dim)
        self._qk_out_h = None
        if c.head_dim == c.head_dim_kv:
            self._qk_out_h = self._up(np.arange(pos_q, pos_q + q_dim + k_dim))
            g.register_loc_span(self._qk_out_h, 0, pos_q, q_dim + k_dim)
        self._qkv_out_h = self._up(np.arange(pos_q, pos_q + q_dim + 2 * k_dim))
        g.register_loc_span(self._qkv_out_h, 0, pos_q, q_dim + 2 * k_dim)
        pos_gate = self._ws['gate'][2]
        self._gateup_out_h = self._up(np.arange(pos_gate, pos_gate + 2 * c.n_ff))
        g.register_loc_span(self._gateup_out_h, 0, pos_gate, 2 * c.n_ff)
        self._k_src_base_h = self._up([pos_k])
        g.register_loc_span(self._k_src_base_h, 0, pos_k, 1)

        # KV cache: layer L -> K heads [Hkv, kv_cap, d] then V heads, start aligned to d
        kv_step = kv_cap * c.head_dim_kv
        kv_per_layer = 2 * c.n_head_kv * kv_step
        if pos % c.head_dim_kv:
            pos += c.head_dim_kv - pos % c.head_dim_kv
        self._kv_start, self._kv_step, self._kv_per_layer = pos, kv_step, kv_per_layer
        self._kv_per_seq = c.n_layer * kv_per_layer
        # one cache per sequence of the batch (sequence 0 is the one single-sequence decoding uses)
        self._k_base_s = [[pos + sq * self._kv_per_seq + L * kv_per_layer for L in range(c.n_layer)] for sq in range(self._batch)]
        self._v_base_s = [[kb + c.n_head_kv * kv_step for kb in row] for row in self._k_base_s]
        self._k_base, self._v_base = self._k_base_s[0], self._v_base_s[0]
        pos += self._batch * self._kv_per_seq
        self._k_locs_hs, self._v_locs_hs, self._kv_copy_h = [], [], []
        heads = np.arange(c.n_head) // gs
        for sq in range(self._batch):
            hks, hvs = [], []
            for L in range(c.n_layer):
                kb, vb = self._k_base_s[sq][L], self._v_base_s[sq][L]
                hk = self._up(kb + heads * kv_step); hv = self._up(vb + heads * kv_step)
                g.register_row_base_span(hk, 0, kb, c.n_head_kv, kv_step, kv_step)
                g.register_row_base_span(hv, 0, vb, c.n_head_kv, kv_step, kv_step)
                hks.append(hk); hvs.append(hv)
                if sq == 0:
                    spec = np.empty(4 * c.n_head_kv, np.uint32)
                    for gi in range(c.n_head_kv):
                        spec[4 * gi:4 * gi + 4] = (gi, kb // c.head_dim_kv + gi * kv_cap,
                                                   gi + c.n_head_kv, vb // c.head_dim_kv + gi * kv_cap)
                    self._kv_copy_h.append(self._up(spec))
                if self._chunk:
                    self._chunk_kv_spec(sq, L, kb, vb)
            self._k_locs_hs.append(hks); self._v_locs_hs.append(hvs)
        self._k_locs_h, self._v_locs_h = self._k_locs_hs[0], self._v_locs_hs[0]
        if self._batch > 1:
            self._batch_kv_spec()
        pos_ao = self._ws['attn_out'][2]
        self._ao_rows_h = self._up(pos_ao + np.arange(c.n_head) * c.head_dim_kv)
        g.register_row_base_span(self._ao_rows_h, 0, pos_ao, c.n_head, c.head_dim_kv, c.head_dim_kv)

        self._hid_locs = np.arange(self._ws['hidden'][2], self._ws['hidden'][2] + c.n_embd, dtype=np.uint32)
        self._sample_locs = np.array([self._ws['sample_token'][2]], dtype=np.uint32)
        self._rand_locs = np.array([self._ws['sample_rand'][2]], dtype=np.uint32)
        self._sample_fused_base_h = self._up([self._ws['sample_fused_idx'][2]])
        self._sample_exact_base_h = self._up([self._ws['sample_exact_idx'][2]])
        span_of = lambda n: np.arange(self._ws[n][2], self._ws[n][2] + self._ws[n][1], dtype=np.uint32)
        self._logit_locs = span_of('logits')
        self._fused_val_locs = span_of('sample_fused_val')
        self._short_sel_locs, self._exact_idx_locs, self._exact_val_locs = (
            span_of('sample_short_sel'), span_of('sample_exact_idx'), span_of('sample_exact_val'))
        self._short_sel_chunk_h, self._exact_idx_chunk_h, self._exact_val_chunk_h = [], [], []
        for lo in range(0, self.SAMPLE_APPROX_SHORTLIST_MAX, self.SAMPLE_TOPK_MAX):      # rerank runs in chunks of 64
            hi = lo + self.SAMPLE_TOPK_MAX
            self._short_sel_chunk_h.append(self._up(self._short_sel_locs[lo:hi]))
            self._exact_idx_chunk_h.append(self._up(self._exact_idx_locs[lo:hi]))
            self._exact_val_chunk_h.append(self._up(self._exact_val_locs[lo:hi]))
        self._sample_rerank_n = 0
        self._sample_fused_partial_n = 0
        self._sample_repeat_ids = np.zeros(self.SAMPLE_REPEAT_MAX, np.uint32)
        self._sample_repeat_ids_h = self._up(self._sample_repeat_ids)
        self._ws_total = pos

    # ------------------------------------------------------------------ chunked prefill: workspace
    def _alloc_chunk_slots(self, pos):
        """Row-major [M, width] slots for a prefill chunk of M tokens and the handles its ops take: one
        element offset per matrix operand, one row base per token for the row-wise ops, contiguous
        spans for the element-wise ones, per-token head-row lists for attention."""
        c, g, M = self.cfg, self.gpu, self._chunk
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        d = c.head_dim_kv
        pos += (-pos) % max(c.head_dim, d)                    # K / V rows are addressed in units of the head size
        gemma = c.head_dim == c.head_dim_kv and any('attn_q_norm' in n for n in self._norm_names)
        widths = [('hidden', c.n_embd), ('normed', c.n_embd), ('q', q_dim), ('k', k_dim), ('v', k_dim),
                  ('attn_out', c.n_head * c.head_dim_kv), ('o_proj', c.n_embd),
                  ('gate', c.n_ff), ('up', c.n_ff), ('act', c.n_ff), ('ffn_out', c.n_embd), ('normed2', c.n_embd)]
        if gemma:                                             # rotated [q heads | k heads] of every token
            widths.append(('qk', q_dim + k_dim))
        self._cp, self._cw = {}, dict(widths)
        for name, w in widths:
            if name in ('k', 'v', 'qk'):
                pos += (-pos) % d
            self._cp[name] = pos
            pos += M * w
        t = np.arange(M)
        self._c1 = {n: self._up([p]) for n, p in self._cp.items()}                        # matrix operands
        self._crow = {n: self._up(self._cp[n] + t * self._cw[n]) for n in ('hidden', 'normed', 'normed2', 'o_proj', 'ffn_out', 'q', 'k')}
        self._cspan = {n: self._up(np.arange(self._cp[n], self._cp[n] + M * self._cw[n]))
                       for n in ('hidden', 'o_proj', 'ffn_out', 'gate', 'up', 'act')}
        self._chunk_qk = gemma
        qsrc, qw = ('qk', q_dim + k_dim) if gemma else ('q', q_dim)
        heads = np.arange(c.n_head)
        self._c_qrows = [self._up(self._cp[qsrc] + i * qw + heads * c.head_dim) for i in range(M)]
        self._c_aorows = [self._up(self._cp['attn_out'] + i * c.n_head * c.head_dim_kv + heads * c.head_dim_kv) for i in range(M)]
        if gemma:
            kh = np.arange(c.n_head_kv)
            self._c_lq = [self._up(self._cp['q'] + i * q_dim + heads * c.head_dim) for i in range(M)]
            self._c_lk = [self._up(self._cp['k'] + i * k_dim + kh * d) for i in range(M)]
            self._c_qkdst = [self._up([self._cp['qk'] + i * (q_dim + k_dim)]) for i in range(M)]
        self._c_qbase, self._c_kbase = self._up([self._cp['q']]), self._up([self._cp['k']])   # first row of the chunk
        self._c_n1 = [self._up([self._cp['normed'] + i * c.n_embd]) for i in range(M)]
        self._c_tok_pos = pos
        self._c_tok1 = [self._up([pos + i]) for i in range(M)]                               # sampled token of row i
        self._c_tok_locs = np.arange(pos, pos + M, dtype=np.uint32)
        pos += M
        self._c_last = self._up(np.zeros(c.n_embd, np.uint32))
        self._c_last_m = 0
        self._c_zero = self._up([0])
        self._c_emb_hs = {}
        self._c_wrows = {}
        self._c_kvspec = {}
        if c.emb_scale != 1.0:
            self._c_embscale_h = self._up(np.full(M * c.n_embd, self._pos_emb_scale))
        return pos

    def _chunk_kv_spec(self, sq, L, kb, vb):
        """(source row, cache row) pairs of a whole chunk, token-major, so that a prefix serves a shorter
        chunk; rows are counted in head-size units from element 0 of the workspace."""
        c, M, d = self.cfg, self._chunk, self.cfg.head_dim_kv
        k_dim = c.n_head_kv * d
        if self._chunk_qk:
            ksrc, kstride = self._cp['qk'] + c.n_head * c.head_dim, c.n_head * c.head_dim + k_dim
        else:
            ksrc, kstride = self._cp['k'], k_dim
        spec = np.empty((M, 2 * c.n_head_kv, 2), np.uint32)
        for gi in range(c.n_head_kv):
            t = np.arange(M)
            spec[:, 2 * gi, 0] = (ksrc + t * kstride + gi * d) // d
            spec[:, 2 * gi, 1] = kb // d + gi * self._kv_cap + t
            spec[:, 2 * gi + 1, 0] = (self._cp['v'] + t * k_dim + gi * d) // d
            spec[:, 2 * gi + 1, 1] = vb // d + gi * self._kv_cap + t
        assert ksrc % d == 0 and kstride % d == 0 and self._cp['v'] % d == 0
        self._c_kvspec[(sq, L)] = self._up(spec.reshape(-1))

    def _batch_kv_spec(self):
        """Per layer: (source row, cache row) pairs of one decode step of the whole batch -- row s of the
        chunk slots goes to the cache of sequence s."""
        c, B, d = self.cfg, self._batch, self.cfg.head_dim_kv
        k_dim = c.n_head_kv * d
        if self._chunk_qk:
            ksrc, kstride = self._cp['qk'] + c.n_head * c.head_dim, c.n_head * c.head_dim + k_dim
        else:
            ksrc, kstride = self._cp['k'], k_dim
        self._b_kvspec = []
        for L in range(c.n_layer):
            spec = np.empty((B, 2 * c.n_head_kv, 2), np.uint32)
            for sq in range(B):
                for gi in range(c.n_head_kv):
                    spec[sq, 2 * gi] = ((ksrc + sq * kstride + gi * d) // d, self._k_base_s[sq][L] // d + gi * self._kv_cap)
                    spec[sq, 2 * gi + 1] = ((self._cp['v'] + sq * k_dim + gi * d) // d, self._v_base_s[sq][L] // d + gi * self._kv_cap)
            self._b_kvspec.append(self._up(spec.reshape(-1)))

    def _wrows(self, name):
        """Norm weight handle with one (identical) base per chunk row."""
        h = self._c_wrows.get(name)
        if h is None:
            h = self._c_wrows[name] = self._up(np.full(self._chunk, self._off[name]))
        return h

    # ------------------------------------------------------------------ upload
    def _upload_all(self):
        g, A, t = self.gpu, self.A, self.tensors
        g.set_dtype(A.DTYPE_F32)
        g.map_create(self.WS_MAP, 1, self._ws_total)
        if self._kv_fp16:
            g.kv_cache_fp16(self.WS_MAP, self._kv_start, self._batch * self.cfg.n_layer * self._kv_per_layer)
        chunk = 1 << 25
        for mid, total in self._q4_sizes.items():
            g.map_create_typed(mid, A.DTYPE_Q4, 1, total, self.Q4_GROUP)
            names = [n for n in self._off if self._map_of.get(n) == mid and self._kind.get(n) == 'q4']
            names.sort(key=lambda n: self._off[n])
            ng = (total + self.Q4_GROUP - 1) // self.Q4_GROUP
            sc = np.ones(ng, np.float32); zp = np.zeros(ng, np.float32)
            for n in names:
                s, z = t[n].qparams()
                g0 = self._off[n] // self.Q4_GROUP
                sc[g0:g0 + s.size] = s; zp[g0:g0 + z.size] = z
            g.set_qparams(mid, sc, zp)
            for n in names:
                if t[n].kind == 'q4_req':      # float values: the map's own quantiser makes the codes (reference engine.py:1086-1096)
                    data = t[n].data
                    for b in range(0, data.size, chunk):
                        g.scatter_contiguous(mid, self._off[n] + b, data[b:b + chunk])
                    continue
                codes = t[n].codes
                for b in range(0, codes.size, chunk):
                    part = codes[b:b + chunk]
                    g.scatter_q4_packed_contiguous(mid, self._off[n] + 2 * b, part, n_locs=2 * part.size)
        if self._q8_total:
            g.map_create_typed(self.Q8_MAP, A.DTYPE_Q8, 1, self._q8_total, self.Q4_GROUP)
            ng = (self._q8_total + self.Q4_GROUP - 1) // self.Q4_GROUP
            sc = np.ones(ng, np.float32); zp = np.zeros(ng, np.float32)
            for n, kind in self._kind.items():
                if kind != 'q8':
                    continue
                s, z = t[n].qparams()
                g0 = self._off[n] // self.Q4_GROUP
                sc[g0:g0 + s.size] = s; zp[g0:g0 + z.size] = z
                codes = t[n].codes
                for b in range(0, codes.size, chunk):
                    g.scatter_contiguous(self.Q8_MAP, self._off[n] + b, codes[b:b + chunk])
            g.set_qparams(self.Q8_MAP, sc, zp)
        for n in self._norm_names:
            off = self._off[n]
            g.scatter(self.WS_MAP, np.arange(off, off + t[n].size, dtype=np.uint32),
                      np.ascontiguousarray(t[n], np.float32))

    def _alloc_kv_cache(self):
        c, g = self.cfg, self.gpu
        self.reset()
        one = lambda p, v: g.scatter(self.WS_MAP, np.array([p], np.uint32), np.array([v], np.float32))
        one(self._pos_scale, 1.0 / np.sqrt(c.head_dim))
        if c.emb_scale != 1.0:
            one(self._pos_emb_scale, c.emb_scale)
        if c.attn_softcap > 0:
            one(self._pos_attn_cap, c.attn_softcap)
        if c.final_softcap > 0:
            one(self._pos_final_cap, c.final_softcap)

    def _upload_locs(self):
        c = self.cfg
        self._wh = {n: self._up([self._off[n]]) for n in self._kind}

        def merged(names):
            if len({self._map_of[n] for n in names}) != 1 or len({self._kind[n] for n in names}) != 1:
                return None
            for a, b in zip(names, names[1:]):
                if self._off[b] != self._off[a] + self.tensors[a].size:
                    return None
            return self._wh[names[0]]

        self._qkv_wt, self._gateup_wt = {}, {}
        for L in range(c.n_layer):
            p = f'blk.{L}'
            h = merged([f'{p}.attn_q.weight', f'{p}.attn_k.weight', f'{p}.attn_v.weight'])
            if h:
                self._qkv_wt[L] = h
            h = merged([f'{p}.ffn_gate.weight', f'{p}.ffn_up.weight'])
            if h:
                self._gateup_wt[L] = h
        for n in self._norm_names:
            off, sz = self._off[n], self.tensors[n].size
            if 'attn_q_norm' in n:
                rows, hd = c.n_head, c.head_dim
                locs = [off] * rows if sz == hd else [off + i * hd for i in range(rows)]
            elif 'attn_k_norm' in n:
                rows, hd = c.n_head_kv, c.head_dim_kv
                locs = [off] * rows if sz == hd else [off + i * hd for i in range(rows)]
            else:
                locs = [off]
            self._wh[n] = self._up(locs)
        # embedding fetch: tied Q4 matrix -> per-token gather locs; untied -> host rows
        self._emb_gather_h = 0
        if self._tied:
            self._emb_base = (np.uint32(self._off[self._lm_name]) + np.arange(c.n_embd, dtype=np.uint32))
            self._emb_locs = np.empty(c.n_embd, np.uint32)
            self._emb_gather_h = self._up(self._emb_base)

    # ------------------------------------------------------------------ op helpers
    def _proj(self, in_h, name, out_h, K, N, wt_h=None):
        g = self.gpu
        fn = g.map_matmul_t_xq8_dev if self._kind[name] == 'q8' else g.map_matmul_t_xq4_dev
        fn(self.WS_MAP, self._map_of[name], in_h, wt_h or self._wh[name], out_h, 1, K, N)

    def _rms(self, src_h, name, dst_h, rows, dim):
        self.gpu.map_rmsnorm_dev(self.WS_MAP, src_h, self._wh[name], dst_h, rows, dim, self.cfg.norm_eps)

    # ------------------------------------------------------------------ decode plan
    def _plan_ops(self):
        """The layer loop of `_forward` (plus the output norm) as DecodePlanOp records; `pos` and
        `seq_len` are the runtime sentinels.  Field use per kind: adamah.c:10265-10338."""
        c, A, ws = self.cfg, self.A, self.WS_MAP
        P, S = A.DECODE_RUNTIME_POS, A.DECODE_RUNTIME_SEQ_LEN
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        W = self._ws
        hid_h, normed_h, q_h, k_h, v_h = (W[n][0] for n in ('hidden', 'normed', 'q', 'k', 'v'))
        ao_h, op_h, n2_h, gate_h, up_h, act_h, ffn_h = (
            W[n][0] for n in ('attn_out', 'o_proj', 'normed2', 'gate', 'up', 'act', 'ffn_out'))
        alias_fast = self._sched != 'legacy'
        Op = A.DecodePlanOp
        ops = []

        def rms(src, name, dst, dim):
            ops.append(Op(kind=A.DECODE_OP_RMSNORM, map_id=ws, h0=src, h1=self._wh[name], h2=dst, u0=1, u1=dim,
                          f0=c.norm_eps))

        def rms_add(src, name, res, dst, dim):
            ops.append(Op(kind=A.DECODE_OP_RMSNORM_ADD, map_id=ws, h0=src, h1=self._wh[name], h2=res, h3=dst, u0=1,
                          u1=dim, f0=c.norm_eps))

        def proj(in_h, name, out_h, K, N, wt_h=None):
            kind = A.DECODE_OP_MATMUL_T_XQ8 if self._kind[name] == 'q8' else A.DECODE_OP_MATMUL_T_XQ4
            ops.append(Op(kind=kind, map_id=ws, map_id2=self._map_of[name], h0=in_h, h1=wt_h or self._wh[name],
                          h2=out_h, u0=1, u1=K, u2=N, u3=1))

        def op2(code, a, b, d, n):
            ops.append(Op(kind=A.DECODE_OP_OP2, map_id=ws, op_code=code, h0=a, h1=b, h2=d, u0=n))

        for L in range(c.n_layer):
            p = f'blk.{L}'
            freq = c.rope_base_global if c.is_global(L) else c.rope_base_local
            rms(hid_h, f'{p}.attn_norm.weight', normed_h, c.n_embd)
            if alias_fast and L in self._qkv_wt:
                proj(normed_h, f'{p}.attn_q.weight', self._qkv_out_h, c.n_embd, q_dim + 2 * k_dim, self._qkv_wt[L])
            else:
                proj(normed_h, f'{p}.attn_q.weight', q_h, c.n_embd, q_dim)
                proj(normed_h, f'{p}.attn_k.weight', k_h, c.n_embd, k_dim)
                proj(normed_h, f'{p}.attn_v.weight', v_h, c.n_embd, k_dim)
            qnn = f'{p}.attn_q_norm.weight'
            if qnn in self._wh:
                ops.append(Op(kind=A.DECODE_OP_QK_NORM_ROPE_X, map_id=ws, map_id2=ws, h0=self._q_rows_h, h1=self._wh[qnn],
                              h2=self._k_rows_h, h3=self._wh[f'{p}.attn_k_norm.weight'], h4=self._qk_out_h,
                              u0=c.n_head, u1=c.head_dim, u2=c.n_head_kv, u3=c.head_dim_kv, u4=P, f0=freq))
            else:
                ops.append(Op(kind=A.DECODE_OP_ROPE, map_id=ws, h0=self._q_rope_src_h, h1=q_h, u0=1, u1=c.n_head,
                              u2=c.head_dim, u3=P, f0=freq))
                ops.append(Op(kind=A.DECODE_OP_ROPE, map_id=ws, h0=self._k_rope_src_h, h1=k_h, u0=1, u1=c.n_head_kv,
                              u2=c.head_dim_kv, u3=P, f0=freq))
            ops.append(Op(kind=A.DECODE_OP_ROW_COPY_OFFSET, map_id=ws, h0=self._kv_copy_h[L], h1=self._k_src_base_h,
                          u0=P, u1=2 * c.n_head_kv, u2=c.head_dim_kv))
            ops.append(Op(kind=A.DECODE_OP_MATMUL_T, map_id=ws, h0=self._q_rows_h, h1=self._k_locs_h[L],
                          h2=self._scores_row_h, u0=1, u1=c.head_dim, u2=S, u3=c.n_head))
            ops.append(Op(kind=A.DECODE_OP_ATTN_SOFTMAX_VALUE, map_id=ws, h0=self._scores_row_h, h1=self._v_locs_h[L],
                          h2=self._ao_rows_h, u0=c.n_head, u1=S, u2=c.head_dim_kv,
                          f0=float(1.0 / np.sqrt(c.head_dim)), f1=float(c.attn_softcap)))
            ops.append(Op(kind=A.DECODE_OP_FUSION_FLUSH))
            proj(ao_h, f'{p}.attn_output.weight', op_h, c.n_head * c.head_dim_kv, c.n_embd)
            pan = f'{p}.post_attention_norm.weight'
            if pan in self._wh:
                rms_add(op_h, pan, hid_h, hid_h, c.n_embd)
            else:
                op2(A.OP_ADD, hid_h, op_h, hid_h, c.n_embd)
            rms(hid_h, f'{p}.ffn_norm.weight', n2_h, c.n_embd)
            if alias_fast and L in self._gateup_wt:
                proj(n2_h, f'{p}.ffn_gate.weight', self._gateup_out_h, c.n_embd, 2 * c.n_ff, self._gateup_wt[L])
            else:
                proj(n2_h, f'{p}.ffn_gate.weight', gate_h, c.n_embd, c.n_ff)
                proj(n2_h, f'{p}.ffn_up.weight', up_h, c.n_embd, c.n_ff)
            op2(A.OP_GEGLU if c.ffn_act == 'gelu' else A.OP_SWIGLU, gate_h, up_h, act_h, c.n_ff)
            proj(act_h, f'{p}.ffn_down.weight', ffn_h, c.n_ff, c.n_embd)
            pfn = f'{p}.post_ffw_norm.weight'
            if pfn in self._wh:
                rms_add(ffn_h, pfn, hid_h, hid_h, c.n_embd)
            else:
                op2(A.OP_ADD, hid_h, ffn_h, hid_h, c.n_embd)
        rms(hid_h, 'output_norm.weight', normed_h, c.n_embd)
        return ops

    # ------------------------------------------------------------------ token feed (lookahead)
    def _token_feed(self):
        """(map, first element) of the [V, E] table the device gathers embedding rows from, plus the handles of the
        token slots.  Tied models read the LM head's quantised rows, as their host-driven gather does; untied
        ones get their float32 table uploaded once into a map of its own (the reference keeps it on the host,
        engine.py:2986-2992, which forces a round trip per token).  None: no room for the table."""
        if self._feed is not None:
            return self._feed or None
        c, g, A = self.cfg, self.gpu, self.A
        if self._tied:
            src = (self._map_of[self._lm_name], self._off[self._lm_name])
        else:
            emb = self.tensors['token_embd.weight']
            if self.EMB_MAP in self._q4_sizes or c.n_vocab * c.n_embd > self._q4_limit:
                self._feed = False
                return None
            t0 = time.perf_counter()
            try:
                g.set_dtype(A.DTYPE_F32)
                g.map_create(self.EMB_MAP, 1, c.n_vocab * c.n_embd)
                step = max(1, (1 << 24) // c.n_embd)
                for lo in range(0, c.n_vocab, step):
                    hi = min(c.n_vocab, lo + step)
                    rows = emb.rows(lo, hi) if hasattr(emb, 'rows') else np.stack([emb.row(t) for t in range(lo, hi)])
                    g.scatter_contiguous(self.EMB_MAP, lo * c.n_embd, np.ascontiguousarray(rows, np.float32).reshape(-1))
            except (RuntimeError, MemoryError):
                # no room for the table (or the upload failed): the loops fall back to the host lookup per token
                self._feed = False
                return None
            self.feed_table_bytes = 4 * c.n_vocab * c.n_embd
            self.feed_table_upload_s = time.perf_counter() - t0
            src = (self.EMB_MAP, 0)
        self._feed = {'src': src, 'tok_h': self._up(self._sample_locs),
                      'tok_hs': {self._batch: self._up(self._c_tok_locs[:self._batch])} if self._batch > 1 else {}}
        return self._feed

    def _wait_tokens(self, ticket, m=1):
        return [int(t) for t in self.gpu.token_wait(ticket, m)]

    # ------------------------------------------------------------------ forward
    def _forward(self, tok, pos, sample=True, sample_cfg=None, sample_prev=(), from_device=False, on_token=None,
                 sample_mode=None, return_logits=False):
        """One decode step; op order of reference engine.py:2971-3402 (default discrete-GPU path).
        `sample_mode`: the LM-head / sampling tail to issue (reference engine.py:3318-3640); None picks
        'gpu_fused_topk' for a sampling configuration and 'gpu_matvec_argmax' otherwise, as before the other
        modes existed.  `return_logits`: the full logits (final soft-cap applied) are computed and returned.
        `from_device`: the input token is the one the previous step's LM head left in the token slot (`tok` is
        not looked at); its embedding row is gathered on the device.  `on_token` (with `from_device`): called with
        that token once it has reached the host -- after the layers have been issued, before the LM head's ops are
        (their repeat-penalty list may depend on it); returning False ends the step there."""
        c, g, A, ws = self.cfg, self.gpu, self.A, self.WS_MAP
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        seq_len = pos + 1
        W = self._ws
        hid_h, normed_h, q_h, k_h, v_h = (W[n][0] for n in ('hidden', 'normed', 'q', 'k', 'v'))
        ao_h, op_h, n2_h, gate_h, up_h, act_h, ffn_h = (
            W[n][0] for n in ('attn_out', 'o_proj', 'normed2', 'gate', 'up', 'act', 'ffn_out'))
        alias_fast = self._sched != 'legacy'

        if from_device:
            feed = self._token_feed()
        elif self._tied:
            np.add(self._emb_base, np.uint32(tok * c.n_embd), out=self._emb_locs)
            g.upload_dev(self._emb_locs, handle=self._emb_gather_h)
        else:
            row = self.tensors['token_embd.weight'].row(tok)
            if c.emb_scale != 1.0:
                row = row * np.float32(c.emb_scale)
            g.scatter(ws, self._hid_locs, row)

        g.batch_begin()
        if from_device:     # (the same launch hands the token to the host: _wait_tokens(self._feed_ticket))
            self._feed_ticket = g.embed_post_tokens_dev(ws, feed['src'][0], feed['tok_h'], feed['src'][1],
                                                        int(self._hid_locs[0]), 1, c.n_embd, c.n_vocab, float(c.emb_scale))
        elif self._tied:
            src_h, _, _, _ = g.map_gather_dev(self._map_of[self._lm_name], self._emb_gather_h, c.n_embd)
            if src_h == 0:        # the binding reports a failed gather as handle 0, like the reference's
                raise RuntimeError("map_gather_dev failed (embedding row)")
            g.map_scatter_dev(ws, hid_h, c.n_embd, src_h)
            if c.emb_scale != 1.0:
                g.map_broadcast_dev(ws, A.OP_MUL, hid_h, W['emb_scale'][0], hid_h, c.n_embd)

        for L in range(c.n_layer if self._plan_id is None else 0):
            p = f'blk.{L}'
            freq = c.rope_base_global if c.is_global(L) else c.rope_base_local
            self._rms(hid_h, f'{p}.attn_norm.weight', normed_h, 1, c.n_embd)
            if alias_fast and L in self._qkv_wt:
                self._proj(normed_h, f'{p}.attn_q.weight', self._qkv_out_h, c.n_embd,
                           q_dim + 2 * k_dim, wt_h=self._qkv_wt[L])
            else:
                self._proj(normed_h, f'{p}.attn_q.weight', q_h, c.n_embd, q_dim)
                self._proj(normed_h, f'{p}.attn_k.weight', k_h, c.n_embd, k_dim)
                self._proj(normed_h, f'{p}.attn_v.weight', v_h, c.n_embd, k_dim)

            qnn = f'{p}.attn_q_norm.weight'
            if qnn in self._wh:
                g.map_qk_norm_rope_x_dev(ws, ws, self._q_rows_h, self._wh[qnn], self._k_rows_h,
                                         self._wh[f'{p}.attn_k_norm.weight'], self._qk_out_h,
                                         c.n_head, c.head_dim, c.n_head_kv, c.head_dim_kv, pos, freq)
            else:
                g.map_rope_dev(ws, self._q_rope_src_h, q_h, 1, c.n_head, c.head_dim, pos, freq)
                g.map_rope_dev(ws, self._k_rope_src_h, k_h, 1, c.n_head_kv, c.head_dim_kv, pos, freq)

            g.map_row_copy_offset_dev(ws, self._kv_copy_h[L], self._k_src_base_h, pos,
                                      2 * c.n_head_kv, c.head_dim_kv)
            g.map_matmul_t_dev(ws, self._q_rows_h, self._k_locs_h[L], self._scores_row_h,
                               1, c.head_dim, seq_len, c.n_head)
            g.map_attn_softmax_value_dev(ws, self._scores_row_h, self._v_locs_h[L], self._ao_rows_h,
                                         c.n_head, seq_len, c.head_dim_kv,
                                         float(1.0 / np.sqrt(c.head_dim)), float(c.attn_softcap))
            g.fusion_flush()
            self._proj(ao_h, f'{p}.attn_output.weight', op_h, c.n_head * c.head_dim_kv, c.n_embd)
            pan = f'{p}.post_attention_norm.weight'
            if pan in self._wh:
                g.map_rmsnorm_add_dev(ws, op_h, self._wh[pan], hid_h, hid_h, 1, c.n_embd, c.norm_eps)
            else:
                g.map_op2_dev(ws, A.OP_ADD, hid_h, op_h, hid_h, c.n_embd)

            self._rms(hid_h, f'{p}.ffn_norm.weight', n2_h, 1, c.n_embd)
            if alias_fast and L in self._gateup_wt:
                self._proj(n2_h, f'{p}.ffn_gate.weight', self._gateup_out_h, c.n_embd, 2 * c.n_ff,
                           wt_h=self._gateup_wt[L])
            else:
                self._proj(n2_h, f'{p}.ffn_gate.weight', gate_h, c.n_embd, c.n_ff)
                self._proj(n2_h, f'{p}.ffn_up.weight', up_h, c.n_embd, c.n_ff)
            g.map_op2_dev(ws, A.OP_GEGLU if c.ffn_act == 'gelu' else A.OP_SWIGLU, gate_h, up_h, act_h, c.n_ff)
            self._proj(act_h, f'{p}.ffn_down.weight', ffn_h, c.n_ff, c.n_embd)
            pfn = f'{p}.post_ffw_norm.weight'
            if pfn in self._wh:
                g.map_rmsnorm_add_dev(ws, ffn_h, self._wh[pfn], hid_h, hid_h, 1, c.n_embd, c.norm_eps)
            else:
                g.map_op2_dev(ws, A.OP_ADD, hid_h, ffn_h, hid_h, c.n_embd)

        if self._plan_id is None:
            self._rms(hid_h, 'output_norm.weight', normed_h, 1, c.n_embd)
        else:
            g.decode_step(self._plan_id, pos, seq_len)
        if from_device and on_token is not None and not on_token(self._wait_tokens(self._feed_ticket)[0]):
            g.batch_end()
            return
        if callable(sample_prev):                            # evaluated late: it may include the token just read
            sample_prev = sample_prev()
        mode = sample_mode
        if mode is None and sample:
            mode = ('gpu_fused_topk' if sample_cfg is not None and sample_cfg.temperature > 0.0 and sample_cfg.top_k > 1
                    else 'gpu_matvec_argmax')
        if not sample:
            mode = None
        if mode == 'gpu_fused_topk':
            self._sample_fused_topk(sample_cfg, sample_prev, normed_h)
        elif mode == 'gpu_matvec_argmax':
            fn = (g.map_matvec_argmax_t_xq8_dev if self._kind[self._lm_name] == 'q8'
                  else g.map_matvec_argmax_t_xq4_dev)
            fn(ws, self._map_of[self._lm_name], normed_h, self._wh[self._lm_name],
               W['sample_fused_idx'][0], W['sample_fused_val'][0], W['sample_token'][0],
               c.n_embd, c.n_vocab, self._rows_per_group)
            self._sample_token_ready = True
        elif mode == 'gpu_approx_rerank':
            self._issue_approx_shortlist(sample_cfg, sample_prev, normed_h)
        elif mode in ('gpu_argmax', 'gpu_topk', 'cpu') or return_logits:
            self._issue_full_logits(mode, sample_cfg, sample_prev, normed_h)
        g.batch_end()
        if mode == 'gpu_approx_rerank':
            self._rerank_shortlist(sample_cfg, normed_h)
        if return_logits or mode == 'cpu':
            return g.gather(ws, self._logit_locs).view(np.float32).copy()
        return None

    # ------------------------------------------------------------------ LM-head / sampling modes
    def _effective_top_k(self, cfg):
        """Deterministic decoding collapses to top-1 (reference engine.py:1843-1850)."""
        if cfg.temperature <= 0.0:
            return 1
        k = int(cfg.top_k)
        return 0 if k <= 0 else min(k, self.SAMPLE_TOPK_MAX, self.cfg.n_vocab)

    def _select_sampling_mode(self, cfg):
        """The reference's order of preference (engine.py:3783-3805, predicates :1852-1958) without its host-side
        top-1 mode, which exists for one device family only."""
        g, k = self.gpu, self._effective_top_k(cfg)
        kind = self._kind[self._lm_name]
        has = lambda n: bool(getattr(g, n, False)) or hasattr(g, n.replace('_has_', '', 1))
        matvec_argmax = (k == 1 and cfg.repeat_penalty == 1.0 and has(f'_has_map_matvec_argmax_t_x{kind}_dev'))
        can_topk = 0 < k <= self.SAMPLE_TOPK_MAX
        fused = self._gpu_fused_topk and can_topk and has(f'_has_map_matvec_topk_t_x{kind}_dev')
        rerank = (k > 1 and self._gpu_approx_rerank and self._lm_q4_approx_name is not None and kind == 'q8'
                  and has('_has_map_matvec_topk_t_xq4_ex_dev') and has('_has_map_matvec_rerank_t_xq8_dev'))
        gpu_argmax = k == 1 and cfg.repeat_penalty == 1.0
        if self._force_mode is not None:
            ok = {'gpu_matvec_argmax': matvec_argmax, 'gpu_fused_topk': fused, 'gpu_argmax': gpu_argmax,
                  'gpu_approx_rerank': rerank, 'gpu_topk': can_topk, 'cpu': True}
            if not ok.get(self._force_mode, False):
                raise RuntimeError(f"sampling mode '{self._force_mode}' cannot serve this configuration")
            return self._force_mode
        if k == 1 and matvec_argmax:
            return 'gpu_matvec_argmax'
        if k == 1 and fused:
            return 'gpu_fused_topk'
        if gpu_argmax:
            return 'gpu_argmax'
        if rerank:
            return 'gpu_approx_rerank'
        if fused:
            return 'gpu_fused_topk'
        if can_topk:
            return 'gpu_topk'
        return 'cpu'

    def _repeat_history(self, prompt, generated, cfg):
        """reference engine.py:3731-3738"""
        if cfg.repeat_penalty == 1.0:
            return None
        hist = (list(prompt) + list(generated)) if cfg.repeat_on_prompt else list(generated)
        return hist or None

    def _prepare_repeat_ids(self, prev):
        """The distinct ids among the last SAMPLE_REPEAT_MAX tokens, ascending, into the penalty list's handle
        (reference engine.py:1960-1967); returns how many."""
        recent = sorted({int(t) for t in list(prev)[-self.SAMPLE_REPEAT_MAX:] if 0 <= int(t) < self.cfg.n_vocab})
        if not recent:
            return 0
        self._sample_repeat_ids[:] = 0
        self._sample_repeat_ids[:len(recent)] = recent
        self.gpu.upload_dev(self._sample_repeat_ids, handle=self._sample_repeat_ids_h)
        return len(recent)

    def _write_rand(self):
        self.gpu.scatter(self.WS_MAP, self._rand_locs, np.array([self._rng.random()], np.float32))

    def _softcap(self, val_h, n):
        c, g, A, ws = self.cfg, self.gpu, self.A, self.WS_MAP
        if c.final_softcap > 0:
            g.map_broadcast_dev(ws, A.OP_DIV, val_h, self._final_cap_h, val_h, n)
            g.map_op1_dev(ws, A.OP_TANH, val_h, val_h, n)
            g.map_broadcast_dev(ws, A.OP_MUL, val_h, self._final_cap_h, val_h, n)

    def _issue_full_logits(self, mode, cfg, prev, normed_h):
        """Full logits with the final soft-cap, then, inside the same batch, the arg-max ('gpu_argmax') or
        repeat penalty, top-k, top-p and the draw ('gpu_topk'); reference engine.py:3509-3548."""
        c, g, ws, W = self.cfg, self.gpu, self.WS_MAP, self._ws
        lo_h = W['logits'][0]
        self._proj(normed_h, self._lm_name, lo_h, c.n_embd, c.n_vocab)
        self._softcap(lo_h, c.n_vocab)
        if mode == 'gpu_argmax':
            g.map_argmax_dev(ws, lo_h, W['sample_token'][0], c.n_vocab)
            self._sample_token_ready = True
        elif mode == 'gpu_topk' and cfg is not None:
            if cfg.repeat_penalty != 1.0 and prev:
                n_rep = self._prepare_repeat_ids(prev)
                if n_rep:
                    g.map_repeat_penalty_dev(ws, lo_h, self._sample_repeat_ids_h, n_rep, float(cfg.repeat_penalty))
            k = self._effective_top_k(cfg)
            idx_h, val_h, prob_h = W['sample_topk_idx'][0], W['sample_topk_val'][0], W['sample_topk_prob'][0]
            g.map_topk_dev(ws, lo_h, idx_h, val_h, c.n_vocab, k)
            if cfg.temperature > 0.0:
                g.map_topp_dev(ws, val_h, prob_h, k, float(cfg.temperature), float(cfg.top_p))
                self._write_rand()
                g.map_sample_categorical_dev(ws, idx_h, prob_h, W['sample_rand'][0], W['sample_token'][0], k)
                self._sample_token_ready = True
            # (deterministic decoding reaches this mode only under a repeat penalty with the fused modes switched
            # off: the token is then the first entry of the top-k list, which generate() reads.  The reference
            # applies the penalty a second time on that path, engine.py:2046-2051 after :3524-3529; here it is
            # applied once.)

    def _issue_approx_shortlist(self, cfg, prev, normed_h):
        """First pass of 'gpu_approx_rerank' (reference engine.py:3331-3356): partial top-k per group of rows over
        the 4-bit copy of the LM head, repeat penalty applied."""
        c, g, ws, W = self.cfg, self.gpu, self.WS_MAP, self._ws
        k = min(self._gpu_approx_partial_k, c.n_vocab)
        self._approx_penalty_n = self._prepare_repeat_ids(prev) if (cfg.repeat_penalty != 1.0 and prev) else 0
        self._sample_fused_partial_n = self._fused_groups * k
        self._sample_rerank_n = 0
        name = self._lm_q4_approx_name
        g.map_matvec_topk_t_xq4_ex_dev(ws, self._map_of[name], normed_h, self._wh[name], self._sample_repeat_ids_h,
                                       W['sample_fused_idx'][0], W['sample_fused_val'][0], c.n_embd, c.n_vocab, k,
                                       self._approx_penalty_n, float(cfg.repeat_penalty), self._rows_per_group)

    def _rerank_shortlist(self, cfg, normed_h):
        """Second pass (reference engine.py:3641-3700): the best SAMPLE_APPROX_SHORTLIST_MAX partial values are
        picked on the host, their rows recomputed exactly over the 8-bit head in chunks of SAMPLE_TOPK_MAX."""
        g, ws, c = self.gpu, self.WS_MAP, self.cfg
        n_part = self._sample_fused_partial_n
        if n_part <= 0:
            return
        vals = g.gather(ws, self._fused_val_locs[:n_part]).view(np.float32)
        # (unused slots of a group shorter than k hold -FLT_MAX with row 0: finite, so the reference's test for
        # finiteness lets them through when the whole list is shorter than the shortlist; they are left out here)
        valid = np.flatnonzero(np.isfinite(vals) & (vals > np.float32(-3.0e38)))
        if not valid.size:
            return
        n = min(self.SAMPLE_APPROX_SHORTLIST_MAX, int(valid.size))
        keep = valid[np.argpartition(vals[valid], -n)[-n:]] if n < valid.size else valid
        keep = keep[np.argsort(vals[keep], kind='stable')[::-1]]
        g.batch_begin()
        try:
            g.scatter(ws, self._short_sel_locs[:n], keep.astype(np.float32))
            for ci, lo in enumerate(range(0, n, self.SAMPLE_TOPK_MAX)):
                m = min(self.SAMPLE_TOPK_MAX, n - lo)
                g.map_matvec_rerank_t_xq8_dev(ws, self._map_of[self._lm_name], normed_h, self._wh[self._lm_name],
                                              self._sample_fused_base_h, self._short_sel_chunk_h[ci],
                                              self._sample_repeat_ids_h, self._exact_idx_chunk_h[ci],
                                              self._exact_val_chunk_h[ci], c.n_embd, m, self._approx_penalty_n,
                                              float(cfg.repeat_penalty))
        finally:
            g.batch_end()
        self._sample_rerank_n = n

    def _sample_approx_rerank(self, cfg):
        """Token of 'gpu_approx_rerank' (reference engine.py:2100-2145, device path): top-k of the exact values,
        final soft-cap, then the best one, or top-p and a draw."""
        n, self._sample_rerank_n = self._sample_rerank_n, 0
        if n <= 0:
            return 0
        c, g, ws, W = self.cfg, self.gpu, self.WS_MAP, self._ws
        idx_h, val_h, prob_h = W['sample_topk_idx'][0], W['sample_topk_val'][0], W['sample_topk_prob'][0]
        k = min(self._effective_top_k(cfg), n, self.SAMPLE_TOPK_MAX)
        if k <= 0:
            k = min(n, self.SAMPLE_TOPK_MAX)
        g.batch_begin()
        try:
            g.map_topk_dev(ws, W['sample_exact_val'][0], idx_h, val_h, n, k)
            self._softcap(val_h, k)
            if cfg.temperature <= 0.0:
                g.map_resolve_idx_dev(ws, self._sample_exact_base_h, idx_h, W['sample_token'][0], 1)
            else:
                sel_h = W['sample_short_sel'][0]
                g.map_resolve_idx_dev(ws, self._sample_exact_base_h, idx_h, sel_h, k)
                g.map_topp_dev(ws, val_h, prob_h, k, float(cfg.temperature), float(cfg.top_p))
                self._write_rand()
                g.map_sample_categorical_dev(ws, sel_h, prob_h, W['sample_rand'][0], W['sample_token'][0], k)
        finally:
            g.batch_end()
        return self.read_token()

    def _sample_host(self, logits, cfg, prev):
        """'cpu' mode: the reference's host sampler (engine.py:3708-3729) on the full logits, with this engine's
        seeded generator in place of NumPy's global one."""
        logits = np.array(logits, dtype=np.float32)
        if cfg.repeat_penalty != 1.0 and prev:
            for t in set(prev[-64:]):
                if t < len(logits):
                    logits[t] = logits[t] / cfg.repeat_penalty if logits[t] > 0 else logits[t] * cfg.repeat_penalty
        if cfg.temperature <= 0:
            return int(np.argmax(logits))
        logits /= np.float32(cfg.temperature)
        if cfg.top_k > 0:
            tk = min(cfg.top_k, len(logits))
            ti = np.argpartition(logits, -tk)[-tk:]
            m = np.full_like(logits, -np.inf); m[ti] = logits[ti]; logits = m
        pr = np.exp(logits - np.max(logits)); pr /= pr.sum()
        if cfg.top_p < 1.0:
            si = np.argsort(pr)[::-1]; cs = np.cumsum(pr[si])
            co = int(np.searchsorted(cs, cfg.top_p)) + 1
            m = np.zeros_like(pr); m[si[:co]] = pr[si[:co]]; pr = m / m.sum()
        return int(self._rng.choice(len(pr), p=pr.astype(np.float64) / float(pr.astype(np.float64).sum())))

    def _sample_fused_topk(self, cfg, prev, normed_h):
        """Sampled LM head inside the forward batch, the reference's 'gpu_fused_topk' mode
        (engine.py:3404-3508): partial top-k per group of rows with the repeat penalty, top-k of the
        partial values, final soft-cap on the k survivors, temperature / top-p, token ids resolved
        through the partial list, one categorical draw with a uniform number from the host.  With an
        effective k of 1 (deterministic decoding under a repeat penalty): arg-max of the partial values, resolved."""
        c, g, A, ws, W = self.cfg, self.gpu, self.A, self.WS_MAP, self._ws
        top_k = max(1, self._effective_top_k(cfg))
        n_pen = self._prepare_repeat_ids(prev) if (cfg.repeat_penalty != 1.0 and prev) else 0
        if top_k > 1:
            self._write_rand()            # ahead of the ops: a host write in their middle would split the queue
        pidx_h, pval_h = W['sample_fused_idx'][0], W['sample_fused_val'][0]
        fn = (g.map_matvec_topk_t_xq8_ex_dev if self._kind[self._lm_name] == 'q8' else g.map_matvec_topk_t_xq4_ex_dev)
        fn(ws, self._map_of[self._lm_name], normed_h, self._wh[self._lm_name], self._sample_repeat_ids_h, pidx_h, pval_h,
           c.n_embd, c.n_vocab, top_k, n_pen, float(cfg.repeat_penalty), self._rows_per_group)
        self._sample_fused_partial_n = self._fused_groups * top_k
        idx_h, val_h, prob_h = W['sample_topk_idx'][0], W['sample_topk_val'][0], W['sample_topk_prob'][0]
        if top_k == 1:
            g.map_argmax_dev(ws, pval_h, idx_h, self._sample_fused_partial_n)
            g.map_resolve_idx_dev(ws, self._sample_fused_base_h, idx_h, W['sample_token'][0], 1)
            self._sample_token_ready = True
            return
        g.map_topk_dev(ws, pval_h, idx_h, val_h, self._sample_fused_partial_n, top_k)
        self._softcap(val_h, top_k)
        g.map_topp_dev(ws, val_h, prob_h, top_k, float(cfg.temperature), float(cfg.top_p))
        sel_h = W['sample_short_sel'][0]
        g.map_resolve_idx_dev(ws, self._sample_fused_base_h, idx_h, sel_h, top_k)
        g.map_sample_categorical_dev(ws, sel_h, prob_h, W['sample_rand'][0], W['sample_token'][0], top_k)
        self._sample_token_ready = True

    # ------------------------------------------------------------------ chunked prefill: forward
    def _lockstep_plan_ops(self, m):
        """The layer loop of a lockstep step over m sequences (`_forward_chunk(..., lockstep=True)`) as
        DecodePlanOp records, position and context length as runtime sentinels."""
        c, A, ws = self.cfg, self.A, self.WS_MAP
        P, S = A.DECODE_RUNTIME_POS, A.DECODE_RUNTIME_SEQ_LEN
        E, FF = c.n_embd, c.n_ff
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        C1, CR, CS = self._c1, self._crow, self._cspan
        Op = A.DecodePlanOp
        ops = []
        scale = float(1.0 / np.sqrt(c.head_dim))

        def mm(src, name, dst, K, N):
            kind = A.DECODE_OP_MATMUL_T_XQ8 if self._kind[name] == 'q8' else A.DECODE_OP_MATMUL_T_XQ4
            ops.append(Op(kind=kind, map_id=ws, map_id2=self._map_of[name], h0=C1[src], h1=self._wh[name], h2=C1[dst],
                          u0=m, u1=K, u2=N, u3=1))

        def rms(src, name, dst):
            ops.append(Op(kind=A.DECODE_OP_RMSNORM, map_id=ws, h0=CR[src], h1=self._wrows(name), h2=CR[dst], u0=m, u1=E,
                          f0=c.norm_eps))

        def residual(src, name):
            if name in self._wh:
                ops.append(Op(kind=A.DECODE_OP_RMSNORM_ADD, map_id=ws, h0=CR[src], h1=self._wrows(name), h2=CR['hidden'],
                              h3=CR['hidden'], u0=m, u1=E, f0=c.norm_eps))
            else:
                ops.append(Op(kind=A.DECODE_OP_OP2, map_id=ws, op_code=A.OP_ADD, h0=CS['hidden'], h1=CS[src], h2=CS['hidden'],
                              u0=m * E))

        for L in range(c.n_layer):
            p = f'blk.{L}'
            freq = c.rope_base_global if c.is_global(L) else c.rope_base_local
            rms('hidden', f'{p}.attn_norm.weight', 'normed')
            mm('normed', f'{p}.attn_q.weight', 'q', E, q_dim)
            mm('normed', f'{p}.attn_k.weight', 'k', E, k_dim)
            mm('normed', f'{p}.attn_v.weight', 'v', E, k_dim)
            if self._chunk_qk:
                qn, kn = self._wh[f'{p}.attn_q_norm.weight'], self._wh[f'{p}.attn_k_norm.weight']
                for t in range(m):
                    ops.append(Op(kind=A.DECODE_OP_QK_NORM_ROPE_X, map_id=ws, map_id2=ws, h0=self._c_lq[t], h1=qn,
                                  h2=self._c_lk[t], h3=kn, h4=self._c_qkdst[t], u0=c.n_head, u1=c.head_dim,
                                  u2=c.n_head_kv, u3=c.head_dim_kv, u4=P, f0=freq))
            else:
                ops.append(Op(kind=A.DECODE_OP_ROPE, map_id=ws, h0=self._c_qbase, h1=self._c_qbase, u0=1, u1=m * c.n_head,
                              u2=c.head_dim, u3=P, f0=freq))
                ops.append(Op(kind=A.DECODE_OP_ROPE, map_id=ws, h0=self._c_kbase, h1=self._c_kbase, u0=1,
                              u1=m * c.n_head_kv, u2=c.head_dim_kv, u3=P, f0=freq))
            ops.append(Op(kind=A.DECODE_OP_ROW_COPY_OFFSET, map_id=ws, h0=self._b_kvspec[L], h1=self._c_zero, u0=P,
                          u1=2 * c.n_head_kv * m, u2=c.head_dim_kv))
            for t in range(m):
                ops.append(Op(kind=A.DECODE_OP_MATMUL_T, map_id=ws, h0=self._c_qrows[t], h1=self._k_locs_hs[t][L],
                              h2=self._scores_row_h, u0=1, u1=c.head_dim, u2=S, u3=c.n_head))
                ops.append(Op(kind=A.DECODE_OP_ATTN_SOFTMAX_VALUE, map_id=ws, h0=self._scores_row_h,
                              h1=self._v_locs_hs[t][L], h2=self._c_aorows[t], u0=c.n_head, u1=S, u2=c.head_dim_kv,
                              f0=scale, f1=float(c.attn_softcap)))
            mm('attn_out', f'{p}.attn_output.weight', 'o_proj', c.n_head * c.head_dim_kv, E)
            residual('o_proj', f'{p}.post_attention_norm.weight')
            rms('hidden', f'{p}.ffn_norm.weight', 'normed2')
            mm('normed2', f'{p}.ffn_gate.weight', 'gate', E, FF)
            mm('normed2', f'{p}.ffn_up.weight', 'up', E, FF)
            ops.append(Op(kind=A.DECODE_OP_OP2, map_id=ws, op_code=A.OP_GEGLU if c.ffn_act == 'gelu' else A.OP_SWIGLU,
                          h0=CS['gate'], h1=CS['up'], h2=CS['act'], u0=m * FF))
            mm('act', f'{p}.ffn_down.weight', 'ffn_out', FF, E)
            residual('ffn_out', f'{p}.post_ffw_norm.weight')
        return ops

    def _forward_chunk(self, toks, pos0, sample=True, seq=0, lockstep=False, from_device=False):
        """m <= prefill_chunk prompt tokens at positions pos0 .. pos0 + m - 1 in one pass: the row-wise ops
        over m rows, the projections as [m, K] x [N, K]^T matmuls (the fp16 matrix-core kernel for Q4
        blocks), RoPE and the KV append for all tokens at once, attention token by token over the growing
        cache (sequence `seq` of the batch).  Same ops, operands and order per token as `_forward`; the
        last token's hidden state lands in the decode slots, so decoding continues from there.

        `lockstep`: the rows are one token of each of the first m sequences of the batch instead, all at
        position pos0 -- a batched decode step: every row is rotated for pos0, appended to and attended
        over its own sequence's cache, and gets its own LM head pass (tokens in `read_tokens`).
        `from_device` (a lockstep step of the full batch): the rows' tokens are the ones the previous step left in
        the token slots (`toks` is not looked at); their embedding rows are gathered on the device."""
        c, g, A, ws = self.cfg, self.gpu, self.A, self.WS_MAP
        m = self._batch if from_device else len(toks)
        if not self._chunk or m == 0 or m > self._chunk:
            raise RuntimeError(f"chunk of {m} tokens does not fit prefill_chunk={self._chunk}")
        E, FF = c.n_embd, c.n_ff
        q_dim, k_dim = c.n_head * c.head_dim, c.n_head_kv * c.head_dim_kv
        C1, CR, CS, W = self._c1, self._crow, self._cspan, self._ws
        if from_device:
            feed = self._token_feed()                 # nothing to send: the tokens are on the device
        else:
            toks = np.asarray(toks, np.int64)
        if from_device:
            pass
        elif self._tied:
            locs = (np.uint32(self._off[self._lm_name]) + (toks[:, None] * E + np.arange(E)[None, :])).astype(np.uint32)
            if m in self._c_emb_hs:                   # a handle can be re-uploaded at its own size only
                g.upload_dev(np.ascontiguousarray(locs.reshape(-1)), handle=self._c_emb_hs[m])
            else:
                self._c_emb_hs[m] = self._up(locs.reshape(-1))
            emb_h = self._c_emb_hs[m]
        else:
            emb = self.tensors['token_embd.weight']
            rows = np.empty((m, E), np.float32)
            for i, t in enumerate(toks):
                rows[i] = emb.row(int(t))
            if c.emb_scale != 1.0:
                rows *= np.float32(c.emb_scale)
            g.scatter_contiguous(ws, self._cp['hidden'], rows)      # one range: no list of locations to send along
        if self._c_last_m != m:                                      # where the last row sits only depends on m
            last = self._cp['hidden'] + (m - 1) * E
            g.upload_dev(np.arange(last, last + E, dtype=np.uint32), handle=self._c_last)
            self._c_last_m = m

        def mm(src, name, dst, K, N):
            fn = g.map_matmul_t_xq8_dev if self._kind[name] == 'q8' else g.map_matmul_t_xq4_dev
            fn(ws, self._map_of[name], C1[src], self._wh[name], C1[dst], m, K, N)

        g.batch_begin()
        if from_device:     # (the same launch hands the tokens to the host: _wait_tokens(self._feed_ticket, m))
            self._feed_ticket = g.embed_post_tokens_dev(ws, feed['src'][0], feed['tok_hs'][m], feed['src'][1],
                                                        self._cp['hidden'], m, E, c.n_vocab, float(c.emb_scale))
        elif self._tied:
            src_h, _, _, _ = g.map_gather_dev(self._map_of[self._lm_name], emb_h, m * E)
            g.map_scatter_dev(ws, CS['hidden'], m * E, src_h)
            if c.emb_scale != 1.0:
                g.map_broadcast_dev(ws, A.OP_MUL, CS['hidden'], self._c_embscale_h, CS['hidden'], m * E)
        scale = float(1.0 / np.sqrt(c.head_dim))
        planned = lockstep and self._ls_plan_id is not None and m == self._batch
        if planned:
            g.decode_step(self._ls_plan_id, pos0, pos0 + 1)
        for L in range(0 if planned else c.n_layer):
            p = f'blk.{L}'
            freq = c.rope_base_global if c.is_global(L) else c.rope_base_local
            g.map_rmsnorm_dev(ws, CR['hidden'], self._wrows(f'{p}.attn_norm.weight'), CR['normed'], m, E, c.norm_eps)
            mm('normed', f'{p}.attn_q.weight', 'q', E, q_dim)
            mm('normed', f'{p}.attn_k.weight', 'k', E, k_dim)
            mm('normed', f'{p}.attn_v.weight', 'v', E, k_dim)
            if self._chunk_qk and not lockstep and hasattr(g, 'qk_norm_rope_rows_dev'):
                g.qk_norm_rope_rows_dev(ws, ws, self._c_lq[:m], self._wh[f'{p}.attn_q_norm.weight'], self._c_lk[:m],
                                        self._wh[f'{p}.attn_k_norm.weight'], self._c_qkdst[:m], c.n_head, c.head_dim,
                                        c.n_head_kv, c.head_dim_kv, pos0, freq)
            elif self._chunk_qk:
                qn, kn = self._wh[f'{p}.attn_q_norm.weight'], self._wh[f'{p}.attn_k_norm.weight']
                for t in range(m):
                    g.map_qk_norm_rope_x_dev(ws, ws, self._c_lq[t], qn, self._c_lk[t], kn, self._c_qkdst[t],
                                             c.n_head, c.head_dim, c.n_head_kv, c.head_dim_kv,
                                             pos0 if lockstep else pos0 + t, freq)
            elif lockstep:
                # every row sits at the same position: the m rows' heads rotate as the heads of one token
                g.map_rope_dev(ws, self._c_qbase, self._c_qbase, 1, m * c.n_head, c.head_dim, pos0, freq)
                g.map_rope_dev(ws, self._c_kbase, self._c_kbase, 1, m * c.n_head_kv, c.head_dim_kv, pos0, freq)
            else:
                g.map_rope_dev(ws, CR['q'], CR['q'], m, c.n_head, c.head_dim, pos0, freq)
                g.map_rope_dev(ws, CR['k'], CR['k'], m, c.n_head_kv, c.head_dim_kv, pos0, freq)
            g.map_row_copy_offset_dev(ws, self._b_kvspec[L] if lockstep else self._c_kvspec[(seq, L)], self._c_zero, pos0,
                                      2 * c.n_head_kv * m, c.head_dim_kv)
            if not lockstep and hasattr(g, 'attn_causal_rows_dev'):
                # the m (scores, softmax . V) pairs of the chunk in one native call
                g.attn_causal_rows_dev(ws, self._c_qrows[:m], self._k_locs_hs[seq][L], self._scores_row_h,
                                       self._v_locs_hs[seq][L], self._c_aorows[:m], c.head_dim, pos0 + 1, c.n_head,
                                       c.head_dim_kv, scale, float(c.attn_softcap))
            for t in range(0 if not lockstep and hasattr(g, 'attn_causal_rows_dev') else m):
                n_keys = pos0 + 1 if lockstep else pos0 + t + 1
                sq = t if lockstep else seq
                g.map_matmul_t_dev(ws, self._c_qrows[t], self._k_locs_hs[sq][L], self._scores_row_h, 1, c.head_dim, n_keys,
                                   c.n_head)
                g.map_attn_softmax_value_dev(ws, self._scores_row_h, self._v_locs_hs[sq][L], self._c_aorows[t], c.n_head,
                                             n_keys, c.head_dim_kv, scale, float(c.attn_softcap))
            mm('attn_out', f'{p}.attn_output.weight', 'o_proj', c.n_head * c.head_dim_kv, E)
            pan = f'{p}.post_attention_norm.weight'
            if pan in self._wh:
                g.map_rmsnorm_add_dev(ws, CR['o_proj'], self._wrows(pan), CR['hidden'], CR['hidden'], m, E, c.norm_eps)
            else:
                g.map_op2_dev(ws, A.OP_ADD, CS['hidden'], CS['o_proj'], CS['hidden'], m * E)
            g.map_rmsnorm_dev(ws, CR['hidden'], self._wrows(f'{p}.ffn_norm.weight'), CR['normed2'], m, E, c.norm_eps)
            mm('normed2', f'{p}.ffn_gate.weight', 'gate', E, FF)
            mm('normed2', f'{p}.ffn_up.weight', 'up', E, FF)
            g.map_op2_dev(ws, A.OP_GEGLU if c.ffn_act == 'gelu' else A.OP_SWIGLU, CS['gate'], CS['up'], CS['act'], m * FF)
            mm('act', f'{p}.ffn_down.weight', 'ffn_out', FF, E)
            pfn = f'{p}.post_ffw_norm.weight'
            if pfn in self._wh:
                g.map_rmsnorm_add_dev(ws, CR['ffn_out'], self._wrows(pfn), CR['hidden'], CR['hidden'], m, E, c.norm_eps)
            else:
                g.map_op2_dev(ws, A.OP_ADD, CS['hidden'], CS['ffn_out'], CS['hidden'], m * E)
        if lockstep:
            # every row is the newest token of its sequence: output norm over the rows, one LM head pass per row
            fn = (g.map_matvec_argmax_t_xq8_dev if self._kind[self._lm_name] == 'q8' else g.map_matvec_argmax_t_xq4_dev)
            g.map_rmsnorm_dev(ws, CR['hidden'], self._wrows('output_norm.weight'), CR['normed'], m, E, c.norm_eps)
            for t in range(m):
                fn(ws, self._map_of[self._lm_name], self._c_n1[t], self._wh[self._lm_name], W['sample_fused_idx'][0],
                   W['sample_fused_val'][0], self._c_tok1[t], E, c.n_vocab, self._rows_per_group)
            g.batch_end()
            return
        # the last token's hidden state -> the decode slots; output norm and LM head as in a decode step
        src_h, _, _, _ = g.map_gather_dev(ws, self._c_last, E)
        g.map_scatter_dev(ws, W['hidden'][0], E, src_h)
        if sample:
            self._rms(W['hidden'][0], 'output_norm.weight', W['normed'][0], 1, E)
            fn = (g.map_matvec_argmax_t_xq8_dev if self._kind[self._lm_name] == 'q8' else g.map_matvec_argmax_t_xq4_dev)
            fn(ws, self._map_of[self._lm_name], W['normed'][0], self._wh[self._lm_name], W['sample_fused_idx'][0],
               W['sample_fused_val'][0], W['sample_token'][0], E, c.n_vocab, self._rows_per_group)
            self._sample_token_ready = True
        g.batch_end()

    def prefill(self, token_ids, pos0=0, sample=True, seq=0):
        """The prompt in chunks of `prefill_chunk` tokens (token by token when the engine was built
        without one); the LM head runs after the last token only.  `seq`: which sequence of the batch."""
        n = len(token_ids)
        if not self._chunk:
            for i, t in enumerate(token_ids):
                self._forward(int(t), pos0 + i, sample=sample and i == n - 1)
            return
        for lo in range(0, n, self._chunk):
            hi = min(n, lo + self._chunk)
            self._forward_chunk(token_ids[lo:hi], pos0 + lo, sample=sample and hi == n, seq=seq)

    def read_token(self):
        # reference engine.py:1979-1981: token id crosses the boundary as float32
        tok = self.gpu.gather(self.WS_MAP, self._sample_locs).view(np.float32)
        return int(tok[0]) if tok.size else 0

    def read_tokens(self, m):
        """Tokens of the first m rows after a batched decode step."""
        return [int(t) for t in self.gpu.gather(self.WS_MAP, self._c_tok_locs[:m]).view(np.float32)]

    def generate_batch(self, prompts, max_tokens, forced=None):
        """Greedy decoding of len(prompts) <= batch sequences in lockstep (prompts of equal length): each
        prompt is prefilled into its own cache, then every step runs the row-wise ops and projections
        once over all sequences ([B, K] x [N, K]^T matmuls) and attention per sequence.  `forced[s]`:
        tokens fed back for sequence s instead of its own choices.  Returns (tokens per sequence, stats)."""
        B, P = len(prompts), len(prompts[0])
        if B > self._batch or any(len(p) != P for p in prompts):
            raise RuntimeError(f"need at most {self._batch} prompts of equal length")
        if P + max_tokens > self._kv_cap:
            raise RuntimeError(f"KV cache too small: need {P + max_tokens} tokens but kv_cap={self._kv_cap}.")
        self.reset()
        # (the device-side embedding table of an untied model is filled on first use: before the clock starts)
        ahead = (forced is None and self._lookahead and B == self._batch and B > 1 and max_tokens > 1
                 and self._token_feed() is not None)
        t0 = time.perf_counter()
        cur = []
        for sq, pr in enumerate(prompts):
            self.prefill([int(t) for t in pr], seq=sq)
            cur.append(self.read_token())
        self.gpu.sync()
        t_pre = time.perf_counter() - t0
        out = [[] for _ in range(B)]
        t0 = time.perf_counter()
        if ahead:
            # One step of lookahead: step n + 1 takes its tokens from the slots step n's LM head passes write and is
            # issued before the host has seen them; the host still reads every step's tokens, in order, one issue late.
            for sq in range(B):
                out[sq].append(cur[sq])
            self._forward_chunk(cur, P, lockstep=True)
            for step in range(1, max_tokens):
                self._forward_chunk(None, P + step, lockstep=True, from_device=True)
                cur = self._wait_tokens(self._feed_ticket, B)      # the tokens that step consumes
                for sq in range(B):
                    out[sq].append(cur[sq])
        for step in range(0 if not ahead else max_tokens, max_tokens):
            for sq in range(B):
                out[sq].append(cur[sq])
            feed = cur if forced is None else [int(forced[sq][step]) for sq in range(B)]
            self._forward_chunk(feed, P + step, lockstep=True)
            cur = self.read_tokens(B)
        self.gpu.sync()
        t_dec = time.perf_counter() - t0
        return out, {'n_seq': B, 'n_prompt': P, 'n_gen': max_tokens, 'prefill_s': t_pre, 'decode_s': t_dec,
                     'decode_tps': B * max_tokens / t_dec if t_dec > 0 else 0.0}

    def read_slot(self, name):
        _, sz, pos = self._ws[name]
        return self.gpu.gather(self.WS_MAP, np.arange(pos, pos + sz, dtype=np.uint32)).view(np.float32).copy()

    def reset(self):
        c = self.cfg
        sc_sz = c.n_head * self._kv_cap
        self.gpu.scatter(self.WS_MAP, np.arange(sc_sz, dtype=np.uint32), np.full(sc_sz, -1e30, np.float32))
        self._sample_token_ready = False

    # ------------------------------------------------------------------ generate
    def generate(self, token_ids, config=None, forced=None, reuse_prefix=0):
        """Generation with the LM-head / sampling mode the configuration selects (`_select_sampling_mode`: greedy
        GEMV + arg-max, partial top-k fused into the LM head, full logits + arg-max / top-k, approximate shortlist
        + exact rerank, or the host sampler; one uniform number per drawn token from a host generator seeded with
        `config.seed`).  Prefill is the same `_forward` once per prompt token (in chunks on the matrix cores when
        the engine was built with `prefill_chunk`), LM head only on the last one; `decode_tps = n_gen /
        wall(decode loop)` including the per-token read-back (reference engine.py:3838-3931).  The greedy and the
        fused top-k loops run one step ahead of the read-back unless `forced` is given or the engine was built
        with `lookahead=False`: same tokens, same number of steps.
        `forced`, when given, is a token list fed back instead of the model's own choices (teacher forcing)
        while the choices are still returned.
        `reuse_prefix=n`: the caches still hold the rows of the first n prompt tokens from the previous call (same
        tokens, e.g. the earlier turns of a conversation); prefill starts at position n (reference
        engine.py:3815-3833)."""
        config = config or GenerationConfig()
        token_ids = [int(t) for t in token_ids]
        if len(token_ids) + config.max_tokens > self._kv_cap:
            raise RuntimeError(
                f"KV cache too small: need {len(token_ids) + config.max_tokens} tokens but "
                f"kv_cap={self._kv_cap}. Reinitialize with kv_cap>={len(token_ids) + config.max_tokens}.")
        mode = self._select_sampling_mode(config)
        reuse = max(0, int(reuse_prefix or 0))
        if reuse >= len(token_ids):
            reuse = 0
        self.reset()
        # (the device-side embedding table of an untied model is filled on first use: before the clock starts)
        ahead = (forced is None and self._lookahead and config.max_tokens > 0
                 and mode in ('gpu_matvec_argmax', 'gpu_fused_topk') and self._token_feed() is not None)
        self._rng = np.random.default_rng(config.seed)
        fed = []                                             # tokens fed back after the prompt
        prev = lambda: self._repeat_history(token_ids, fed, config)
        tp = time.perf_counter()
        last = len(token_ids) - 1
        logits = None
        todo = token_ids[reuse:]
        if self._chunk and mode == 'gpu_matvec_argmax':
            self.prefill(todo, pos0=reuse)
        else:
            if self._chunk and len(todo) > 1:                # all but the last token: no LM head needed
                self.prefill(todo[:-1], pos0=reuse, sample=False)
                reuse = last
            for i in range(reuse, len(token_ids)):
                logits = self._forward(token_ids[i], i, sample=(i == last), sample_cfg=config, sample_prev=prev,
                                       sample_mode=mode if i == last else None)
        n_reused = len(token_ids) - len(todo)
        self.gpu.sync()
        t_pre = time.perf_counter() - tp
        out, ttimes = [], []
        td = time.perf_counter()
        if ahead and mode == 'gpu_fused_topk':
            # Sampled decoding one step ahead: the layers of the step that consumes token n are issued at once (the
            # token's embedding row is gathered on the device); the host reads token n while they run, builds the
            # repeat-penalty list that includes it and only then issues the step's LM head and sampling ops.
            def seen(nt):
                if nt in config.eos_token_ids:
                    return False
                out.append(nt)
                fed.append(nt)
                return True
            for step in range(config.max_tokens):
                t0 = time.perf_counter()
                n_before = len(out)
                self._forward(None, len(token_ids) + step, sample=True, sample_cfg=config, sample_prev=prev,
                              from_device=True, on_token=seen, sample_mode=mode)
                if len(out) == n_before:
                    break
                ttimes.append(time.perf_counter() - t0)
        elif ahead:
            # One step of lookahead: the step that consumes token n takes it from the device slot and is issued
            # before the host has seen token n; the host reads every token, in order, one issue late.  A stop token
            # is therefore noticed after one step too many was issued (its KV row is never read).
            for step in range(config.max_tokens):
                t0 = time.perf_counter()
                self._forward(None, len(token_ids) + step, from_device=True, sample_mode=mode)
                nt = self._wait_tokens(self._feed_ticket)[0]       # the token that step consumes
                if nt in config.eos_token_ids:
                    break
                out.append(nt)
                fed.append(nt)
                ttimes.append(time.perf_counter() - t0)
        for step in range(0 if not ahead else config.max_tokens, config.max_tokens):
            t0 = time.perf_counter()
            nt = self._next_token(mode, config, logits, prev())
            if nt in config.eos_token_ids:
                break
            out.append(nt)
            fed.append(nt if forced is None else int(forced[step]))
            logits = self._forward(fed[-1], len(token_ids) + step, sample=True, sample_cfg=config, sample_prev=prev,
                                   sample_mode=mode)
            ttimes.append(time.perf_counter() - t0)
        self.gpu.sync()
        t_dec = time.perf_counter() - td
        n_p, n_g = len(token_ids) - n_reused, len(out)
        return out, {
            'n_prompt': n_p, 'n_prompt_total': len(token_ids), 'n_prompt_reused': n_reused, 'n_prompt_prefilled': n_p,
            'n_gen': n_g, 'prefill_s': t_pre, 'decode_s': t_dec,
            'prefill_tps': n_p / t_pre if t_pre > 0 else 0.0,
            'decode_tps': n_g / t_dec if t_dec > 0 else 0.0,
            'avg_ms': float(np.mean(ttimes) * 1000) if ttimes else 0.0,
            'sampling_mode': mode,
        }

    def _next_token(self, mode, cfg, logits, prev):
        """The token the last forward pass chose, per mode (reference engine.py:3856-3875)."""
        ready, self._sample_token_ready = self._sample_token_ready, False
        if mode == 'gpu_approx_rerank':
            return self._sample_approx_rerank(cfg)
        if mode == 'cpu':
            return self._sample_host(logits, cfg, prev)
        if mode == 'gpu_topk' and not ready:                 # deterministic: the head of the top-k list
            pos = self._ws['sample_topk_idx'][2]
            return int(self.gpu.gather(self.WS_MAP, np.array([pos], np.uint32)).view(np.float32)[0])
        return self.read_token()
