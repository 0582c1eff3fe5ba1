"""NumPy restatement of the ADAMAH op surface (oracle; test infrastructure, never shipped).

Every method follows the reference's definition of the op -- the GLSL shader that computes
it and the C dispatcher that validates it -- cited per method as
``adamah-MAIN/adamah/...`` paths.  Method names, argument order and error behaviour are
those of the reference Python binding ``adamah-MAIN/adamah/__init__.py`` (class Adamah),
so a decode harness can run unchanged on this backend or on the HIP library.

Representation: a map is a flat array (float32 for F32 maps; raw codes for Q4/Q8 maps plus
float32 per-group ``scale``/``zp``); a handle is a byte blob interpreted as ``uint32`` locs
or ``float32`` data exactly like the reference's device resources.

Floating point: element-wise ops are evaluated in float32 in the shader's order.  Dot
products and reductions are accumulated in float64 and rounded once -- the reference's own
summation order (a 128- or 256-lane strided partial sum and a tree) is one of many valid
float32 orders, and the float64 value is what all of them approximate; parity tests
compare within the stated relative-L2 tolerance.  Per-weight dequantisation
(``float(code) * scale + zp``, two float32 roundings) is bit-exact.

Parity pins (what checks this file against something other than itself) live in
``tests/test_oracle_kat.py`` (the reference's literal known-answer vectors) and
``tests/test_oracle_math.py`` (closed forms / invariants).  Unpinned at ulp level:
``OP1``/``OP2`` transcendental codes other than TANH/EXP/GEGLU/SWIGLU, and the device
quantiser's ``round()`` tie direction (implementation-defined in GLSL).
"""
import numpy as np

ERR_BACKEND, ERR_MEMORY, ERR_INVALID, ERR_NOT_FOUND = -1, -2, -3, -4
DTYPE_F32, DTYPE_BF16, DTYPE_Q8, DTYPE_Q4, DTYPE_Q6 = 0, 1, 2, 3, 4
MAX_MAPS = 16
NEG_MAX = np.float32(-3.402823466e+38)

OP_MUL, OP_DIV, OP_ADD, OP_SUB = 2, 3, 0, 1
OP_GEGLU, OP_SWIGLU, OP_TANH = 34, 35, 5

f32 = np.float32


class _Map:
    def __init__(self, dtype, pack_size, n_packs, group_size):
        self.dtype, self.pack_size, self.n_packs = dtype, pack_size, n_packs
        self.n = int(pack_size) * int(n_packs)
        self.group_size = group_size if dtype in (DTYPE_Q8, DTYPE_Q4, DTYPE_Q6) else 0
        if dtype == DTYPE_F32:
            self.data = np.zeros(self.n, np.float32)
        elif dtype == DTYPE_Q8:
            self.data = np.zeros(((self.n + 3) // 4) * 4, np.uint8)      # one code per byte
        elif dtype == DTYPE_Q4:
            self.data = np.zeros(((self.n + 7) // 8) * 4, np.uint8)      # two codes per byte
        else:
            raise NotImplementedError("oracle covers F32, Q8 and Q4 maps only")
        self.n_groups = 0
        self.scale = self.zp = None
        if self.group_size > 0:
            # adamah.c:2801-2820 -- default qparams are (scale=1, zp=0)
            self.n_groups = (self.n + group_size - 1) // group_size
            self.scale = np.ones(self.n_groups, np.float32)
            self.zp = np.zeros(self.n_groups, np.float32)
        self.cache = {}

    def codes(self, idx):
        idx = np.asarray(idx, dtype=np.int64)
        if self.dtype == DTYPE_Q8:
            return self.data[idx]
        b = self.data[idx >> 1]
        return np.where(idx & 1, b >> 4, b & 0x0F).astype(np.uint8)

    def deq(self, idx):
        """float(code) * scale[g] + zp[g], g = idx // group_size over the whole map
        (shaders/src/f32/map_matvec_t_xq4.comp:49-55, map_matvec_t_xq8.comp:47-53)."""
        idx = np.asarray(idx, dtype=np.int64)
        g = idx // self.group_size
        return (self.codes(idx).astype(np.float32) * self.scale[g] + self.zp[g]).astype(np.float32)

    def deq_range(self, start, count):
        """Dequantised values of elements [start, start+count) (cached; same arithmetic as deq)."""
        key = (start, count)
        w = self.cache.get(key)
        if w is None:
            gs = self.group_size
            if start % gs == 0 and count % gs == 0 and (self.dtype == DTYPE_Q8 or start % 2 == 0):
                # whole groups: slice the code bytes instead of building an index per element
                if self.dtype == DTYPE_Q8:
                    c = self.data[start:start + count]
                else:
                    b = self.data[start // 2:(start + count) // 2]
                    c = np.empty(count, np.uint8)
                    c[0::2] = b & 0x0F
                    c[1::2] = b >> 4
                g0 = start // gs
                sc = self.scale[g0:g0 + count // gs][:, None]
                zp = self.zp[g0:g0 + count // gs][:, None]
                w = (c.reshape(-1, gs).astype(np.float32) * sc + zp).astype(np.float32).reshape(-1)
            else:
                w = self.deq(np.arange(start, start + count, dtype=np.int64))
            if len(self.cache) > 512:
                self.cache.clear()
            self.cache[key] = w
        return w


class NumpyAdamah:
    """CPU oracle with the reference binding's method surface."""

    DTYPE_F32, DTYPE_BF16, DTYPE_Q8, DTYPE_Q4, DTYPE_Q6 = 0, 1, 2, 3, 4

    def __init__(self):
        self.maps = {}
        self.res = {}
        self._next = 1
        self._fusion = False
        self._sched = 0
        self._active_dtype = 0
        self._group_size = 128
        self._has_map_scatter_contiguous = True
        self._has_map_scatter_q4_packed_contiguous = True
        self._has_map_matvec_argmax_t_xq4_dev = True
        self._has_map_matvec_argmax_t_xq8_dev = True
        self._has_decode_plan = False
        self._is_integrated_gpu = False
        self.op_count = 0

    # ------------------------------------------------------------------ helpers
    def _fail(self, fn, code):
        raise RuntimeError(f"{fn} failed with code {code}")

    def _map(self, fn, mid, dtype=None):
        m = self.maps.get(mid) if 0 <= mid < MAX_MAPS else None
        if m is None or (dtype is not None and m.dtype != dtype):
            self._fail(fn, ERR_INVALID)
        return m

    def _h(self, fn, h, min_words=0):
        r = self.res.get(h)
        if r is None or r.size < 4 * min_words:
            self._fail(fn, ERR_INVALID)
        return r

    def _locs(self, fn, h, n=1):
        return self._h(fn, h, n).view(np.uint32)[:n].astype(np.int64)

    def _chk(self, fn, m, lo, hi):
        if lo < 0 or hi > m.n:
            self._fail(fn, ERR_INVALID)

    # ------------------------------------------------------------------ lifecycle
    def shutdown(self):
        self.maps.clear(); self.res.clear()

    def sync(self): pass
    def synchronize(self, ticket): pass
    def synchronize_all(self): pass
    def batch_begin(self): pass
    def batch_end(self): pass

    def fusion_enable(self, enable): self._fusion = bool(enable)
    def fusion_is_enabled(self): return self._fusion
    def fusion_flush(self): pass

    def fusion_set_scheduler_mode(self, mode):
        names = {"legacy": 0, "alias_safe": 1, "level_batched": 2}
        self._sched = names[mode.strip().lower()] if isinstance(mode, str) else int(mode)

    def fusion_get_scheduler_mode(self):
        return {0: "legacy", 1: "alias_safe", 2: "level_batched"}.get(self._sched, "unknown")

    def register_loc_span(self, handle, map_id, start, count): pass
    def register_row_base_span(self, handle, map_id, start, count, stride, row_size): pass
    def clear_loc_alias_meta(self, handle): pass
    def reset_native_stats(self): self.op_count = 0
    def get_native_stats(self): return {"dispatch_count": self.op_count}

    # ------------------------------------------------------------------ maps
    def set_dtype(self, dtype, group_size=128):
        self._active_dtype, self._group_size = dtype, group_size

    def map_create_typed(self, map_id, dtype, pack_size, n_packs, group_size=128):
        # adamah.c:2698-2824
        if not (0 <= map_id < MAX_MAPS) or dtype > DTYPE_Q6:
            raise RuntimeError(f"map_init_dtype({dtype}) failed: {ERR_INVALID}")
        self.maps[map_id] = _Map(dtype, pack_size, n_packs, group_size)

    def map_create(self, map_id, pack_size=0, n_packs=0, word_size=0, **kw):
        self.map_create_typed(map_id, self._active_dtype, pack_size, n_packs, self._group_size)

    def map_init(self, map_id, word_size, pack_size, n_packs):
        self.map_create_typed(map_id, {4: 0, 2: 1, 1: 2}.get(word_size, 0), pack_size, n_packs, 128)

    def map_destroy(self, map_id):
        if map_id not in self.maps:
            self._fail("map_destroy", ERR_INVALID)
        del self.maps[map_id]

    def map_size(self, map_id):
        m = self.maps.get(map_id)
        return m.n_packs if m else 0

    def set_qparams(self, map_id, scales, zero_points):
        # adamah.c:4621-4633: groups [0, n) are overwritten; n > n_groups is invalid
        m = self.maps.get(map_id)
        s = np.ascontiguousarray(scales, np.float32); z = np.ascontiguousarray(zero_points, np.float32)
        if m is None or m.scale is None or s.size > m.n_groups:
            self._fail("map_set_qparams", ERR_INVALID)
        m.scale[:s.size] = s; m.zp[:s.size] = z[:s.size]; m.cache.clear()

    # ------------------------------------------------------------------ host <-> map
    def scatter(self, map_id, locs, data):
        """adamah.c:3087-3372.  F32/Q8: copy packs as stored.  Q4: ``data`` is float32 and
        is quantised on the device (shaders/src/q4/map_scatter.comp:13-34)."""
        m = self._map("map_scatter", map_id)
        locs = np.ascontiguousarray(locs, np.uint32).astype(np.int64)
        if locs.size == 0:
            return 0
        ps = m.pack_size
        idx = (locs[:, None] * ps + np.arange(ps)).reshape(-1)
        if idx.min() < 0 or idx.max() >= m.n:
            self._fail("map_scatter", ERR_INVALID)
        if m.dtype == DTYPE_Q4:
            self._quantise_q4(m, idx, np.ascontiguousarray(data, np.float32).reshape(-1)[:idx.size])
        elif m.dtype == DTYPE_Q8:
            m.data[idx] = np.ascontiguousarray(data).view(np.uint8).reshape(-1)[:idx.size]
        else:
            m.data[idx] = self._kv_round(map_id, idx, np.ascontiguousarray(data).view(np.float32).reshape(-1)[:idx.size])
        m.cache.clear()
        return 0

    map_scatter = scatter

    def _kv_round(self, map_id, idx, vals):
        """Values written into a declared fp16 KV range are rounded to fp16 (see kv_cache_fp16)."""
        kv = getattr(self, "_kv_fp16", {}).get(map_id)
        if kv is None:
            return vals
        inside = (idx >= kv[0]) & (idx < kv[0] + kv[1])
        out = np.array(vals, dtype=np.float32, copy=True)
        out[inside] = out[inside].astype(np.float16).astype(np.float32)
        return out

    def scatter_contiguous(self, map_id, start_pack, data, n_locs=None):
        arr = np.ascontiguousarray(data)
        n = int(arr.size if n_locs is None else n_locs)
        m = self._map("map_scatter_contiguous", map_id)
        if n and (start_pack >= m.n_packs or start_pack + n > m.n_packs):
            self._fail("map_scatter_contiguous", ERR_INVALID)
        return self.scatter(map_id, np.arange(start_pack, start_pack + n, dtype=np.uint32), arr)

    def scatter_q4_packed_contiguous(self, map_id, start_pack, packed_u8, n_locs=None):
        # adamah.c:3035-3082: raw nibble bytes land at byte start_pack/2
        arr = np.ascontiguousarray(packed_u8, np.uint8).reshape(-1)
        n = int(arr.size * 2 if n_locs is None else n_locs)
        m = self._map("map_scatter_q4_packed_contiguous", map_id)
        if n == 0:
            return 0
        if (m.dtype != DTYPE_Q4 or m.pack_size != 1 or start_pack >= m.n_packs or
                start_pack + n > m.n_packs or (start_pack & 1) or (n & 1)):
            self._fail("map_scatter_q4_packed_contiguous", ERR_INVALID)
        m.data[start_pack // 2: start_pack // 2 + n // 2] = arr[:n // 2]
        m.cache.clear()
        return 0

    def _quantise_q4(self, m, idx, vals):
        g = idx // m.group_size
        qf = (vals - m.zp[g]) / np.maximum(m.scale[g], np.float32(1e-10))
        q = np.clip(np.rint(qf), 0, 15).astype(np.uint8)   # rint: ties-to-even (GLSL leaves ties open)
        for i, c in zip(idx, q):
            b = m.data[i >> 1]
            m.data[i >> 1] = (b & 0x0F) | (c << 4) if (i & 1) else (b & 0xF0) | c

    def gather(self, map_id, locs, n_packs=None, n_locs=None):
        """adamah.c:3374-3565: returns the stored words; float32 maps are read back with
        ``.view(np.float32)`` by callers (__init__.py:1347-1360)."""
        m = self._map("map_gather", map_id)
        locs = np.ascontiguousarray(locs, np.uint32).astype(np.int64)
        n = n_locs if n_locs is not None else (n_packs if n_packs is not None else len(locs))
        locs = locs[:n]
        out = np.zeros(n, np.uint32)
        if m.dtype == DTYPE_F32 and m.pack_size == 1:
            ok = locs < m.n
            out.view(np.float32)[ok] = m.data[locs[ok]]
        elif m.dtype == DTYPE_F32:
            out = np.zeros(n * m.pack_size, np.uint32)
            idx = (locs[:, None] * m.pack_size + np.arange(m.pack_size)).reshape(-1)
            out.view(np.float32)[:] = m.data[idx]
        else:
            raw = m.data[np.minimum(locs, m.data.size - 1)]
            out.view(np.uint8)[:n] = raw
        return out

    map_gather = gather

    # ------------------------------------------------------------------ handles
    def upload_dev(self, data, handle=0):
        # adamah.c:3570-3663: new handle when 0; re-upload needs identical byte size; 0 = failure
        arr = np.ascontiguousarray(data)
        raw = arr.view(np.uint8).reshape(-1).copy()
        if raw.size == 0:
            return 0, 0
        if handle == 0:
            handle = self._next; self._next += 1
        elif handle not in self.res or self.res[handle].size != raw.size:
            return 0, 0
        self.res[handle] = raw
        return handle, 0

    def download_dev(self, handle, n_elems, dtype=np.float32):
        r = self.res.get(handle)
        nb = int(n_elems) * np.dtype(dtype).itemsize
        if r is None or nb == 0 or nb > r.size:
            self._fail("map_download_dev", ERR_INVALID)
        return r[:nb].view(dtype).copy()

    def map_gather_dev(self, map_id, locs_handle, n_locs):
        """adamah.c:3788-3927: always materialises logical values as float32 (Q4/Q8 maps are
        dequantised, shaders/src/q4/map_gather.comp)."""
        m = self.maps.get(map_id)
        r = self.res.get(locs_handle)
        if m is None or n_locs == 0 or r is None or r.size < 4 * n_locs:
            return 0, 0, 0, np.float32
        locs = r.view(np.uint32)[:n_locs].astype(np.int64)
        idx = (locs[:, None] * m.pack_size + np.arange(m.pack_size)).reshape(-1)
        vals = m.data[idx] if m.dtype == DTYPE_F32 else m.deq(idx)
        h = self._next; self._next += 1
        self.res[h] = np.ascontiguousarray(vals, np.float32).view(np.uint8).copy()
        return h, 0, n_locs * m.pack_size, np.float32

    def map_scatter_dev(self, map_id, locs_handle, n_locs, src_handle):
        # adamah.c:3703-3786 + shaders/src/f32/map_scatter.comp
        m = self.maps.get(map_id)
        lr, sr = self.res.get(locs_handle), self.res.get(src_handle)
        if m is None or n_locs == 0 or lr is None or sr is None or lr.size < 4 * n_locs:
            return 0
        if sr.size < n_locs * m.pack_size * 4 or m.dtype != DTYPE_F32:
            return 0
        locs = lr.view(np.uint32)[:n_locs].astype(np.int64)
        idx = (locs[:, None] * m.pack_size + np.arange(m.pack_size)).reshape(-1)
        m.data[idx] = self._kv_round(map_id, idx, sr.view(np.float32)[:idx.size])
        return 0

    # ------------------------------------------------------------------ elementwise
    def _ew_idx(self, fn, m, h, n):
        locs = self._locs(fn, h, n)
        idx = (locs[:, None] * m.pack_size + np.arange(m.pack_size)).reshape(-1)
        if idx.size and idx.max() >= m.n:
            self._fail(fn, ERR_INVALID)
        return idx

    def map_op1_dev(self, map_id, op, locs_in_handle, locs_out_handle, n):
        """shaders/src/f32/map_op1.comp:20-56 (codes 0..33)."""
        self.op_count += 1
        m = self._map("map_op1_dev", map_id, DTYPE_F32)
        if n == 0:
            return
        v = m.data[self._ew_idx("map_op1_dev", m, locs_in_handle, n)]
        one = f32(1.0)
        with np.errstate(all="ignore"):
            gelu = lambda x: f32(0.5) * x * (one + np.tanh(f32(0.797884583) * (x + f32(0.0447149985) * x * x * x)))
            table = {
                0: lambda: -v, 1: lambda: np.abs(v), 2: lambda: np.sqrt(np.maximum(v, 0)),
                3: lambda: np.exp(v), 4: lambda: np.log(np.maximum(v, f32(1e-7))),
                5: lambda: np.tanh(v), 6: lambda: np.maximum(f32(0), v), 7: lambda: gelu(v),
                8: lambda: np.sin(v), 9: lambda: np.cos(v), 10: lambda: np.tan(v),
                11: lambda: np.arcsin(np.clip(v, -1, 1)), 12: lambda: np.arccos(np.clip(v, -1, 1)),
                13: lambda: np.arctan(v), 14: lambda: np.sinh(v), 15: lambda: np.cosh(v),
                16: lambda: one / (one + np.exp(-v)), 17: lambda: v / (one + np.exp(-v)),
                18: lambda: v * np.tanh(np.log(one + np.exp(v))),
                19: lambda: np.where(v > 0, v, f32(1.67325997) * (np.exp(v) - one)) * f32(1.05069995),
                20: lambda: np.where(v > 0, v, np.exp(v) - one), 21: lambda: np.maximum(v, f32(0.01) * v),
                22: lambda: np.ceil(v), 23: lambda: np.floor(v), 24: lambda: np.rint(v),
                25: lambda: np.sign(v), 26: lambda: one / v, 27: lambda: v * v, 28: lambda: v * v * v,
                29: lambda: np.log(one + np.exp(v)), 30: lambda: np.clip(f32(0.2) * v + f32(0.5), 0, 1),
                31: lambda: v * np.clip(f32(0.2) * v + f32(0.5), 0, 1), 32: lambda: np.exp(v) - one,
                33: lambda: np.log(one + v),
            }
            r = table.get(op, lambda: v)()
        m.data[self._ew_idx("map_op1_dev", m, locs_out_handle, n)] = np.asarray(r, np.float32)

    def map_op2_dev(self, map_id, op, locs_a_handle, locs_b_handle, locs_out_handle, n):
        """shaders/src/f32/map_op2.comp:11-46 (0 ADD .. 19, 34 GEGLU, 35 SWIGLU)."""
        self.op_count += 1
        m = self._map("map_op2_dev", map_id, DTYPE_F32)
        if n == 0:
            return
        a = m.data[self._ew_idx("map_op2_dev", m, locs_a_handle, n)]
        b = m.data[self._ew_idx("map_op2_dev", m, locs_b_handle, n)]
        one = f32(1.0)
        with np.errstate(all="ignore"):
            if op == 0: r = a + b
            elif op == 1: r = a - b
            elif op == 2: r = a * b
            elif op == 3: r = a / b
            elif op == 4: r = np.power(a, b)
            elif op == 5: r = np.minimum(a, b)
            elif op == 6: r = np.maximum(a, b)
            elif op == 7: r = a - b * np.floor(a / b)
            elif op == 8: r = (a == b).astype(np.float32)
            elif op == 9: r = (a != b).astype(np.float32)
            elif op == 10: r = (a < b).astype(np.float32)
            elif op == 11: r = (a <= b).astype(np.float32)
            elif op == 12: r = (a > b).astype(np.float32)
            elif op == 13: r = (a >= b).astype(np.float32)
            elif op == 14: r = ((a != 0) & (b != 0)).astype(np.float32)
            elif op == 15: r = ((a != 0) | (b != 0)).astype(np.float32)
            elif op == 16: r = ((a != 0) != (b != 0)).astype(np.float32)
            elif op == 17: r = np.arctan2(a, b)
            elif op == 18: r = (b >= a).astype(np.float32)
            elif op == 19:
                t = np.clip((f32(0.5) - a) / (b - a), 0, 1); r = t * t * (f32(3) - f32(2) * t)
            elif op == 34:
                r = (f32(0.5) * a * (one + np.tanh(f32(0.797884583) * (a + f32(0.0447149985) * a * a * a)))) * b
            elif op == 35:
                r = (a / (one + np.exp(-a))) * b
            else: r = a
        m.data[self._ew_idx("map_op2_dev", m, locs_out_handle, n)] = np.asarray(r, np.float32)

    def map_broadcast_dev(self, map_id, op, locs_src_handle, locs_scalar_handle, locs_dst_handle, n):
        """shaders/src/f32/map_broadcast.comp; OP_MUL/DIV/ADD/SUB remapped to 0..3 by the
        binding (__init__.py:2099-2104); scalar loc is NOT multiplied by pack_size."""
        self.op_count += 1
        op = {OP_MUL: 0, OP_DIV: 1, OP_ADD: 2, OP_SUB: 3}.get(op, op)
        m = self._map("map_broadcast_dev", map_id, DTYPE_F32)
        if n == 0:
            return
        v = m.data[self._ew_idx("map_broadcast_dev", m, locs_src_handle, n)]
        s = np.repeat(m.data[self._locs("map_broadcast_dev", locs_scalar_handle, n)], m.pack_size)
        with np.errstate(all="ignore"):
            r = v * s if op == 0 else v / s if op == 1 else v + s if op == 2 else v - s
        m.data[self._ew_idx("map_broadcast_dev", m, locs_dst_handle, n)] = r.astype(np.float32)

    def map_fma_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, locs_dst_handle, n_locs):
        self.op_count += 1
        m = self._map("map_fma_dev", map_id, DTYPE_F32)
        a, b, c = (m.data[self._ew_idx("map_fma_dev", m, h, n_locs)]
                   for h in (locs_a_handle, locs_b_handle, locs_c_handle))
        m.data[self._ew_idx("map_fma_dev", m, locs_dst_handle, n_locs)] = (a * b + c).astype(np.float32)

    # ------------------------------------------------------------------ norms / rope
    def _rms_rows(self, x, w, eps):
        ss = (x.astype(np.float64) ** 2).sum(axis=1)
        inv = (f32(1.0) / np.sqrt((ss / x.shape[1]).astype(np.float32) + f32(eps))).astype(np.float32)
        return (x * inv[:, None] * w).astype(np.float32)

    def _rows(self, fn, m, bases, dim):
        idx = bases[:, None] + np.arange(dim)
        if idx.size and idx.max() >= m.n:
            self._fail(fn, ERR_INVALID)
        return idx

    def map_rmsnorm_dev(self, map_id, locs_src_handle, locs_wt_handle, locs_dst_handle, n_rows, dim, eps=1e-5):
        """shaders/src/f32/map_rmsnorm.comp: y = x * (1/sqrt(sum(x^2)/dim + eps)) * w, row bases from locs."""
        self.map_rmsnorm_x_dev(map_id, map_id, locs_src_handle, locs_wt_handle, locs_dst_handle, n_rows, dim, eps)

    def map_rmsnorm_x_dev(self, map_act, map_wt, locs_src_handle, locs_wt_handle, locs_dst_handle, n_rows, dim, eps=1e-5):
        """shaders/src/f32/map_rmsnorm_x.comp:26-48."""
        self.op_count += 1
        fn = "map_rmsnorm_x_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_F32)
        if n_rows == 0:
            return
        x = ma.data[self._rows(fn, ma, self._locs(fn, locs_src_handle, n_rows), dim)]
        w = mw.data[self._rows(fn, mw, self._locs(fn, locs_wt_handle, n_rows), dim)]
        ma.data[self._rows(fn, ma, self._locs(fn, locs_dst_handle, n_rows), dim)] = self._rms_rows(x, w, eps)

    def map_rmsnorm_add_dev(self, map_id, locs_src_handle, locs_wt_handle, locs_resid_handle,
                            locs_dst_handle, n_rows, dim, eps=1e-5):
        """shaders/src/f32/map_rmsnorm_add.comp:14-44: x*inv_rms*w + r."""
        self.op_count += 1
        fn = "map_rmsnorm_add_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_rows == 0:
            return
        x = m.data[self._rows(fn, m, self._locs(fn, locs_src_handle, n_rows), dim)]
        w = m.data[self._rows(fn, m, self._locs(fn, locs_wt_handle, n_rows), dim)]
        r = m.data[self._rows(fn, m, self._locs(fn, locs_resid_handle, n_rows), dim)]
        m.data[self._rows(fn, m, self._locs(fn, locs_dst_handle, n_rows), dim)] = \
            (self._rms_rows(x, w, eps) + r).astype(np.float32)

    @staticmethod
    def _rope_cs(half, dim, pos, freq_base):
        """freq = 1/pow(base, 2i/dim); angle = float(pos)*freq (map_rope.comp:24-28).  The exponent
        2i/dim and the reciprocal are float32 operations; pow is evaluated exactly (float64) on those
        float32 inputs and rounded once, i.e. what a correctly rounded float32 pow returns."""
        e = ((2 * np.arange(half)).astype(np.float32) / f32(dim)).astype(np.float32)
        p = np.power(np.float64(f32(freq_base)), e.astype(np.float64)).astype(np.float32)
        freq = (f32(1.0) / p).astype(np.float32)
        ang = (f32(pos) * freq).astype(np.float32)
        return np.cos(ang.astype(np.float64)).astype(np.float32), np.sin(ang.astype(np.float64)).astype(np.float32)

    def map_rope_dev(self, map_id, locs_src_handle, locs_dst_handle, n_tokens, n_heads, head_dim,
                     pos_offset=0, freq_base=10000.0):
        """shaders/src/f32/map_rope.comp:11-37: half-split pairs (d, d+half); token t at pos_offset+t;
        row base = locs[token] + head*head_dim."""
        self.op_count += 1
        fn = "map_rope_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        half = head_dim // 2
        if n_tokens == 0 or n_heads == 0 or half == 0:
            return
        sb = self._locs(fn, locs_src_handle, n_tokens); db = self._locs(fn, locs_dst_handle, n_tokens)
        for t in range(n_tokens):
            c, s = self._rope_cs(half, head_dim, pos_offset + t, freq_base)
            hb = np.arange(n_heads) * head_dim
            i0 = (sb[t] + hb)[:, None] + np.arange(half)
            o0 = (db[t] + hb)[:, None] + np.arange(half)
            if max(i0.max(), o0.max()) + half >= m.n:
                self._fail(fn, ERR_INVALID)
            x0 = m.data[i0]; x1 = m.data[i0 + half]
            m.data[o0] = x0 * c - x1 * s
            m.data[o0 + half] = x0 * s + x1 * c

    def map_qk_norm_rope_x_dev(self, map_act_id, map_wt_id, locs_q_src_handle, locs_q_wt_handle,
                               locs_k_src_handle, locs_k_wt_handle, locs_qk_dst_handle,
                               q_rows, q_dim, k_rows, k_dim, pos_offset, freq_base):
        """shaders/src/f32/map_qk_norm_rope_x.comp:32-84: per-row RMSNorm with eps fixed at 1e-6,
        then half-split RoPE at pos_offset; Q rows then K rows written contiguously from
        locs_qk_dst[0]."""
        self.op_count += 1
        fn = "map_qk_norm_rope_x_dev"
        ma = self._map(fn, map_act_id, DTYPE_F32); mw = self._map(fn, map_wt_id, DTYPE_F32)
        dst = int(self._locs(fn, locs_qk_dst_handle, 1)[0])
        outs = []
        for rows, dim, sh, wh in ((q_rows, q_dim, locs_q_src_handle, locs_q_wt_handle),
                                  (k_rows, k_dim, locs_k_src_handle, locs_k_wt_handle)):
            half = dim // 2
            if rows == 0 or half == 0:
                outs.append(np.zeros(0, np.float32)); continue
            x = ma.data[self._rows(fn, ma, self._locs(fn, sh, rows), dim)]
            w = mw.data[self._rows(fn, mw, self._locs(fn, wh, rows), dim)]
            y = self._rms_rows(x, w, 1e-6)
            c, s = self._rope_cs(half, dim, pos_offset, freq_base)
            y0, y1 = y[:, :half], y[:, half:2 * half]
            o = y.copy()
            o[:, :half] = y0 * c - y1 * s
            o[:, half:2 * half] = y0 * s + y1 * c
            outs.append(o.reshape(-1))
        flat = np.concatenate(outs).astype(np.float32)
        self._chk(fn, ma, dst, dst + flat.size)
        ma.data[dst:dst + flat.size] = flat

    # ------------------------------------------------------------------ KV append
    def map_row_copy_offset_dev(self, map_id, copy_spec_handle, src_base_handle, dst_row_offset, n_copies, row_size):
        """shaders/src/f32/map_row_copy.comp:13-24: spec = [src_row, dst_row] pairs;
        src = src_base[0] + src_row*row_size, dst = (dst_row + dst_row_offset)*row_size."""
        self.op_count += 1
        fn = "map_row_copy_offset_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_copies == 0 or row_size == 0:
            return
        spec = self._locs(fn, copy_spec_handle, 2 * n_copies).reshape(n_copies, 2)
        base = int(self._locs(fn, src_base_handle, 1)[0])
        src = (base + spec[:, 0] * row_size)[:, None] + np.arange(row_size)
        dst = ((spec[:, 1] + dst_row_offset) * row_size)[:, None] + np.arange(row_size)
        if max(src.max(), dst.max()) >= m.n:
            self._fail(fn, ERR_INVALID)
        m.data[dst] = self._kv_round(map_id, dst, m.data[src].copy())

    def map_row_copy_dev(self, map_id, copy_spec_handle, src_base_handle, n_copies, row_size):
        self.map_row_copy_offset_dev(map_id, copy_spec_handle, src_base_handle, 0, n_copies, row_size)

    def attn_causal_rows_dev(self, map_id, q_handles, locs_k_handle, locs_scores_handle, locs_v_handle, out_handles,
                             head_dim, n_keys0, n_heads, value_dim, scale, softcap=0.0):
        """Extension shared with the HIP library (no counterpart in the reference): the (scores, softmax . V)
        pair of m consecutive tokens over one growing cache, token t over n_keys0 + t keys."""
        for t, (qh, oh) in enumerate(zip(q_handles, out_handles)):
            self.map_matmul_t_dev(map_id, qh, locs_k_handle, locs_scores_handle, 1, head_dim, n_keys0 + t, n_heads)
            self.map_attn_softmax_value_dev(map_id, locs_scores_handle, locs_v_handle, oh, n_heads, n_keys0 + t,
                                            value_dim, scale, softcap)

    def qk_norm_rope_rows_dev(self, map_act, map_wt, q_src_handles, locs_q_wt_handle, k_src_handles, locs_k_wt_handle,
                              dst_handles, q_rows, q_dim, k_rows, k_dim, pos0, freq_base):
        """Extension shared with the HIP library: map_qk_norm_rope_x_dev of m consecutive tokens, token t at pos0 + t."""
        for t, (qh, kh, dh) in enumerate(zip(q_src_handles, k_src_handles, dst_handles)):
            self.map_qk_norm_rope_x_dev(map_act, map_wt, qh, locs_q_wt_handle, kh, locs_k_wt_handle, dh, q_rows, q_dim,
                                        k_rows, k_dim, pos0 + t, freq_base)

    def kv_cache_fp16(self, map_id, start, count):
        """Extension shared with the HIP library: elements [start, start+count) of a float32
        map are a KV cache kept in fp16.  Values copied or scattered into that range are rounded
        to fp16 (round-to-nearest-even), as is whatever the range holds when it is declared; reads
        see the rounded values."""
        m = self._map("adamah_kv_cache_fp16", map_id, DTYPE_F32)
        if count == 0 or start + count > m.n:
            self._fail("adamah_kv_cache_fp16", ERR_INVALID)
        if not hasattr(self, "_kv_fp16"):
            self._kv_fp16 = {}
        self._kv_fp16[map_id] = (int(start), int(count))
        m.data[start:start + count] = m.data[start:start + count].astype(np.float16).astype(np.float32)

    # ------------------------------------------------------------------ matmuls
    def _mm(self, fn, ma, wfun, la, lb, lc, M, K, N, n_ops, transposed=True):
        for op in range(n_ops):
            a, b, c = int(la[op]), int(lb[op]), int(lc[op])
            self._chk(fn, ma, a, a + M * K); self._chk(fn, ma, c, c + M * N)
            A = ma.data[a:a + M * K].reshape(M, K).astype(np.float64)
            W = wfun(b, N * K).astype(np.float64)
            W = W.reshape(N, K).T if transposed else W.reshape(K, N)
            with np.errstate(all="ignore"):
                ma.data[c:c + M * N] = (A @ W).astype(np.float32).reshape(-1)

    def map_matmul_t_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """shaders/src/f32/map_matmul_t.comp: C[M,N] = A[M,K] . B[N,K]^T per op, bases locs[op]."""
        self.op_count += 1
        fn = "map_matmul_t_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_ops == 0 or M == 0 or N == 0:
            return
        def w(b, cnt):
            self._chk(fn, m, b, b + cnt); return m.data[b:b + cnt]
        self._mm(fn, m, w, self._locs(fn, locs_a_handle, n_ops), self._locs(fn, locs_b_handle, n_ops),
                 self._locs(fn, locs_c_handle, n_ops), M, K, N, n_ops, True)

    def map_matmul_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """shaders/src/f32/map_matmul.comp: C = A[M,K] . B[K,N]."""
        self.op_count += 1
        fn = "map_matmul_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_ops == 0 or M == 0 or N == 0:
            return
        def w(b, cnt):
            self._chk(fn, m, b, b + cnt); return m.data[b:b + cnt]
        self._mm(fn, m, w, self._locs(fn, locs_a_handle, n_ops), self._locs(fn, locs_b_handle, n_ops),
                 self._locs(fn, locs_c_handle, n_ops), M, K, N, n_ops, False)

    def _xq(self, fn, map_act, map_wt, dtype, la_h, lb_h, lc_h, M, K, N, n_ops, transposed):
        self.op_count += 1
        ma = self._map(fn, map_act, DTYPE_F32)
        mw = self._map(fn, map_wt)
        if n_ops == 0 or N == 0:
            return
        if mw.scale is None or (dtype is not None and mw.dtype != dtype):
            self._fail(fn, ERR_INVALID)
        def w(b, cnt):
            self._chk(fn, mw, b, b + cnt); return mw.deq_range(b, cnt)
        self._mm(fn, ma, w, self._locs(fn, la_h, n_ops), self._locs(fn, lb_h, n_ops),
                 self._locs(fn, lc_h, n_ops), M, K, N, n_ops, transposed)

    def map_matmul_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """adamah.c:8693-8803; shaders/src/f32/map_matvec_t_xq4.comp:57-135 (M==1, n_ops==1) and
        map_matmul_t_xq4.comp:33-73: y[n] = sum_k x[k] * deq(b + n*K + k)."""
        self._xq("map_matmul_t_xq4_dev", map_act, map_wt, DTYPE_Q4, locs_a_handle, locs_b_handle,
                 locs_c_handle, M, K, N, n_ops, True)

    def map_matmul_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """adamah.c:9834-9910; shaders/src/f32/map_matvec_t_xq8.comp:55-132."""
        self._xq("map_matmul_t_xq8_dev", map_act, map_wt, DTYPE_Q8, locs_a_handle, locs_b_handle,
                 locs_c_handle, M, K, N, n_ops, True)

    def map_matmul_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """shaders/src/f32/map_matmul_xq4.comp: C = A . B with B[K,N] row-major in the Q4 map."""
        self._xq("map_matmul_xq4_dev", map_act, map_wt, DTYPE_Q4, locs_a_handle, locs_b_handle,
                 locs_c_handle, M, K, N, n_ops, False)

    def map_matmul_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xq("map_matmul_xq8_dev", map_act, map_wt, DTYPE_Q8, locs_a_handle, locs_b_handle,
                 locs_c_handle, M, K, N, n_ops, False)

    def map_matmul_t_x_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self.op_count += 1
        fn = "map_matmul_t_x_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_F32)
        def w(b, cnt):
            self._chk(fn, mw, b, b + cnt); return mw.data[b:b + cnt]
        if n_ops and N:
            self._mm(fn, ma, w, self._locs(fn, locs_a_handle, n_ops), self._locs(fn, locs_b_handle, n_ops),
                     self._locs(fn, locs_c_handle, n_ops), M, K, N, n_ops, True)

    def map_matmul_x_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        """shaders/src/f32/map_matmul_x.comp:16-32: C[M,N] = A[M,K] . B[K,N], A and C in map_act, B row-major
        in the f32 map map_wt, bases locs[op]."""
        self.op_count += 1
        fn = "map_matmul_x_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_F32)
        def w(b, cnt):
            self._chk(fn, mw, b, b + cnt); return mw.data[b:b + cnt]
        if n_ops and N:
            self._mm(fn, ma, w, self._locs(fn, locs_a_handle, n_ops), self._locs(fn, locs_b_handle, n_ops),
                     self._locs(fn, locs_c_handle, n_ops), M, K, N, n_ops, False)

    def map_row_gather_xq8_dev(self, map_act, map_wt, src_base, dst_base, row_idx, row_size, scale=1.0):
        """shaders/src/f32/map_row_gather_xq8.comp: dst[e] = deq(src_base + row*row_size + e) * scale."""
        self.op_count += 1
        fn = "map_row_gather_xq8_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_Q8)
        s = src_base + row_idx * row_size
        self._chk(fn, mw, s, s + row_size); self._chk(fn, ma, dst_base, dst_base + row_size)
        ma.data[dst_base:dst_base + row_size] = mw.deq(np.arange(s, s + row_size)) * f32(scale)

    # ------------------------------------------------------------------ softmax / attention
    @staticmethod
    def _prep(v, scale, cap):
        v = (v * f32(scale)).astype(np.float32)
        if cap > 0.0:
            v = (np.tanh(v / f32(cap)) * f32(cap)).astype(np.float32)
        return v

    @staticmethod
    def _softmax(v):
        e = np.exp((v - v.max()).astype(np.float32)).astype(np.float32)
        return (e * (f32(1.0) / f32(e.astype(np.float64).sum()))).astype(np.float32)

    def map_softmax_abs_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows):
        """shaders/src/f32/map_softmax_abs.comp: row bases are absolute element offsets."""
        self.map_attn_softmax_abs_dev(map_id, locs_in_handle, locs_out_handle, row_size, n_rows, 1.0, 0.0)

    def map_attn_softmax_abs_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows, scale, cap):
        """shaders/src/f32/map_attn_softmax_abs.comp: softmax(cap*tanh(s*scale/cap)) (cap only if >0)."""
        self.op_count += 1
        fn = "map_attn_softmax_abs_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_rows == 0 or row_size == 0:
            return
        sb = self._locs(fn, locs_in_handle, n_rows); db = self._locs(fn, locs_out_handle, n_rows)
        for r in range(n_rows):
            self._chk(fn, m, sb[r], sb[r] + row_size); self._chk(fn, m, db[r], db[r] + row_size)
            m.data[db[r]:db[r] + row_size] = self._softmax(self._prep(m.data[sb[r]:sb[r] + row_size], scale, cap))

    def map_softmax_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows):
        """shaders/src/f32/map_softmax.comp: row base = locs[ri] * row_size."""
        self.op_count += 1
        fn = "map_softmax_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        sb = self._locs(fn, locs_in_handle, n_rows) * row_size; db = self._locs(fn, locs_out_handle, n_rows) * row_size
        for r in range(n_rows):
            self._chk(fn, m, sb[r], sb[r] + row_size); self._chk(fn, m, db[r], db[r] + row_size)
            m.data[db[r]:db[r] + row_size] = self._softmax(m.data[sb[r]:sb[r] + row_size])

    def map_attn_softmax_value_dev(self, map_id, locs_scores_handle, locs_values_handle, locs_out_handle,
                                   n_ops, row_size, value_dim, scale, cap):
        """shaders/src/f32/map_attn_softmax_value.comp:39-89: per op, p = softmax(prep(scores)),
        out[d] = sum_t p[t] * V[t*value_dim + d].  The shader's 2048-row bail-out is a shared-
        memory limit of that implementation, not part of the op; any row_size is evaluated."""
        self.op_count += 1
        fn = "map_attn_softmax_value_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_ops == 0 or row_size == 0 or value_dim == 0:
            return
        sb = self._locs(fn, locs_scores_handle, n_ops); vb = self._locs(fn, locs_values_handle, n_ops)
        ob = self._locs(fn, locs_out_handle, n_ops)
        for op in range(n_ops):
            self._chk(fn, m, sb[op], sb[op] + row_size)
            self._chk(fn, m, vb[op], vb[op] + row_size * value_dim)
            self._chk(fn, m, ob[op], ob[op] + value_dim)
            p = self._softmax(self._prep(m.data[sb[op]:sb[op] + row_size], scale, cap))
            V = m.data[vb[op]:vb[op] + row_size * value_dim].reshape(row_size, value_dim)
            m.data[ob[op]:ob[op] + value_dim] = (p.astype(np.float64) @ V.astype(np.float64)).astype(np.float32)

    def map_layernorm_dev(self, map_id, locs_src_handle, locs_dst_handle, locs_gamma_handle, locs_beta_handle,
                          dim, eps=1e-5, n_rows=0):
        """shaders/src/f32/map_layernorm.comp: src/dst bases = locs*dim, gamma/beta bases absolute."""
        self.op_count += 1
        fn = "map_layernorm_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        for r in range(n_rows):
            sb = int(self._locs(fn, locs_src_handle, n_rows)[r]) * dim
            db = int(self._locs(fn, locs_dst_handle, n_rows)[r]) * dim
            gb = int(self._locs(fn, locs_gamma_handle, n_rows)[r]); bb = int(self._locs(fn, locs_beta_handle, n_rows)[r])
            x = m.data[sb:sb + dim].astype(np.float64)
            mean = f32(x.sum() / dim)
            var = f32(((x - mean) ** 2).sum() / dim)
            inv = f32(1.0) / np.sqrt(var + f32(eps))
            m.data[db:db + dim] = ((m.data[sb:sb + dim] - mean) * inv * m.data[gb:gb + dim] + m.data[bb:bb + dim])

    def map_reduce_dev(self, map_id, op, locs_src_handle, locs_dst_handle, n):
        """shaders/src/f32/map_reduce.comp: per loc, reduce the pack (0 sum, 1 max, 2 min)."""
        self.op_count += 1
        fn = "map_reduce_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        src = self._locs(fn, locs_src_handle, n) * m.pack_size; dst = self._locs(fn, locs_dst_handle, n)
        for i in range(n):
            x = m.data[src[i]:src[i] + m.pack_size]
            m.data[dst[i]] = f32(x.astype(np.float64).sum()) if op == 0 else x.max() if op == 1 else x.min()

    # ------------------------------------------------------------------ argmax tail
    @staticmethod
    def _argbest(vals, idxs):
        """strict > or (== and lower index); reference `better()` in map_argmax.comp:15-19."""
        best_v, best_i = None, 0xFFFFFFFF
        for v, i in zip(vals, idxs):
            if best_i == 0xFFFFFFFF or (i != 0xFFFFFFFF and (v > best_v or (v == best_v and i < best_i))):
                best_v, best_i = v, i
        return best_v, best_i

    def map_argmax_dev(self, map_id, locs_src_handle, locs_dst_handle, n):
        """shaders/src/f32/map_argmax.comp: NaN -> -FLT_MAX, ties -> lower index, result stored as
        float(index) at locs_dst[0]; n == 0 -> 0."""
        self.op_count += 1
        fn = "map_argmax_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        dst = int(self._locs(fn, locs_dst_handle, 1)[0])
        if n == 0:
            m.data[dst] = 0.0; return
        v = m.data[self._locs(fn, locs_src_handle, n)].copy()
        v[np.isnan(v)] = NEG_MAX
        best = v.max()
        m.data[dst] = f32(int(np.flatnonzero(v == best)[0]))

    # ---- sampling tail ----------------------------------------------------------------------
    def map_topk_dev(self, map_id, locs_src_handle, locs_idx_dst_handle, locs_val_dst_handle, n, k):
        """shaders/src/f32/map_topk.comp:38-90 (dispatch adamah.c:6978-7093): k rounds of the best value not
        yet chosen; NaN -> -FLT_MAX, ties -> lower index; rounds past n store index 0 and -FLT_MAX."""
        self.op_count += 1
        fn = "map_topk_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n == 0 or k == 0:
            return
        if k > 64:
            self._fail(fn, ERR_INVALID)
        v = m.data[self._locs(fn, locs_src_handle, n)].copy()
        v[np.isnan(v)] = NEG_MAX
        li = self._locs(fn, locs_idx_dst_handle, k); lv = self._locs(fn, locs_val_dst_handle, k)
        taken = np.zeros(n, bool)
        for o in range(k):
            if taken.all():
                m.data[li[o]] = 0.0; m.data[lv[o]] = NEG_MAX
                continue
            cand = np.where(taken, -np.inf, v.astype(np.float64))
            w = int(np.flatnonzero(cand == cand.max())[0])
            taken[w] = True
            m.data[li[o]] = f32(w); m.data[lv[o]] = v[w]

    def map_topp_dev(self, map_id, locs_src_handle, locs_dst_handle, n, temperature, top_p):
        """shaders/src/f32/map_topp.comp:23-95 (dispatch adamah.c:7095-7208), float32 and sequential like
        the shader's single lane: softmax(logit / max(T, 1e-6)) in list order, cut after the first prefix
        whose mass reaches top_p, renormalised over the prefix."""
        self.op_count += 1
        fn = "map_topp_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n == 0:
            return
        if n > 64:
            self._fail(fn, ERR_INVALID)
        lg = m.data[self._locs(fn, locs_src_handle, n)].copy()
        ld = self._locs(fn, locs_dst_handle, n)
        lg[~np.isfinite(lg)] = NEG_MAX
        temp = max(f32(temperature), f32(1e-6)); keep_p = min(max(f32(top_p), f32(0.0)), f32(1.0))
        mx = lg.max()
        if mx == NEG_MAX:
            m.data[ld] = 0.0; return
        pr = np.zeros(n, np.float32); tot = f32(0.0)
        for i in range(n):
            if lg[i] == NEG_MAX:
                continue
            pr[i] = np.exp(f32(f32(lg[i] - mx) / temp), dtype=np.float32)
            tot = f32(tot + pr[i])
        if tot <= 0:
            out = np.zeros(n, np.float32); out[0] = 1.0
            m.data[ld] = out; return
        pr = (pr / tot).astype(np.float32)
        keep, cs = 0, f32(0.0)
        for i in range(n):
            cs = f32(cs + pr[i]); keep = i + 1
            if keep_p >= f32(0.999999) or cs >= keep_p:
                break
        ks = f32(0.0)
        for i in range(keep):
            ks = f32(ks + pr[i])
        if ks <= 0:
            ks = f32(1.0)
        out = np.zeros(n, np.float32)
        out[:keep] = (pr[:keep] / ks).astype(np.float32)
        m.data[ld] = out

    def map_resolve_idx_dev(self, map_id, base_locs_handle, sel_locs_handle, dst_locs_handle, n):
        """shaders/src/f32/map_resolve_idx.comp:13-26: dst[i] = data[base + uint(data[sel[i]])]; negative or
        non-finite selectors and results count as 0."""
        self.op_count += 1
        fn = "map_resolve_idx_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n == 0:
            return
        base = int(self._locs(fn, base_locs_handle, 1)[0])
        sel = self._locs(fn, sel_locs_handle, n); dst = self._locs(fn, dst_locs_handle, n)
        for i in range(n):
            sv = m.data[sel[i]]
            if not np.isfinite(sv) or sv < 0:
                sv = f32(0.0)
            t = m.data[base + int(sv)]
            if not np.isfinite(t) or t < 0:
                t = f32(0.0)
            m.data[dst[i]] = t

    def map_sample_categorical_dev(self, map_id, locs_idx_handle, locs_prob_handle, rand_loc_handle, dst_loc_handle, n):
        """shaders/src/f32/map_sample_categorical.comp:14-50: inverse-CDF draw, float32 running sums in list
        order, r clamped to [0, 0.99999994], zero total -> first index."""
        self.op_count += 1
        fn = "map_sample_categorical_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n == 0:
            return
        if n > 64:
            self._fail(fn, ERR_INVALID)
        li = self._locs(fn, locs_idx_handle, n); lp = self._locs(fn, locs_prob_handle, n)
        r_loc = int(self._locs(fn, rand_loc_handle, 1)[0]); d_loc = int(self._locs(fn, dst_loc_handle, 1)[0])
        p = m.data[lp].copy()
        p[~np.isfinite(p) | (p < 0)] = 0.0
        tot = f32(0.0)
        for x in p:
            tot = f32(tot + x)
        if not tot > 0:
            m.data[d_loc] = m.data[li[0]]; return
        r = m.data[r_loc]
        if not np.isfinite(r):
            r = f32(0.0)
        r = min(max(r, f32(0.0)), f32(0.99999994))
        target = f32(r * tot)
        acc, chosen = f32(0.0), n - 1
        for i in range(n):
            acc = f32(acc + p[i])
            if target < acc:
                chosen = i; break
        m.data[d_loc] = m.data[li[chosen]]

    def map_repeat_penalty_dev(self, map_id, locs_src_handle, token_ids_handle, n_ids, penalty):
        """shaders/src/f32/map_repeat_penalty.comp:13-21: logit / penalty when positive, * penalty otherwise.
        The callers pass distinct ids (adam/models/engine.py:2052); with a repeated id the shader's
        invocations race, so the definition used here is: every distinct id once."""
        self.op_count += 1
        fn = "map_repeat_penalty_dev"
        m = self._map(fn, map_id, DTYPE_F32)
        if n_ids == 0:
            return
        if n_ids > 64:
            self._fail(fn, ERR_INVALID)
        toks = self._locs(fn, token_ids_handle, n_ids)
        for t in dict.fromkeys(int(x) for x in toks):
            loc = int(self._locs(fn, locs_src_handle, int(t) + 1)[int(t)])
            v = m.data[loc]
            m.data[loc] = f32(v / f32(penalty)) if v > 0 else f32(v * f32(penalty))

    def _matvec_argmax(self, fn, dtype, map_act, map_wt, la_h, lb_h, idx_h, val_h, dst_h, K, N, rpg):
        """adamah.c:9558-9721; pass 1 shaders/src/f32/map_matvec_argmax_t_xq4.comp:66-158 (per group of
        rows_per_group rows: best (value,row)), pass 2 map_argmax_pairs.comp:34-67.  Row values are
        NOT NaN-filtered in pass 1 (plain `better`), partials land at locs_idx/val[group]."""
        self.op_count += 1
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, dtype)
        if N == 0:
            return
        if rpg == 0 or mw.scale is None:
            self._fail(fn, ERR_INVALID)
        ng = (N + rpg - 1) // rpg
        il = self._locs(fn, idx_h, ng); vl = self._locs(fn, val_h, ng)
        dst = int(self._locs(fn, dst_h, 1)[0])
        a = int(self._locs(fn, la_h, 1)[0]); b = int(self._locs(fn, lb_h, 1)[0])
        self._chk(fn, ma, a, a + K); self._chk(fn, mw, b, b + N * K)
        y = (mw.deq_range(b, N * K).reshape(N, K).astype(np.float64) @ ma.data[a:a + K].astype(np.float64)).astype(np.float32)
        gv = np.empty(ng, np.float32); gi = np.empty(ng, np.int64)
        for g in range(ng):
            seg = y[g * rpg:(g + 1) * rpg]
            v, i = self._argbest(seg, range(g * rpg, g * rpg + seg.size))
            gv[g], gi[g] = v, i
        ma.data[il] = gi.astype(np.float32); ma.data[vl] = gv
        _, tok = self._argbest(gv, gi)
        ma.data[dst] = f32(0 if tok == 0xFFFFFFFF else tok)
        self.last_logits = y

    def map_matvec_argmax_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_idx_tmp_handle,
                                    locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group):
        self._matvec_argmax("map_matvec_argmax_t_xq4_dev", DTYPE_Q4, map_act, map_wt, locs_a_handle, locs_b_handle,
                            locs_idx_tmp_handle, locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group)

    def map_matvec_argmax_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_idx_tmp_handle,
                                    locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group):
        self._matvec_argmax("map_matvec_argmax_t_xq8_dev", DTYPE_Q8, map_act, map_wt, locs_a_handle, locs_b_handle,
                            locs_idx_tmp_handle, locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group)

    # ---- fused GEMV + partial top-k, shortlist rerank -----------------------------------------
    def _matvec_topk(self, fn, dtype, map_act, map_wt, la_h, lb_h, pen_h, idx_h, val_h, K, N, k, n_pen, rp, rpg):
        """shaders/src/f32/map_matvec_topk_t_xq4.comp:108-208 (Q8 twin map_matvec_topk_t_xq8.comp), dispatch
        adamah.c:9727-9830 / :9911-10016: per group of rows_per_group rows, logits -> repeat penalty on the
        rows listed in penalty_ids (value > 0 ? value / p : value * p, membership test, so once per row) ->
        list of k = min(k, 64) entries sorted by (value descending, row ascending); slots the group cannot
        fill hold index 0 and -FLT_MAX.  A NaN logit ranks as -FLT_MAX (the shader's insertion would leave it
        wherever it was first put)."""
        self.op_count += 1
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, dtype)
        if N == 0 or k == 0:
            return
        if k > 64 or n_pen > 64 or rpg == 0 or mw.scale is None:
            self._fail(fn, ERR_INVALID)
        ng = (N + rpg - 1) // rpg
        il = self._locs(fn, idx_h, ng * k); vl = self._locs(fn, val_h, ng * k)
        self._h(fn, pen_h)
        pen = set(int(t) for t in self._locs(fn, pen_h, n_pen)) if n_pen else set()
        a = int(self._locs(fn, la_h, 1)[0]); b = int(self._locs(fn, lb_h, 1)[0])
        self._chk(fn, ma, a, a + K); self._chk(fn, mw, b, b + N * K)
        y = (mw.deq_range(b, N * K).reshape(N, K).astype(np.float64) @ ma.data[a:a + K].astype(np.float64)).astype(np.float32)
        rp = f32(rp)
        y[np.isnan(y)] = NEG_MAX
        for r in pen:
            if r < N:
                y[r] = y[r] / rp if y[r] > 0 else y[r] * rp
        for g in range(ng):
            rows = np.arange(g * rpg, min(N, (g + 1) * rpg))
            order = sorted(rows.tolist(), key=lambda r: (-float(y[r]), r))[:k]
            for t in range(k):
                if t < len(order):
                    ma.data[il[g * k + t]] = f32(order[t]); ma.data[vl[g * k + t]] = y[order[t]]
                else:
                    ma.data[il[g * k + t]] = 0.0; ma.data[vl[g * k + t]] = NEG_MAX
        self.last_logits = y

    def map_matvec_topk_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                  locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0, repeat_penalty=1.0):
        self._matvec_topk("map_matvec_topk_t_xq4_dev", DTYPE_Q4, map_act, map_wt, locs_a_handle, locs_b_handle,
                          penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty,
                          repeat_penalty, 256)

    def map_matvec_topk_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                  locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0, repeat_penalty=1.0):
        self._matvec_topk("map_matvec_topk_t_xq8_dev", DTYPE_Q8, map_act, map_wt, locs_a_handle, locs_b_handle,
                          penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty,
                          repeat_penalty, 256)

    def map_matvec_topk_t_xq4_ex_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                     locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0,
                                     repeat_penalty=1.0, rows_per_group=256):
        self._matvec_topk("map_matvec_topk_t_xq4_ex_dev", DTYPE_Q4, map_act, map_wt, locs_a_handle, locs_b_handle,
                          penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty,
                          repeat_penalty, rows_per_group)

    def map_matvec_topk_t_xq8_ex_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                     locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0,
                                     repeat_penalty=1.0, rows_per_group=256):
        self._matvec_topk("map_matvec_topk_t_xq8_ex_dev", DTYPE_Q8, map_act, map_wt, locs_a_handle, locs_b_handle,
                          penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty,
                          repeat_penalty, rows_per_group)

    def map_matvec_rerank_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, partial_idx_base_handle,
                                    sel_locs_handle, penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle,
                                    K, n_ids, n_penalty=0, repeat_penalty=1.0):
        """shaders/src/f32/map_matvec_rerank_t_xq8.comp:43-82 (dispatch adamah.c:10018-10110): for each of the
        n_ids <= 64 shortlist slots, token = uint(act[partial_base + uint(act[sel_locs[i]])]), value = exact
        logit of that row (with the repeat penalty when the token is listed); stores float(token), value."""
        self.op_count += 1
        fn = "map_matvec_rerank_t_xq8_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_Q8)
        if n_ids == 0:
            return
        if n_ids > 64 or n_penalty > 64 or mw.scale is None:
            self._fail(fn, ERR_INVALID)
        a = int(self._locs(fn, locs_a_handle, 1)[0]); b = int(self._locs(fn, locs_b_handle, 1)[0])
        pb = int(self._locs(fn, partial_idx_base_handle, 1)[0])
        sel = self._locs(fn, sel_locs_handle, n_ids)
        il = self._locs(fn, locs_idx_dst_handle, n_ids); vl = self._locs(fn, locs_val_dst_handle, n_ids)
        self._h(fn, penalty_ids_handle)
        pen = set(int(t) for t in self._locs(fn, penalty_ids_handle, n_penalty)) if n_penalty else set()
        self._chk(fn, ma, a, a + K)
        x = ma.data[a:a + K].astype(np.float64)
        rp = f32(repeat_penalty)
        for i in range(n_ids):
            tok = int(ma.data[pb + int(ma.data[sel[i]])])
            self._chk(fn, mw, b + tok * K, b + (tok + 1) * K)
            v = f32(mw.deq_range(b + tok * K, K).astype(np.float64) @ x)
            if tok in pen:
                v = v / rp if v > 0 else v * rp
            ma.data[il[i]] = f32(tok); ma.data[vl[i]] = v

    # ---- projections that share one activation vector -----------------------------------------
    def _fused_proj(self, fn, dtype, map_act, map_wt, la_h, parts, K):
        """adamah.c:8826-8951 (and the Q8 / gate-up twins): every handle must exist, nothing to do when all
        row counts are zero; each projection is the M = 1 transposed matmul of its own matrix
        (shaders/src/f32/map_fused_qkv_t_xq4.comp, map_fused_gateup_t_xq4.comp)."""
        self.op_count += 1
        self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt)
        if not any(n for _, _, n in parts):
            return
        if mw.scale is None:
            self._fail(fn, ERR_INVALID)
        self._h(fn, la_h)
        for hb, hc, _ in parts:
            self._h(fn, hb); self._h(fn, hc)
        for hb, hc, n in parts:
            if n:
                self.op_count -= 1
                self._xq(fn, map_act, map_wt, dtype, la_h, hb, hc, 1, K, n, 1, True)

    def map_fused_qkv_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle, locs_bv_handle,
                                locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v):
        self._fused_proj("map_fused_qkv_t_xq4_dev", DTYPE_Q4, map_act, map_wt, locs_a_handle,
                         [(locs_bq_handle, locs_cq_handle, N_q), (locs_bk_handle, locs_ck_handle, N_k),
                          (locs_bv_handle, locs_cv_handle, N_v)], K)

    def map_fused_qkv_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle, locs_bv_handle,
                                locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v):
        self._fused_proj("map_fused_qkv_t_xq8_dev", DTYPE_Q8, map_act, map_wt, locs_a_handle,
                         [(locs_bq_handle, locs_cq_handle, N_q), (locs_bk_handle, locs_ck_handle, N_k),
                          (locs_bv_handle, locs_cv_handle, N_v)], K)

    def map_fused_gateup_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                   locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up):
        self._fused_proj("map_fused_gateup_t_xq4_dev", DTYPE_Q4, map_act, map_wt, locs_a_handle,
                         [(locs_b_gate_handle, locs_c_gate_handle, N_gate), (locs_b_up_handle, locs_c_up_handle, N_up)], K)

    def map_fused_gateup_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                   locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up):
        self._fused_proj("map_fused_gateup_t_xq8_dev", DTYPE_Q8, map_act, map_wt, locs_a_handle,
                         [(locs_b_gate_handle, locs_c_gate_handle, N_gate), (locs_b_up_handle, locs_c_up_handle, N_up)], K)

    def map_fused_gateup_act_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                       locs_c_out_handle, K, N_ff):
        """shaders/src/f32/map_fused_gateup_act_t_xq8.comp:62-160 (dispatch adamah.c:9353-9466):
        out[i] = silu(x . Wgate[i]) * (x . Wup[i]) with silu(v) = v / (1 + exp(-v)), float32."""
        self.op_count += 1
        fn = "map_fused_gateup_act_t_xq8_dev"
        ma = self._map(fn, map_act, DTYPE_F32); mw = self._map(fn, map_wt, DTYPE_Q8)
        if N_ff == 0:
            return
        if mw.scale is None:
            self._fail(fn, ERR_INVALID)
        a = int(self._locs(fn, locs_a_handle, 1)[0]); bg = int(self._locs(fn, locs_b_gate_handle, 1)[0])
        bu = int(self._locs(fn, locs_b_up_handle, 1)[0]); co = int(self._locs(fn, locs_c_out_handle, 1)[0])
        self._chk(fn, ma, a, a + K); self._chk(fn, mw, bg, bg + N_ff * K); self._chk(fn, mw, bu, bu + N_ff * K)
        self._chk(fn, ma, co, co + N_ff)
        x = ma.data[a:a + K].astype(np.float64)
        gate = (mw.deq_range(bg, N_ff * K).reshape(N_ff, K).astype(np.float64) @ x).astype(np.float32)
        upv = (mw.deq_range(bu, N_ff * K).reshape(N_ff, K).astype(np.float64) @ x).astype(np.float32)
        with np.errstate(over="ignore"):
            ma.data[co:co + N_ff] = (gate / (f32(1.0) + np.exp(-gate))) * upv


def init(cache_mb=None, cold_cache_mb=None):
    return NumpyAdamah()
