"""ctypes binding for libadamah_hip.so with the reference binding's op surface.

Method names, positional argument order, return shapes and error strings are those of
`class Adamah` in the reference (adamah-MAIN/adamah/__init__.py:478-2897), so code written
against that class -- the model engine, the decode-primitive tests -- runs on this one.  The
Python-order / C-order quirks of the reference are kept: `(row_size, n_rows)` swapped for the
softmax family (:1552-1594), `(dim, eps, n_rows)` for layernorm (:1645-1659), and the
OP_MUL/DIV/ADD/SUB -> 0..3 remap for broadcast (:2099-2104).

There is no CPU fallback: if the shared library is missing or lacks a symbol, construction
raises.
"""
import ctypes
import os
from contextlib import contextmanager

import numpy as np

__version__ = "0.1.0"

u32, u64, f32c, i32 = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_float, ctypes.c_int
vp = ctypes.c_void_p
pu32 = ctypes.POINTER(ctypes.c_uint32)
pu64 = ctypes.POINTER(ctypes.c_uint64)
pf32 = ctypes.POINTER(ctypes.c_float)

FUSION_SCHEDULER_LEGACY, FUSION_SCHEDULER_ALIAS_SAFE, FUSION_SCHEDULER_LEVEL_BATCHED = 0, 1, 2
_SCHED_NAMES = {0: "legacy", 1: "alias_safe", 2: "level_batched"}

DECODE_RUNTIME_POS = 0xFFFFFFFE
DECODE_RUNTIME_SEQ_LEN = 0xFFFFFFFD
(DECODE_OP_NOP, DECODE_OP_FUSION_FLUSH, DECODE_OP_FUSION_ENABLE) = (0, 1, 2)
(DECODE_OP_OP1, DECODE_OP_OP2, DECODE_OP_RMSNORM, DECODE_OP_RMSNORM_X, DECODE_OP_RMSNORM_ADD,
 DECODE_OP_ROPE, DECODE_OP_MATMUL_T, DECODE_OP_MATMUL_T_X, DECODE_OP_MATMUL_X, DECODE_OP_MATMUL_T_XQ4,
 DECODE_OP_MATMUL_XQ4, DECODE_OP_MATMUL_T_XQ8, DECODE_OP_MATMUL_XQ8, DECODE_OP_QK_NORM_ROPE_X,
 DECODE_OP_ROW_COPY_OFFSET, DECODE_OP_ATTN_SOFTMAX_VALUE) = range(10, 26)
(DECODE_OP_FUSED_QKV_T_XQ4, DECODE_OP_FUSED_GATEUP_T_XQ4, DECODE_OP_FUSED_QKV_T_XQ8, DECODE_OP_FUSED_GATEUP_T_XQ8,
 DECODE_OP_FUSED_GATEUP_ACT_T_XQ8) = range(26, 31)

(OP_NEG, OP_ABS, OP_SQRT, OP_EXP, OP_LOG, OP_TANH, OP_RELU, OP_GELU, OP_SIN, OP_COS, OP_TAN, OP_ASIN,
 OP_ACOS, OP_ATAN, OP_SINH, OP_COSH, OP_SIGMOID, OP_SWISH, OP_MISH, OP_SELU, OP_ELU, OP_LEAKY_RELU,
 OP_CEIL, OP_FLOOR, OP_ROUND, OP_SIGN, OP_RECIPROCAL, OP_SQUARE, OP_CUBE, OP_SOFTPLUS, OP_HARDSIGMOID,
 OP_HARDSWISH, OP_EXPM1, OP_LOG1P) = range(34)
(OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_POW, OP_MIN, OP_MAX, OP_MOD, OP_EQ, OP_NE, OP_LT, OP_LE, OP_GT,
 OP_GE, OP_AND, OP_OR, OP_XOR, OP_ATAN2, OP_STEP, OP_SMOOTHSTEP) = range(20)
OP_GEGLU, OP_SWIGLU = 34, 35

DTYPE_F32, DTYPE_BF16, DTYPE_Q8, DTYPE_Q4, DTYPE_Q6 = 0, 1, 2, 3, 4
REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2
BROADCAST_MUL, BROADCAST_DIV, BROADCAST_ADD, BROADCAST_SUB = 0, 1, 2, 3


class DecodePlanOp(ctypes.Structure):
    """Flat decode-plan record: 16 x u32 + 2 x f32 (reference adamah.c:175-194)."""
    _fields_ = [(n, u32) for n in ("kind", "map_id", "map_id2", "op_code", "h0", "h1", "h2", "h3", "h4",
                                   "h5", "u0", "u1", "u2", "u3", "u4", "u5")] + [("f0", f32c), ("f1", f32c)]


def _resolve_lib_path(lib_path=None):
    """arg -> ADAMAH_LIB_PATH -> the library built beside this package (reference :156-181)."""
    if lib_path:
        return lib_path
    env = os.environ.get("ADAMAH_LIB_PATH")
    if env:
        return env
    here = os.path.dirname(os.path.abspath(__file__))
    cand = os.path.join(here, "libadamah_hip.so")
    if os.path.exists(cand):
        return cand
    raise FileNotFoundError(
        f"libadamah_hip.so not found in {here}\nBuild it first: python -m adam_amd.build")


# name -> (restype, argtypes).  Order of C arguments exactly as in include/adamah_hip.h.
_U = u32
_SIGS = {
    "adamah_init": (i32, []), "adamah_init_ex": (i32, [u64, u64]), "adamah_shutdown": (None, []),
    "adamah_sync": (None, []), "adamah_synchronize": (None, [u64]), "adamah_synchronize_all": (None, []),
    "adamah_fusion_enable": (None, [i32]), "adamah_fusion_is_enabled": (i32, []),
    "adamah_fusion_flush": (i32, []), "adamah_fusion_set_scheduler_mode": (None, [i32]),
    "adamah_fusion_get_scheduler_mode": (i32, []),
    "adamah_register_loc_span": (i32, [_U] * 4), "adamah_register_row_base_span": (i32, [_U] * 6),
    "adamah_clear_loc_alias_meta": (None, [_U]),
    "adamah_stats_reset": (None, []), "adamah_stats_get": (None, [pu64] * 9),
    "adamah_get_last_barrier_count": (u32, []), "adamah_is_integrated_gpu": (i32, []),
    "adamah_set_xq_matmul_wg": (None, [_U, _U]), "adamah_get_gpu_caps": (None, [pu32, pu32, pu64]),
    "adamah_probe_device": (i32, [pu64, pu64, pu64, pu32]),
    "adamah_set_dtype": (i32, [_U]), "adamah_get_dtype": (u32, []),
    "adamah_register_decode_plan": (i32, [_U, ctypes.POINTER(DecodePlanOp), _U]),
    "adamah_clear_decode_plan": (None, [_U]), "adamah_decode_step": (i32, [_U] * 3),
    "adamah_kv_cache_fp16": (i32, [_U] * 3),
    "adamah_attn_causal_rows_dev": (i32, [_U, pu32, _U, _U, _U, pu32, _U, _U, _U, _U, _U, f32c, f32c]),
    "adamah_qk_norm_rope_rows_dev": (i32, [_U, _U, pu32, _U, pu32, _U, pu32, _U, _U, _U, _U, _U, _U, f32c]),
    "batch_begin": (None, []), "batch_end": (None, []),
    "map_init": (i32, [_U] * 4), "map_init_dtype": (i32, [_U] * 5), "map_destroy": (i32, [_U]),
    "map_size": (u64, [_U]), "map_get_dtype": (u32, [_U]),
    "map_set_qparams": (i32, [_U, pf32, pf32, _U]),
    "map_scatter": (u64, [_U, pu32, vp, _U]), "map_scatter_contiguous": (u64, [_U, _U, vp, _U]),
    "map_scatter_q4_packed_contiguous": (u64, [_U, _U, vp, _U]),
    "map_gather": (u64, [_U, pu32, vp, _U]),
    "map_upload_dev": (u64, [_U, vp, _U]), "map_download_dev": (i32, [_U, vp, _U]),
    "map_gather_dev": (u64, [_U] * 3), "map_scatter_dev": (u64, [_U] * 4),
    "map_op1": (i32, [_U, _U, pu32, pu32, _U]), "map_op2": (i32, [_U, _U, pu32, pu32, pu32, _U]),
    "map_matmul": (i32, [_U, pu32, pu32, pu32] + [_U] * 4), "map_softmax": (i32, [_U, pu32, pu32, _U, _U]),
    "map_layernorm": (i32, [_U, pu32, pu32, pu32, pu32, _U, _U, f32c]),
    "map_broadcast": (i32, [_U, _U, pu32, pu32, pu32, _U]), "map_reduce": (i32, [_U, _U, pu32, pu32, _U]),
    "map_op1_dev": (i32, [_U] * 5), "map_op2_dev": (i32, [_U] * 6), "map_matmul_dev": (i32, [_U] * 8),
    "map_softmax_dev": (i32, [_U] * 5), "map_softmax_abs_dev": (i32, [_U] * 5),
    "map_attn_softmax_abs_dev": (i32, [_U] * 5 + [f32c, f32c]),
    "map_attn_softmax_value_dev": (i32, [_U] * 7 + [f32c, f32c]),
    "map_layernorm_dev": (i32, [_U] * 7 + [f32c]), "map_broadcast_dev": (i32, [_U] * 6),
    "map_reduce_dev": (i32, [_U] * 5), "map_argmax_dev": (i32, [_U] * 4),
    "map_topk_dev": (i32, [_U] * 6), "map_topp_dev": (i32, [_U] * 4 + [f32c, f32c]),
    "map_resolve_idx_dev": (i32, [_U] * 5), "map_sample_categorical_dev": (i32, [_U] * 6),
    "map_repeat_penalty_dev": (i32, [_U] * 4 + [f32c]),
    "map_rmsnorm_dev": (i32, [_U] * 6 + [f32c]), "map_rmsnorm_add_dev": (i32, [_U] * 7 + [f32c]),
    "map_rmsnorm_x_dev": (i32, [_U] * 7 + [f32c]), "map_rope_dev": (i32, [_U] * 7 + [f32c]),
    "map_qk_norm_rope_x_dev": (i32, [_U] * 12 + [f32c]),
    "map_matmul_t_dev": (i32, [_U] * 8), "map_row_copy_dev": (i32, [_U] * 5),
    "map_row_copy_offset_dev": (i32, [_U] * 6), "map_fma_dev": (i32, [_U] * 6),
    "map_matmul_t_x_dev": (i32, [_U] * 9), "map_matmul_x_dev": (i32, [_U] * 9),
    "map_matmul_t_xq4_dev": (i32, [_U] * 9), "map_matmul_xq4_dev": (i32, [_U] * 9),
    "map_matmul_t_xq8_dev": (i32, [_U] * 9), "map_matmul_xq8_dev": (i32, [_U] * 9),
    "map_row_gather_xq8_dev": (i32, [_U] * 6 + [f32c]),
    "map_matvec_argmax_t_xq4_dev": (i32, [_U] * 10), "map_matvec_argmax_t_xq8_dev": (i32, [_U] * 10),
    "map_matvec_topk_t_xq4_dev": (i32, [_U] * 11 + [f32c]), "map_matvec_topk_t_xq8_dev": (i32, [_U] * 11 + [f32c]),
    "map_matvec_topk_t_xq4_ex_dev": (i32, [_U] * 11 + [f32c, _U]),
    "map_matvec_topk_t_xq8_ex_dev": (i32, [_U] * 11 + [f32c, _U]),
    "map_matvec_rerank_t_xq8_dev": (i32, [_U] * 12 + [f32c]),
    "adamah_matvec_topk_t_xq4_noalloc_dev": (i32, [_U] * 11 + [f32c, _U]),
    "adamah_hip_embed_tokens_dev": (i32, [_U] * 8 + [f32c]),
    "adamah_hip_embed_post_tokens_dev": (i32, [_U] * 8 + [f32c, pu32]),
    "adamah_hip_token_post": (i32, [_U] * 3 + [pu32]), "adamah_hip_token_wait": (i32, [_U, pf32, _U]),
    "map_fused_qkv_t_xq4_dev": (i32, [_U] * 13), "map_fused_qkv_t_xq8_dev": (i32, [_U] * 13),
    "map_fused_gateup_t_xq4_dev": (i32, [_U] * 10), "map_fused_gateup_t_xq8_dev": (i32, [_U] * 10),
    "map_fused_gateup_act_t_xq8_dev": (i32, [_U] * 8),
    # timing helpers for benchmarks (HIP events on the library's own stream)
    "adamah_hip_timer_begin": (i32, []), "adamah_hip_timer_end": (f32c, []),
    "adamah_hip_debug_dequant": (i32, [_U, u64, u64, pf32]),
    "adamah_hip_map_layout": (i32, [_U]),
    "adamah_hip_stream_probe": (f32c, [u64, u64, _U, _U, _U]),
}

# Symbols the reference treats as optional feature flags (__init__.py:579-600, 713-832, 878-1100).
_OPTIONAL_FLAGS = {
    "map_scatter_contiguous": "_has_map_scatter_contiguous",
    "map_scatter_q4_packed_contiguous": "_has_map_scatter_q4_packed_contiguous",
    "map_matvec_argmax_t_xq4_dev": "_has_map_matvec_argmax_t_xq4_dev",
    "map_matvec_argmax_t_xq8_dev": "_has_map_matvec_argmax_t_xq8_dev",
    "adamah_stats_get": "_has_native_stats",
    "adamah_get_last_barrier_count": "_has_get_last_barrier_count",
    "adamah_fusion_set_scheduler_mode": "_has_fusion_scheduler",
    "adamah_register_decode_plan": "_has_decode_plan",
    "adamah_set_dtype": "_has_dtype",
    "adamah_kv_cache_fp16": "_has_kv_cache_fp16",
    "adamah_attn_causal_rows_dev": "_has_attn_causal_rows_dev",
    "adamah_qk_norm_rope_rows_dev": "_has_qk_norm_rope_rows_dev",
    "adamah_hip_embed_tokens_dev": "_has_token_feed",
    "map_resolve_idx_dev": "_has_map_resolve_idx_dev",
    "map_sample_categorical_dev": "_has_map_sample_categorical_dev",
    "map_repeat_penalty_dev": "_has_map_repeat_penalty_dev",
    "map_matvec_topk_t_xq4_dev": "_has_map_matvec_topk_t_xq4_dev",
    "map_matvec_topk_t_xq4_ex_dev": "_has_map_matvec_topk_t_xq4_ex_dev",
    "map_matvec_topk_t_xq8_dev": "_has_map_matvec_topk_t_xq8_dev",
    "map_matvec_topk_t_xq8_ex_dev": "_has_map_matvec_topk_t_xq8_ex_dev",
    "map_matvec_rerank_t_xq8_dev": "_has_map_matvec_rerank_t_xq8_dev",
    "map_fused_qkv_t_xq4_dev": "_has_map_fused_qkv_t_xq4_dev",
    "map_fused_qkv_t_xq8_dev": "_has_map_fused_qkv_t_xq8_dev",
    "map_fused_gateup_t_xq4_dev": "_has_map_fused_gateup_t_xq4_dev",
    "map_fused_gateup_t_xq8_dev": "_has_map_fused_gateup_t_xq8_dev",
    "map_fused_gateup_act_t_xq8_dev": "_has_map_fused_gateup_act_t_xq8_dev",
}
# Present in the reference surface, deliberately absent here: the monolithic full-decode /
# device-address API (the wg-size flag is tied to a Vulkan shader knob that has no effect here).
_ABSENT_FLAGS = (
    "_has_full_decode_step_api", "_has_full_decode_step", "_has_map_device_address", "_has_set_xq_matmul_wg",
)


def _as_u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


class Adamah:
    """ADAMAH op surface on an MI355X through libadamah_hip.so."""

    DTYPE_F32, DTYPE_BF16, DTYPE_Q8, DTYPE_Q4, DTYPE_Q6 = 0, 1, 2, 3, 4

    def __init__(self, lib_path=None, cache_mb=None, cold_cache_mb=None):
        self._lib = ctypes.CDLL(_resolve_lib_path(lib_path))
        for flag in _ABSENT_FLAGS:
            setattr(self, flag, hasattr(self._lib, flag.replace("_has_", "", 1)))
        for name, (res, args) in _SIGS.items():
            fn = getattr(self._lib, name)          # AttributeError when the library lacks it
            fn.restype, fn.argtypes = res, args
            if name in _OPTIONAL_FLAGS:
                setattr(self, _OPTIONAL_FLAGS[name], True)
        if cache_mb is not None or cold_cache_mb is not None:
            hot = int(cache_mb if cache_mb is not None else cold_cache_mb)
            cold = int(cold_cache_mb if cold_cache_mb is not None else hot)
            ret = self._lib.adamah_init_ex(hot << 20, cold << 20)
        else:
            ret = self._lib.adamah_init()
        if ret != 0:
            raise RuntimeError(f"adamah_init failed with code {ret}")
        self._is_integrated_gpu = bool(self._lib.adamah_is_integrated_gpu())
        wg, sub, vram = u32(0), u32(0), u64(0)
        self._lib.adamah_get_gpu_caps(ctypes.byref(wg), ctypes.byref(sub), ctypes.byref(vram))
        self._gpu_max_workgroup_size, self._gpu_subgroup_size = int(wg.value), int(sub.value)
        self._gpu_vram_bytes = int(vram.value)
        self._metrics = {'gather_calls': 0, 'scatter_calls': 0, 'op_calls': 0,
                         'total_bytes_cpu_to_gpu': 0, 'total_bytes_gpu_to_cpu': 0}
        self._maps = {}

    # ---- generic call helpers --------------------------------------------------------
    def _op(self, name, *args):
        self._metrics['op_calls'] += 1
        ret = getattr(self._lib, name)(*args)
        if ret != 0:
            raise RuntimeError(f"{name} failed with code {ret}")

    # ---- dtype / maps ----------------------------------------------------------------
    def set_dtype(self, dtype, group_size=128):
        ret = self._lib.adamah_set_dtype(dtype)
        if ret != 0:
            raise RuntimeError(f"Failed to set dtype {dtype} (code {ret})")
        self._active_dtype, self._group_size = dtype, group_size

    def get_dtype(self):
        return int(self._lib.adamah_get_dtype())

    def map_create_typed(self, map_id, dtype, pack_size, n_packs, group_size=128):
        ret = self._lib.map_init_dtype(map_id, dtype, pack_size, n_packs, group_size)
        if ret != 0:
            raise RuntimeError(f"map_init_dtype({dtype}) failed: {ret}")
        self._maps[map_id] = ({0: 4, 1: 2}.get(dtype, 1), pack_size, n_packs, dtype)

    def map_create(self, map_id, pack_size=0, n_packs=0, word_size=0, **kw):
        dtype = getattr(self, '_active_dtype', 0)
        if word_size > 0 and dtype == 0 and not hasattr(self, '_active_dtype'):
            ret = self._lib.map_init(map_id, word_size, pack_size, n_packs)
            if ret != 0:
                raise RuntimeError(f"map_init failed with code {ret}")
            self._maps[map_id] = (word_size, pack_size, n_packs, 0)
            return
        self.map_create_typed(map_id, dtype, pack_size, n_packs, getattr(self, '_group_size', 128))

    def map_init(self, map_id, word_size, pack_size, n_packs):
        return self.map_create(map_id, pack_size=pack_size, n_packs=n_packs, word_size=word_size)

    def map_destroy(self, map_id):
        ret = self._lib.map_destroy(map_id)
        if ret != 0:
            raise RuntimeError(f"map_destroy failed with code {ret}")
        self._maps.pop(map_id, None)

    def map_size(self, map_id):
        return int(self._lib.map_size(map_id))

    def set_qparams(self, map_id, scales, zero_points):
        s = np.ascontiguousarray(scales, dtype=np.float32)
        z = np.ascontiguousarray(zero_points, dtype=np.float32)
        ret = self._lib.map_set_qparams(map_id, s.ctypes.data_as(pf32), z.ctypes.data_as(pf32), len(s))
        if ret != 0:
            raise RuntimeError(f"map_set_qparams failed with code {ret}")

    def kv_cache_fp16(self, map_id, start, count):
        """Declare elements [start, start+count) of a float32 map an fp16-stored KV cache."""
        ret = self._lib.adamah_kv_cache_fp16(map_id, start, count)
        if ret != 0:
            raise RuntimeError(f"adamah_kv_cache_fp16 failed with code {ret}")

    # ---- host <-> map ----------------------------------------------------------------
    def scatter(self, map_id, locs, data):
        self._metrics['scatter_calls'] += 1
        locs = _as_u32(locs); data = np.ascontiguousarray(data)
        self._metrics['total_bytes_cpu_to_gpu'] += data.nbytes
        return int(self._lib.map_scatter(map_id, locs.ctypes.data_as(pu32), data.ctypes.data_as(vp), len(locs)))

    map_scatter = scatter

    def scatter_contiguous(self, map_id, start_pack, data, n_locs=None):
        arr = np.ascontiguousarray(data)
        n = int(arr.size if n_locs is None else n_locs)
        self._metrics['scatter_calls'] += 1
        self._metrics['total_bytes_cpu_to_gpu'] += arr.nbytes
        return int(self._lib.map_scatter_contiguous(map_id, start_pack, arr.ctypes.data_as(vp), n))

    map_scatter_contiguous = scatter_contiguous

    def scatter_q4_packed_contiguous(self, map_id, start_pack, packed_u8, n_locs=None):
        arr = np.ascontiguousarray(packed_u8, dtype=np.uint8)
        n = int(arr.size * 2 if n_locs is None else n_locs)
        self._metrics['scatter_calls'] += 1
        self._metrics['total_bytes_cpu_to_gpu'] += arr.nbytes
        return int(self._lib.map_scatter_q4_packed_contiguous(map_id, start_pack, arr.ctypes.data_as(vp), n))

    map_scatter_q4_packed_contiguous = scatter_q4_packed_contiguous

    def gather(self, map_id, locs, n_packs=None, n_locs=None):
        self._metrics['gather_calls'] += 1
        locs = _as_u32(locs)
        n = n_locs if n_locs is not None else (n_packs if n_packs is not None else len(locs))
        ps = self._maps.get(map_id, (4, 1, 0, 0))[1] or 1
        out = np.zeros(n * ps, dtype=np.uint32)
        self._lib.map_gather(map_id, locs.ctypes.data_as(pu32), out.ctypes.data_as(vp), n)
        self._metrics['total_bytes_gpu_to_cpu'] += out.nbytes
        return out

    map_gather = gather

    def upload_dev(self, data, handle=0):
        arr = np.ascontiguousarray(data)
        v = int(self._lib.map_upload_dev(handle, arr.ctypes.data_as(vp), arr.nbytes))
        return v & 0xFFFFFFFF, v >> 32

    def download_dev(self, handle, n_elems, dtype=np.float32):
        out = np.empty(n_elems, dtype=dtype)
        ret = self._lib.map_download_dev(handle, out.ctypes.data_as(vp), out.nbytes)
        if ret != 0:
            raise RuntimeError(f"map_download_dev failed with code {ret}")
        return out

    def map_gather_dev(self, map_id, locs_handle, n_locs):
        if map_id not in self._maps:
            raise ValueError(f"Map {map_id} not initialized")
        v = int(self._lib.map_gather_dev(map_id, locs_handle, n_locs))
        return v & 0xFFFFFFFF, v >> 32, n_locs * self._maps[map_id][1], np.float32

    def map_scatter_dev(self, map_id, locs_handle, n_locs, src_handle):
        if map_id not in self._maps:
            raise ValueError(f"Map {map_id} not initialized")
        return int(self._lib.map_scatter_dev(map_id, locs_handle, n_locs, src_handle))

    def synchronize(self, ticket):
        self._lib.adamah_synchronize(ticket)

    def synchronize_all(self):
        self._lib.adamah_synchronize_all()

    def sync(self):
        self._lib.adamah_sync()

    # ---- host-locs variants ----------------------------------------------------------
    def map_op1(self, map_id, op, locs_in, locs_out, n=None):
        a, b = _as_u32(locs_in), _as_u32(locs_out)
        self._op("map_op1", map_id, op, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32), len(a) if n is None else n)

    def map_op2(self, map_id, op, locs_a, locs_b, locs_out, n=None):
        a, b, c = _as_u32(locs_a), _as_u32(locs_b), _as_u32(locs_out)
        self._op("map_op2", map_id, op, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 c.ctypes.data_as(pu32), len(a) if n is None else n)

    def map_matmul(self, map_id, locs_a, locs_b, locs_c, M, K, N, n_ops=1):
        a, b, c = _as_u32(locs_a), _as_u32(locs_b), _as_u32(locs_c)
        self._op("map_matmul", map_id, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 c.ctypes.data_as(pu32), M, K, N, n_ops)

    def map_softmax(self, map_id, locs_in, locs_out, row_size, n_rows=None):
        a, b = _as_u32(locs_in), _as_u32(locs_out)
        self._op("map_softmax", map_id, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 len(a) if n_rows is None else n_rows, row_size)

    def map_layernorm(self, map_id, locs_src, locs_dst, locs_gamma, locs_beta, dim, eps=1e-5, n_rows=None):
        a, b, c, d = (_as_u32(x) for x in (locs_src, locs_dst, locs_gamma, locs_beta))
        self._op("map_layernorm", map_id, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 c.ctypes.data_as(pu32), d.ctypes.data_as(pu32), len(a) if n_rows is None else n_rows, dim, eps)

    def map_broadcast(self, map_id, op, locs_src, locs_scalar, locs_dst, n=None):
        op = {OP_MUL: 0, OP_DIV: 1, OP_ADD: 2, OP_SUB: 3}.get(op, op)
        a, b, c = _as_u32(locs_src), _as_u32(locs_scalar), _as_u32(locs_dst)
        self._op("map_broadcast", map_id, op, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 c.ctypes.data_as(pu32), len(a) if n is None else n)

    def map_reduce(self, map_id, op, locs_src, locs_dst, n=None):
        a, b = _as_u32(locs_src), _as_u32(locs_dst)
        self._op("map_reduce", map_id, op, a.ctypes.data_as(pu32), b.ctypes.data_as(pu32),
                 len(a) if n is None else n)

    # ---- device-locs ops -------------------------------------------------------------
    def map_op1_dev(self, map_id, op, locs_in_handle, locs_out_handle, n):
        self._op("map_op1_dev", map_id, op, locs_in_handle, locs_out_handle, n)

    def map_op2_dev(self, map_id, op, locs_a_handle, locs_b_handle, locs_out_handle, n):
        self._op("map_op2_dev", map_id, op, locs_a_handle, locs_b_handle, locs_out_handle, n)

    def map_matmul_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._op("map_matmul_dev", map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_softmax_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows):
        self._op("map_softmax_dev", map_id, locs_in_handle, locs_out_handle, n_rows, row_size)

    def map_softmax_abs_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows):
        self._op("map_softmax_abs_dev", map_id, locs_in_handle, locs_out_handle, n_rows, row_size)

    def map_attn_softmax_abs_dev(self, map_id, locs_in_handle, locs_out_handle, row_size, n_rows, scale, cap):
        self._op("map_attn_softmax_abs_dev", map_id, locs_in_handle, locs_out_handle, n_rows, row_size, scale, cap)

    def map_attn_softmax_value_dev(self, map_id, locs_scores_handle, locs_values_handle, locs_out_handle,
                                   n_ops, row_size, value_dim, scale, cap):
        self._op("map_attn_softmax_value_dev", map_id, locs_scores_handle, locs_values_handle,
                 locs_out_handle, n_ops, row_size, value_dim, scale, cap)

    def map_layernorm_dev(self, map_id, locs_src_handle, locs_dst_handle, locs_gamma_handle,
                          locs_beta_handle, dim, eps=1e-5, n_rows=0):
        self._op("map_layernorm_dev", map_id, locs_src_handle, locs_dst_handle, locs_gamma_handle,
                 locs_beta_handle, n_rows, dim, eps)

    def map_rmsnorm_dev(self, map_id, locs_src_handle, locs_wt_handle, locs_dst_handle, n_rows, dim, eps=1e-5):
        self._op("map_rmsnorm_dev", map_id, locs_src_handle, locs_wt_handle, locs_dst_handle, n_rows, dim, eps)

    def map_rmsnorm_x_dev(self, map_act, map_wt, locs_src_handle, locs_wt_handle, locs_dst_handle,
                          n_rows, dim, eps=1e-5):
        self._op("map_rmsnorm_x_dev", map_act, map_wt, locs_src_handle, locs_wt_handle, locs_dst_handle,
                 n_rows, dim, eps)

    def map_rmsnorm_add_dev(self, map_id, locs_src_handle, locs_wt_handle, locs_resid_handle,
                            locs_dst_handle, n_rows, dim, eps=1e-5):
        self._op("map_rmsnorm_add_dev", map_id, locs_src_handle, locs_wt_handle, locs_resid_handle,
                 locs_dst_handle, n_rows, dim, eps)

    def attn_causal_rows_dev(self, map_id, q_handles, locs_k_handle, locs_scores_handle, locs_v_handle, out_handles,
                             head_dim, n_keys0, n_heads, value_dim, scale, softcap=0.0):
        """Extension: for t in range(len(q_handles)) the pair map_matmul_t_dev(q_handles[t] -> scores over
        n_keys0 + t keys) / map_attn_softmax_value_dev(-> out_handles[t]) in one native call."""
        m = len(q_handles)
        qa = (ctypes.c_uint32 * m)(*q_handles)
        oa = (ctypes.c_uint32 * m)(*out_handles)
        self._op("adamah_attn_causal_rows_dev", map_id, qa, locs_k_handle, locs_scores_handle, locs_v_handle, oa, m,
                 head_dim, n_keys0, n_heads, value_dim, scale, softcap)

    def embed_tokens_dev(self, map_act, map_src, locs_tokens_handle, src_row0, dst_start, m, E, V, scale=1.0):
        """Extension: embedding rows of m tokens whose ids (float32) are still on the device, scaled, into
        m consecutive rows of map_act -- what map_gather_dev + map_scatter_dev + a multiplication give."""
        self._op("adamah_hip_embed_tokens_dev", map_act, map_src, locs_tokens_handle, src_row0, dst_start, m, E, V,
                 scale)

    def embed_post_tokens_dev(self, map_act, map_src, locs_tokens_handle, src_row0, dst_start, m, E, V, scale=1.0):
        """Extension: embed_tokens_dev whose launch also hands the m token values it reads to the host, as
        token_post does; returns the ticket to wait on."""
        t = ctypes.c_uint32(0)
        self._op("adamah_hip_embed_post_tokens_dev", map_act, map_src, locs_tokens_handle, src_row0, dst_start, m, E, V,
                 scale, ctypes.byref(t))
        return t.value

    def token_post(self, map_id, locs_handle, n):
        """Extension: in stream order, hand the n float32 values at the handle's elements to the host (ring of 8
        in pinned memory); returns the ticket to wait on."""
        t = ctypes.c_uint32(0)
        self._op("adamah_hip_token_post", map_id, locs_handle, n, ctypes.byref(t))
        return t.value

    def token_wait(self, ticket, n=1):
        """Extension: the values posted under `ticket`, as soon as the post has run -- work queued behind it is
        not waited for."""
        out = np.empty(n, np.float32)
        ret = self._lib.adamah_hip_token_wait(ticket, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), n)
        if ret != 0:
            raise RuntimeError(f"adamah_hip_token_wait failed with code {ret}")
        return out

    def qk_norm_rope_rows_dev(self, map_act, map_wt, q_src_handles, locs_q_wt_handle, k_src_handles, locs_k_wt_handle,
                              dst_handles, q_rows, q_dim, k_rows, k_dim, pos0, freq_base):
        """Extension: map_qk_norm_rope_x_dev for token t = 0 .. len(q_src_handles) - 1 at position pos0 + t in one
        native call."""
        m = len(q_src_handles)
        arr = lambda hs: (ctypes.c_uint32 * m)(*hs)
        self._op("adamah_qk_norm_rope_rows_dev", map_act, map_wt, arr(q_src_handles), locs_q_wt_handle, arr(k_src_handles),
                 locs_k_wt_handle, arr(dst_handles), m, q_rows, q_dim, k_rows, k_dim, pos0, freq_base)

    def map_rope_dev(self, map_id, locs_src_handle, locs_dst_handle, n_tokens, n_heads, head_dim,
                     pos_offset=0, freq_base=10000.0):
        self._op("map_rope_dev", map_id, locs_src_handle, locs_dst_handle, n_tokens, n_heads, head_dim,
                 pos_offset, freq_base)

    def map_qk_norm_rope_x_dev(self, map_act_id, map_wt_id, locs_q_src_handle, locs_q_wt_handle,
                               locs_k_src_handle, locs_k_wt_handle, locs_qk_dst_handle, q_rows, q_dim,
                               k_rows, k_dim, pos_offset, freq_base):
        self._op("map_qk_norm_rope_x_dev", map_act_id, map_wt_id, locs_q_src_handle, locs_q_wt_handle,
                 locs_k_src_handle, locs_k_wt_handle, locs_qk_dst_handle, q_rows, q_dim, k_rows, k_dim,
                 pos_offset, freq_base)

    def map_matmul_t_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._op("map_matmul_t_dev", map_id, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def _xmap(self, name, map_act, map_wt, a, b, c, M, K, N, n_ops):
        self._op(name, map_act, map_wt, a, b, c, M, K, N, n_ops)

    def map_matmul_t_x_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_t_x_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_matmul_x_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_x_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_matmul_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_t_xq4_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_matmul_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_xq4_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_matmul_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_matmul_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops=1):
        self._xmap("map_matmul_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_handle, locs_c_handle, M, K, N, n_ops)

    def map_row_gather_xq8_dev(self, map_act, map_wt, src_base, dst_base, row_idx, row_size, scale=1.0):
        self._op("map_row_gather_xq8_dev", map_act, map_wt, src_base, dst_base, row_idx, row_size, scale)

    def map_row_copy_dev(self, map_id, copy_spec_handle, src_base_handle, n_copies, row_size):
        self._op("map_row_copy_dev", map_id, copy_spec_handle, src_base_handle, n_copies, row_size)

    def map_row_copy_offset_dev(self, map_id, copy_spec_handle, src_base_handle, dst_row_offset, n_copies, row_size):
        self._op("map_row_copy_offset_dev", map_id, copy_spec_handle, src_base_handle, dst_row_offset,
                 n_copies, row_size)

    def map_fma_dev(self, map_id, locs_a_handle, locs_b_handle, locs_c_handle, locs_dst_handle, n_locs):
        self._op("map_fma_dev", map_id, locs_a_handle, locs_b_handle, locs_c_handle, locs_dst_handle, n_locs)

    def map_broadcast_dev(self, map_id, op, locs_src_handle, locs_scalar_handle, locs_dst_handle, n):
        op = {OP_MUL: 0, OP_DIV: 1, OP_ADD: 2, OP_SUB: 3}.get(op, op)
        self._op("map_broadcast_dev", map_id, op, locs_src_handle, locs_scalar_handle, locs_dst_handle, n)

    def map_reduce_dev(self, map_id, op, locs_src_handle, locs_dst_handle, n):
        self._op("map_reduce_dev", map_id, op, locs_src_handle, locs_dst_handle, n)

    def map_argmax_dev(self, map_id, locs_src_handle, locs_dst_handle, n):
        self._op("map_argmax_dev", map_id, locs_src_handle, locs_dst_handle, n)

    def map_topk_dev(self, map_id, locs_src_handle, locs_idx_dst_handle, locs_val_dst_handle, n, k):
        self._op("map_topk_dev", map_id, locs_src_handle, locs_idx_dst_handle, locs_val_dst_handle, n, k)

    def map_topp_dev(self, map_id, locs_src_handle, locs_dst_handle, n, temperature, top_p):
        self._op("map_topp_dev", map_id, locs_src_handle, locs_dst_handle, n, temperature, top_p)

    def map_resolve_idx_dev(self, map_id, base_locs_handle, sel_locs_handle, dst_locs_handle, n):
        self._op("map_resolve_idx_dev", map_id, base_locs_handle, sel_locs_handle, dst_locs_handle, n)

    def map_sample_categorical_dev(self, map_id, locs_idx_handle, locs_prob_handle, rand_loc_handle, dst_loc_handle, n):
        self._op("map_sample_categorical_dev", map_id, locs_idx_handle, locs_prob_handle, rand_loc_handle,
                 dst_loc_handle, n)

    def map_repeat_penalty_dev(self, map_id, locs_src_handle, token_ids_handle, n_ids, penalty):
        self._op("map_repeat_penalty_dev", map_id, locs_src_handle, token_ids_handle, n_ids, penalty)

    def map_fused_qkv_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle, locs_bv_handle,
                                locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v):
        self._op("map_fused_qkv_t_xq4_dev", map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle,
                 locs_bv_handle, locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v)

    def map_fused_qkv_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle, locs_bv_handle,
                                locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v):
        self._op("map_fused_qkv_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_bq_handle, locs_bk_handle,
                 locs_bv_handle, locs_cq_handle, locs_ck_handle, locs_cv_handle, K, N_q, N_k, N_v)

    def map_fused_gateup_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                   locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up):
        self._op("map_fused_gateup_t_xq4_dev", map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                 locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up)

    def map_fused_gateup_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                   locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up):
        self._op("map_fused_gateup_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                 locs_c_gate_handle, locs_c_up_handle, K, N_gate, N_up)

    def map_fused_gateup_act_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_gate_handle, locs_b_up_handle,
                                       locs_c_out_handle, K, N_ff):
        self._op("map_fused_gateup_act_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_gate_handle,
                 locs_b_up_handle, locs_c_out_handle, K, N_ff)

    def map_matvec_topk_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                  locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0, repeat_penalty=1.0):
        self._op("map_matvec_topk_t_xq4_dev", map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                 locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty, repeat_penalty)

    def map_matvec_topk_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                  locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0, repeat_penalty=1.0):
        self._op("map_matvec_topk_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                 locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty, repeat_penalty)

    def map_matvec_topk_t_xq4_ex_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                     locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0,
                                     repeat_penalty=1.0, rows_per_group=256):
        self._op("map_matvec_topk_t_xq4_ex_dev", map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                 locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty, repeat_penalty, rows_per_group)

    def map_matvec_topk_t_xq8_ex_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                                     locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty=0,
                                     repeat_penalty=1.0, rows_per_group=256):
        self._op("map_matvec_topk_t_xq8_ex_dev", map_act, map_wt, locs_a_handle, locs_b_handle, penalty_ids_handle,
                 locs_idx_dst_handle, locs_val_dst_handle, K, N, k, n_penalty, repeat_penalty, rows_per_group)

    def map_matvec_rerank_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, partial_idx_base_handle,
                                    sel_locs_handle, penalty_ids_handle, locs_idx_dst_handle, locs_val_dst_handle,
                                    K, n_ids, n_penalty=0, repeat_penalty=1.0):
        self._op("map_matvec_rerank_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_handle,
                 partial_idx_base_handle, sel_locs_handle, penalty_ids_handle, locs_idx_dst_handle,
                 locs_val_dst_handle, K, n_ids, n_penalty, repeat_penalty)

    def map_matvec_argmax_t_xq4_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_idx_tmp_handle,
                                    locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group):
        self._op("map_matvec_argmax_t_xq4_dev", map_act, map_wt, locs_a_handle, locs_b_handle,
                 locs_idx_tmp_handle, locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group)

    def map_matvec_argmax_t_xq8_dev(self, map_act, map_wt, locs_a_handle, locs_b_handle, locs_idx_tmp_handle,
                                    locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group):
        self._op("map_matvec_argmax_t_xq8_dev", map_act, map_wt, locs_a_handle, locs_b_handle,
                 locs_idx_tmp_handle, locs_val_tmp_handle, locs_dst_handle, K, N, rows_per_group)

    # ---- batching / fusion / stats ---------------------------------------------------
    def batch_begin(self):
        self._lib.batch_begin()

    def batch_end(self):
        self._lib.batch_end()

    @contextmanager
    def batch(self):
        self.batch_begin()
        try:
            yield
        finally:
            self.batch_end()

    def fusion_enable(self, enable):
        self._lib.adamah_fusion_enable(1 if enable else 0)

    def fusion_is_enabled(self):
        return bool(self._lib.adamah_fusion_is_enabled())

    def fusion_flush(self):
        ret = self._lib.adamah_fusion_flush()
        if ret != 0:
            raise RuntimeError(f"adamah_fusion_flush failed with code {ret}")

    @contextmanager
    def fusion_disabled(self):
        was = self.fusion_is_enabled()
        if was:
            self.fusion_enable(False)
        try:
            yield
        finally:
            if was:
                self.fusion_enable(True)

    def fusion_set_scheduler_mode(self, mode):
        if isinstance(mode, str):
            rev = {v: k for k, v in _SCHED_NAMES.items()}
            key = mode.strip().lower()
            if key not in rev:
                raise ValueError(f"Unknown fusion scheduler mode: {mode!r}")
            mode = rev[key]
        self._lib.adamah_fusion_set_scheduler_mode(int(mode))

    def fusion_get_scheduler_mode(self):
        return _SCHED_NAMES.get(int(self._lib.adamah_fusion_get_scheduler_mode()), "unknown")

    def register_loc_span(self, handle, map_id, start, count):
        ret = self._lib.adamah_register_loc_span(handle, map_id, start, count)
        if ret != 0:
            raise RuntimeError(f"adamah_register_loc_span failed with code {ret}")

    def register_row_base_span(self, handle, map_id, start, count, stride, row_size):
        ret = self._lib.adamah_register_row_base_span(handle, map_id, start, count, stride, row_size)
        if ret != 0:
            raise RuntimeError(f"adamah_register_row_base_span failed with code {ret}")

    def clear_loc_alias_meta(self, handle):
        self._lib.adamah_clear_loc_alias_meta(handle)

    def reset_native_stats(self):
        self._lib.adamah_stats_reset()

    def get_native_stats(self):
        vals = [u64(0) for _ in range(9)]
        self._lib.adamah_stats_get(*[ctypes.byref(v) for v in vals])
        keys = ("dispatch_count", "submit_count", "barrier_count", "fusion_flush_count",
                "descriptor_set_update_count", "descriptor_cache_hit_count", "descriptor_cache_miss_count",
                "alias_conflict_count", "scheduler_mode")
        out = {k: int(v.value) for k, v in zip(keys, vals)}
        out["scheduler_mode_name"] = _SCHED_NAMES.get(out["scheduler_mode"], "unknown")
        return out

    def get_last_barrier_count(self):
        return int(self._lib.adamah_get_last_barrier_count())

    # ---- decode plan -----------------------------------------------------------------
    def register_decode_plan(self, plan_id, ops):
        ops = list(ops)
        packed = (DecodePlanOp * max(1, len(ops)))()
        for i, op in enumerate(ops):
            if isinstance(op, dict):
                op = DecodePlanOp(**op)
            if not isinstance(op, DecodePlanOp):
                raise TypeError("decode plan ops must be DecodePlanOp instances or dicts")
            packed[i] = op
        ret = self._lib.adamah_register_decode_plan(plan_id, packed if ops else None, len(ops))
        if ret != 0:
            raise RuntimeError(f"adamah_register_decode_plan failed with code {ret}")

    def clear_decode_plan(self, plan_id):
        self._lib.adamah_clear_decode_plan(plan_id)

    def decode_step(self, plan_id, pos, seq_len):
        ret = self._lib.adamah_decode_step(plan_id, pos, seq_len)
        if ret != 0:
            raise RuntimeError(f"adamah_decode_step failed with code {ret}")

    # ---- benchmark / test helpers (not part of the reference surface) ------------------
    def timer_begin(self):
        """Record a HIP event on the library's stream."""
        if self._lib.adamah_hip_timer_begin() != 0:
            raise RuntimeError("adamah_hip_timer_begin failed")

    def timer_end(self):
        """Record the closing event, wait for it, return elapsed milliseconds."""
        ms = float(self._lib.adamah_hip_timer_end())
        if ms < 0:
            raise RuntimeError("adamah_hip_timer_end failed")
        return ms

    def debug_dequant(self, map_id, start, count):
        """Dequantised float32 values of elements [start, start+count) of a Q4/Q8 map, produced by
        the same unpack code the GEMV kernels use (for bit-exactness tests)."""
        out = np.empty(count, np.float32)
        ret = self._lib.adamah_hip_debug_dequant(map_id, start, count, out.ctypes.data_as(pf32))
        if ret != 0:
            raise RuntimeError(f"adamah_hip_debug_dequant failed with code {ret}")
        return out

    def stream_probe(self, bytes_per_launch, pool_bytes, mode=0, wg_per_cu=8, launches=64):
        """Average microseconds per launch of a plain read (mode 0) or copy (mode 1) kernel."""
        us = float(self._lib.adamah_hip_stream_probe(bytes_per_launch, pool_bytes, mode, wg_per_cu, launches))
        if us < 0:
            raise RuntimeError(f"adamah_hip_stream_probe failed with code {int(us)}")
        return us

    def map_layout(self, map_id):
        """0 = generic affine qparams, 1 = fp16-scale block plane (Q4_0 / Q8_0 recognised)."""
        return int(self._lib.adamah_hip_map_layout(map_id))

    # ---- misc ------------------------------------------------------------------------
    def reset_metrics(self):
        for k in self._metrics:
            self._metrics[k] = 0

    def shutdown(self):
        if getattr(self, "_lib", None) is not None:
            self._lib.adamah_shutdown()

    def __repr__(self):
        return f"Adamah(hip, v{__version__})"


def init(cache_mb=None, cold_cache_mb=None, lib_path=None):
    """Create the context (reference `adamah.init()`, __init__.py:2926-2981).  Pool sizes are
    accepted for compatibility; handles live in a growable device arena, so no size ladder is
    needed."""
    return Adamah(lib_path=lib_path, cache_mb=cache_mb, cold_cache_mb=cold_cache_mb)
