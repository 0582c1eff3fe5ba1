"""The C-ABI library loads and exports every symbol the header declares (no GPU calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "adamah_hip.h")
LIB = os.path.join(ROOT, "adam_amd", "libadamah_hip.so")


def declared_symbols():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    src = re.sub(r"typedef struct.*?\}\s*\w+;", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b((?:adamah_|map_|batch_)\w+)\s*\(", src)))


def test_header_declares_the_mandatory_surface():
    names = set(declared_symbols())
    # symbols the reference binding dereferences unconditionally (adamah/__init__.py:530-967)
    mandatory = """adamah_init adamah_shutdown adamah_sync adamah_fusion_enable adamah_fusion_is_enabled
    adamah_fusion_flush map_init map_destroy map_size map_scatter map_gather map_op1 map_op2 map_matmul
    map_softmax map_layernorm map_broadcast map_reduce map_upload_dev map_download_dev map_gather_dev
    map_scatter_dev map_op1_dev map_op2_dev map_matmul_dev map_softmax_dev map_softmax_abs_dev
    map_attn_softmax_abs_dev map_attn_softmax_value_dev map_layernorm_dev map_broadcast_dev map_reduce_dev
    map_argmax_dev map_topk_dev map_topp_dev map_rmsnorm_dev map_rmsnorm_add_dev map_rope_dev
    map_matmul_t_dev map_row_copy_dev map_row_copy_offset_dev map_fma_dev map_matmul_t_x_dev
    map_matmul_x_dev map_matmul_t_xq4_dev map_matmul_xq4_dev map_matmul_t_xq8_dev map_matmul_xq8_dev
    map_row_gather_xq8_dev map_rmsnorm_x_dev map_qk_norm_rope_x_dev adamah_synchronize
    adamah_synchronize_all batch_begin batch_end""".split()
    missing = [m for m in mandatory if m not in names]
    assert not missing, missing


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build the library first: python -m adam_amd.build"
    lib = ctypes.CDLL(LIB)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_library_leaves_out_the_full_decode_api():
    # with these present a non-Broadcom reference engine would build extra maps at init
    # (adam/models/engine.py:2785-2812); they must stay absent
    lib = ctypes.CDLL(LIB)
    for s in ("adamah_full_decode_register", "adamah_full_decode_step", "adamah_has_full_decode_step",
              "adamah_get_map_buffer_device_address", "adamah_get_map_qparam_device_address"):
        assert not hasattr(lib, s), s


def test_binding_signature_table_matches_header():
    from adam_amd import adamah
    assert set(adamah._SIGS) == set(declared_symbols())


def test_uninitialised_calls_return_invalid():
    lib = ctypes.CDLL(LIB)
    lib.map_init.restype = ctypes.c_int
    lib.map_init.argtypes = [ctypes.c_uint32] * 4
    assert lib.map_init(0, 4, 1, 16) == -3          # no context yet
    lib.adamah_decode_step.restype = ctypes.c_int
    lib.adamah_decode_step.argtypes = [ctypes.c_uint32] * 3
    assert lib.adamah_decode_step(8, 0, 0) == -3    # plan id out of range
    assert lib.adamah_decode_step(1, 0, 0) == -4    # plan not registered
