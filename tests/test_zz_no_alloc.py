"""The entry point that allocates nothing, adamah_matvec_topk_t_xq4_noalloc_dev, against the entry point it
is a variant of, map_matvec_topk_t_xq4_ex_dev: both called through the C ABI on the same inputs, outputs
compared bit for bit (same kernels, same order of arithmetic; only the logit buffer differs).  Two calls in a
row, the second with a smaller matrix, so that what the first call left in the fixed array would show.
The limit (N <= 262144) and the refusal while ops are queued in an open batch are checked too, and that the free
device memory the HIP runtime reports is the same before and after the call."""
import ctypes
import os

import numpy as np
import pytest

from adam_amd import quant
from gpu_util import note, up, f32map, read, load_qtensor, device_free_bytes

pytestmark = pytest.mark.gpu


def _lists(g, K, ng, k):
    return read(g, 0, K, ng * k).view(np.uint32).copy(), read(g, 0, K + ng * k, ng * k).view(np.uint32).copy()


def _both(hip, N, K, k, rpg, n_pen, seed):
    rng = np.random.default_rng(seed)
    qt = quant.quantize_q4_0(rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05))
    x = rng.standard_normal(K).astype(np.float32)
    pen = rng.integers(0, N, max(n_pen, 1)).astype(np.uint32)
    ng = (N + rpg - 1) // rpg
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, K + 2 * ng * k + 8, x)
    args = [0, 1, up(hip, [0]), up(hip, [0]), up(hip, pen), up(hip, K + np.arange(ng * k)),
            up(hip, K + ng * k + np.arange(ng * k)), K, N, k, n_pen]
    lib = hip._lib
    outs = []
    for name in ("map_matvec_topk_t_xq4_ex_dev", "adamah_matvec_topk_t_xq4_noalloc_dev"):
        # poison the result lists so that a call that wrote nothing cannot pass
        hip.scatter_contiguous(0, K, np.full(2 * ng * k, 12345.0, np.float32))
        hip.sync()
        note(f"{name} N={N} K={K} k={k} rows_per_group={rpg}")
        free_before = device_free_bytes()
        rc = getattr(lib, name)(*[ctypes.c_uint32(v) for v in args], ctypes.c_float(1.3), ctypes.c_uint32(rpg))
        assert rc == 0, (name, rc)
        hip.sync()
        if name.endswith("_noalloc_dev"):        # its kernels have run before (the sibling launches the same ones)
            assert device_free_bytes() == free_before, "the entry point that allocates nothing changed free device memory"
        outs.append(_lists(hip, K, ng, k))
    return outs


def test_noalloc_equals_the_allocating_entry_point_twice_in_a_row(hip):
    assert hasattr(hip._lib, "adamah_matvec_topk_t_xq4_noalloc_dev")
    for N, K, k, rpg, n_pen, seed in ((6000, 1152, 40, 256, 5, 1), (900, 512, 8, 128, 2, 2)):   # second call: smaller
        (i0, v0), (i1, v1) = _both(hip, N, K, k, rpg, n_pen, seed)
        assert not np.any(v0 == np.float32(12345.0).view(np.uint32))
        assert np.array_equal(i0, i1), f"indices differ at N={N}"
        assert np.array_equal(v0, v1), f"values differ at N={N}"


def test_noalloc_limit_and_queue_refusal(hip):
    lib = hip._lib
    qt = quant.quantize_q4_0(np.ones((8, 32), np.float32))
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, 512, np.ones(32, np.float32))
    a, b, p, i, v = up(hip, [0]), up(hip, [0]), up(hip, [0]), up(hip, 64 + np.arange(64)), up(hip, 200 + np.arange(64))
    u = ctypes.c_uint32
    call = lambda N, rpg: lib.adamah_matvec_topk_t_xq4_noalloc_dev(u(0), u(1), u(a), u(b), u(p), u(i), u(v), u(32), u(N),
                                                                    u(4), u(0), ctypes.c_float(1.0), u(rpg))
    note("noalloc limits")
    assert call(8, 4) == 0
    assert call(262145, 262145) == -3                # beyond the fixed array: refused before anything is launched
    hip.batch_begin()
    hip.map_rmsnorm_dev(0, up(hip, [0]), up(hip, [0]), up(hip, [300]), 1, 32, 1e-6)   # queued in the open batch
    rc_queued = call(8, 4)
    hip.sync()                                       # launches what is queued
    rc_flushed = call(8, 4)
    hip.batch_end()
    assert rc_flushed == 0
    # a one-row norm inside a batch is queued (unless the queue is switched off): refused until flushed
    assert rc_queued == (0 if os.environ.get("ADAMAH_NO_FUSE", "0") not in ("", "0") else -3)
