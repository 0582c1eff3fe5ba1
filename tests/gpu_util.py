"""Helpers for parity tests: run one scenario on the HIP library and on the oracle."""
import sys

import numpy as np

from adam_amd import adamah as A


def note(msg):
    """Name the case before the GPU step runs, flushed, so a lost box still says where it was."""
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def up(g, a):
    h, _ = g.upload_dev(np.asarray(a, np.uint32))
    assert h != 0
    return h


def f32map(g, mid, n, data=None, at=0):
    g.set_dtype(A.DTYPE_F32)
    g.map_create(mid, 1, n)
    if data is not None:
        data = np.ascontiguousarray(data, np.float32).reshape(-1)
        g.scatter_contiguous(mid, at, data)


def put(g, mid, at, data):
    data = np.ascontiguousarray(data, np.float32).reshape(-1)
    g.scatter_contiguous(mid, at, data)


def read(g, mid, lo, n):
    return g.gather(mid, np.arange(lo, lo + n, dtype=np.uint32)).view(np.float32).copy()


def rel_l2(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def load_qtensor(g, mid, qt, offset=0, total=None, scale=None, zp=None):
    """Upload a QTensor the way the harness does (qparams + packed codes) at element `offset`."""
    n = qt.size
    total = total or (offset + n)
    dtype = A.DTYPE_Q4 if qt.kind == 'q4_0' else A.DTYPE_Q8
    g.map_create_typed(mid, dtype, 1, total, 32)
    s, z = qt.qparams()
    if scale is not None:
        s, z = scale, zp
    ng = (total + 31) // 32
    sc = np.ones(ng, np.float32); zz = np.zeros(ng, np.float32)
    sc[offset // 32: offset // 32 + s.size] = s
    zz[offset // 32: offset // 32 + z.size] = z
    g.set_qparams(mid, sc, zz)
    if dtype == A.DTYPE_Q4:
        g.scatter_q4_packed_contiguous(mid, offset, qt.codes, n_locs=n)
    else:
        g.scatter_contiguous(mid, offset, qt.codes)


def device_free_bytes():
    """Free device memory as the HIP runtime reports it (hipMemGetInfo); used to show that a call allocates nothing."""
    import ctypes
    rt = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    rc = rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total))
    assert rc == 0, f"hipMemGetInfo returned {rc}"
    return free.value
