"""GEMV + partial top-k per group of rows, and the shortlist rerank: HIP vs oracle through the C ABI.

Bars.  Logits: within 1e-3 relative L2 of the oracle (float32 accumulation on the device, float64 in the
oracle), every stored value within 1e-3 * max|logit| of the oracle's logit of the stored row.  Ranking:
each group's list is sorted by (value descending, row ascending) on the device's own values, holds no row
twice, and no row it leaves out beats its last entry by more than that tolerance.  Rows listed for the
repeat penalty carry the penalised value.  Empty slots: index 0 and -FLT_MAX, bit-exact."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd import quant
from gpu_util import note, up, f32map, read, load_qtensor

pytestmark = pytest.mark.gpu
NEG_MAX = np.float32(-3.402823466e+38)


def run_topk(g, qt, x, k, rpg, pen, rp, ex=True, offset=0, scale=None, zp=None):
    N, K = qt.shape
    ng = (N + rpg - 1) // rpg
    load_qtensor(g, 1, qt, offset=offset, scale=scale, zp=zp)
    f32map(g, 0, K + 2 * ng * k + 8, x)
    q4 = qt.kind == 'q4_0'
    idx_h, val_h = up(g, K + np.arange(ng * k)), up(g, K + ng * k + np.arange(ng * k))
    pen_h = up(g, pen if len(pen) else [0])
    args = (0, 1, up(g, [0]), up(g, [offset]), pen_h, idx_h, val_h, K, N, k, len(pen), rp)
    g.batch_begin()
    if ex:
        (g.map_matvec_topk_t_xq4_ex_dev if q4 else g.map_matvec_topk_t_xq8_ex_dev)(*args, rpg)
    else:
        (g.map_matvec_topk_t_xq4_dev if q4 else g.map_matvec_topk_t_xq8_dev)(*args)
    g.batch_end()
    return read(g, 0, K, ng * k).reshape(ng, k), read(g, 0, K + ng * k, ng * k).reshape(ng, k)


def check(hip_out, ora, N, k, rpg):
    idx, val = hip_out
    y = ora.last_logits                      # the oracle's logits after the penalty
    tol = 1e-3 * float(np.abs(y).max())
    for g in range(idx.shape[0]):
        rows = np.arange(g * rpg, min(N, (g + 1) * rpg))
        n_fill = min(k, rows.size)
        ids = idx[g, :n_fill].astype(np.int64)
        assert np.all(ids == idx[g, :n_fill]) and len(set(ids.tolist())) == n_fill
        assert np.all((ids >= rows[0]) & (ids <= rows[-1]))
        assert np.all(np.abs(val[g, :n_fill] - y[ids]) <= tol)
        v = val[g, :n_fill]
        assert np.all((v[:-1] > v[1:]) | ((v[:-1] == v[1:]) & (ids[:-1] < ids[1:])))
        left = np.setdiff1d(rows, ids)
        if left.size:
            assert y[left].max() <= v[-1] + 2 * tol
        assert np.all(idx[g, n_fill:] == 0) and np.all(val[g, n_fill:].view(np.uint32) == NEG_MAX.view(np.uint32))


@pytest.mark.parametrize("kind,N,K,k,rpg,n_pen", [
    ("q4", 5000, 1152, 40, 256, 5),      # ragged K, last group short
    ("q4", 4096, 4096, 64, 1000, 64),    # rows_per_group that does not divide N, full penalty list
    ("q4", 300, 4096, 8, 512, 0),        # one group
    ("q4", 70, 256, 64, 32, 3),          # groups shorter than k: empty slots
    ("q4", 4100, 256, 12, 2048, 4),      # groups above 1024 rows: ranked in rounds
    ("q8", 3000, 128, 64, 1500, 0),
    ("q8", 777, 256, 16, 100, 7),
    ("q8", 2048, 1152, 1, 256, 2),
])
def test_topk_against_oracle(hip, kind, N, K, k, rpg, n_pen):
    rng = np.random.default_rng(N + K + k)
    w = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05)
    qt = (quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0)(w)
    x = rng.standard_normal(K).astype(np.float32)
    pen = rng.integers(0, N + 10, n_pen).astype(np.uint32)     # some beyond N, duplicates allowed
    if n_pen > 2:
        pen[1] = pen[0]
    o = oracle.init()
    note(f"matvec_topk {kind} {N}x{K} k={k} rpg={rpg} pen={n_pen}")
    got = run_topk(hip, qt, x, k, rpg, pen, 1.7)
    run_topk(o, qt, x, k, rpg, pen, 1.7)
    check(got, o, N, k, rpg)


def test_topk_default_group_and_penalty_effect(hip):
    """The form without rows_per_group uses 256; a penalised favourite drops out of its group's list."""
    rng = np.random.default_rng(3)
    N, K, k = 600, 512, 4
    w = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05)
    x = rng.standard_normal(K).astype(np.float32)
    qt = quant.quantize_q4_0(w)
    o = oracle.init()
    run_topk(o, qt, x, k, 256, [], 1.0, ex=False)
    fav = int(np.argmax(o.last_logits[:256]))
    note("matvec_topk default group size")
    got = run_topk(hip, qt, x, k, 256, [], 1.0, ex=False)
    check(got, o, N, k, 256)
    assert int(got[0][0, 0]) == fav
    o2 = oracle.init()
    run_topk(o2, qt, x, k, 256, [fav], 1000.0, ex=False)
    got2 = run_topk(hip, qt, x, k, 256, [fav], 1000.0, ex=False)
    check(got2, o2, N, k, 256)
    assert fav not in got2[0][0].astype(np.int64).tolist()


def test_topk_affine_and_unaligned_base(hip):
    """Affine qparams at a base that is not block aligned: the element-wise GEMV path."""
    rng = np.random.default_rng(8)
    N, K, k, rpg = 200, 96, 5, 64
    qt = quant.quantize_q4_0(rng.standard_normal((N + 1, K), dtype=np.float32))
    s = rng.uniform(0.001, 0.1, (N + 1) * K // 32).astype(np.float32)
    z = rng.uniform(-1, 1, (N + 1) * K // 32).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    outs = []
    o = oracle.init()
    for g in (hip, o):
        note("matvec_topk affine unaligned")
        load_qtensor(g, 1, qt, scale=s, zp=z)
        f32map(g, 0, 1024, x)
        g.map_matvec_topk_t_xq4_ex_dev(0, 1, up(g, [0]), up(g, [6]), up(g, [0]), up(g, 128 + np.arange(4 * k)),
                                       up(g, 256 + np.arange(4 * k)), K, N, k, 0, 1.0, rpg)
        outs.append((read(g, 0, 128, 4 * k).reshape(4, k), read(g, 0, 256, 4 * k).reshape(4, k)))
    check(outs[0], o, N, k, rpg)


def test_rerank_against_oracle(hip):
    rng = np.random.default_rng(5)
    N, K, n_ids = 3000, 1152, 48
    qt = quant.quantize_q8_0(rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05))
    x = rng.standard_normal(K).astype(np.float32)
    partial = rng.integers(0, N, 100).astype(np.float32)          # token ids of a partial list
    sel = rng.integers(0, 100, n_ids).astype(np.float32)          # positions picked from it
    pen = np.unique(partial[sel[:9].astype(np.int64)].astype(np.uint32))
    outs = []
    for g in (hip, oracle.init()):
        note("matvec_rerank q8")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + 512, np.concatenate([x, partial, sel]))
        g.batch_begin()
        g.map_matvec_rerank_t_xq8_dev(0, 1, up(g, [0]), up(g, [0]), up(g, [K]), up(g, K + 100 + np.arange(n_ids)),
                                      up(g, pen), up(g, K + 200 + np.arange(n_ids)), up(g, K + 300 + np.arange(n_ids)),
                                      K, n_ids, len(pen), 1.3)
        g.batch_end()
        outs.append((read(g, 0, K + 200, n_ids), read(g, 0, K + 300, n_ids)))
    assert np.array_equal(outs[0][0], outs[1][0])
    assert np.array_equal(outs[0][0], partial[sel.astype(np.int64)])
    assert np.allclose(outs[0][1], outs[1][1], rtol=1e-4, atol=1e-4)


def test_limits_and_errors(hip):
    note("matvec_topk limits")
    qt = quant.quantize_q4_0(np.ones((8, 32), np.float32))
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, 512, np.ones(32, np.float32))
    a, b, p, i, v = up(hip, [0]), up(hip, [0]), up(hip, [0]), up(hip, 64 + np.arange(65)), up(hip, 200 + np.arange(65))
    hip.map_matvec_topk_t_xq4_ex_dev(0, 1, a, b, p, i, v, 32, 0, 4, 0, 1.0, 4)        # N = 0: nothing to do
    hip.map_matvec_topk_t_xq4_ex_dev(0, 1, a, b, p, i, v, 32, 8, 0, 0, 1.0, 4)        # k = 0: nothing to do
    for bad in (dict(k=65), dict(n_pen=65), dict(rpg=0), dict(idx=up(hip, [64, 65, 66])), dict(wt=0), dict(pen=987654)):
        with pytest.raises(RuntimeError):
            hip.map_matvec_topk_t_xq4_ex_dev(0, bad.get("wt", 1), a, b, bad.get("pen", p), bad.get("idx", i), v, 32, 8,
                                             bad.get("k", 4), bad.get("n_pen", 0), 1.0, bad.get("rpg", 4))
    with pytest.raises(RuntimeError):                                                  # Q8 entry on a Q4 map
        hip.map_matvec_topk_t_xq8_dev(0, 1, a, b, p, i, v, 32, 8, 4, 0, 1.0)
    with pytest.raises(RuntimeError):
        hip.map_matvec_rerank_t_xq8_dev(0, 1, a, b, a, i, p, i, v, 32, 65, 0, 1.0)     # n_ids > 64
