"""Projections that share an activation vector (Q/K/V, gate/up, gate/up + SiLU) in one call: HIP vs the
oracle through the C ABI, 1e-3 relative L2 per projection (the bar of the GEMV they are made of).

Also checked: matrices and results that lie back to back cost ONE launch (two when a gated activation
follows: it folds into the same launch), matrices apart cost one launch each, results are the same
either way, and the calls work outside a batch."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd import quant
from gpu_util import note, up, f32map, read, rel_l2, load_qtensor

pytestmark = pytest.mark.gpu
TOL = 1e-3


def stacked(kind, rows, K, seed, gap=0):
    """One QTensor holding the matrices one after the other (`gap` unused rows between them)."""
    rng = np.random.default_rng(seed)
    tot = sum(rows) + gap * (len(rows) - 1)
    w = rng.standard_normal((tot, K), dtype=np.float32) * np.float32(0.05)
    qt = (quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0)(w)
    bases, r = [], 0
    for n in rows:
        bases.append(r * K)
        r += n + gap
    return qt, bases


@pytest.mark.parametrize("kind,K,rows,gap,batch", [
    ("q4", 1152, (1024, 256, 256), 0, True),      # Gemma-3-1B QKV, adjacent: one launch
    ("q4", 4096, (4096, 1024, 1024), 0, False),   # Llama-3-8B QKV outside a batch
    ("q4", 1152, (1024, 256, 256), 36, True),     # matrices apart: three launches
    ("q4", 4096, (512, 0, 256), 0, True),         # a projection without rows
    ("q8", 1152, (1024, 256, 256), 0, True),
])
def test_fused_qkv(hip, kind, K, rows, gap, batch):
    qt, bases = stacked(kind, rows, K, K + sum(rows), gap=gap)
    x = np.random.default_rng(1).standard_normal(K).astype(np.float32)
    outs, launches = [], None
    for g in (hip, oracle.init()):
        note(f"fused_qkv {kind} K={K} rows={rows} gap={gap} batch={batch}")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + sum(rows) + 64, x)
        cs = [K, K + rows[0], K + rows[0] + rows[1]]
        fn = g.map_fused_qkv_t_xq4_dev if kind == "q4" else g.map_fused_qkv_t_xq8_dev
        hs = [up(g, [0])] + [up(g, [b]) for b in bases] + [up(g, [c]) for c in cs]
        if batch:
            g.batch_begin()
        fn(0, 1, *hs, K, *rows)
        if batch:
            g.batch_end()
        if g is hip and batch:
            launches = g.get_last_barrier_count()
        outs.append(read(g, 0, K, sum(rows)))
    lo = 0
    for n in rows:
        if n:
            assert rel_l2(outs[0][lo:lo + n], outs[1][lo:lo + n]) < TOL
        lo += n
    if launches is not None and kind == "q4":
        n_proj = sum(1 for n in rows if n)
        assert launches == (1 if gap == 0 else n_proj), launches


@pytest.fixture(params=["0", "2"], ids=["paired-rows", "split-rows"])
def glu_form(request, monkeypatch):
    """Both ways the gate / up GEMV with the folded gated activation deals out its rows (the default chooses by size)."""
    monkeypatch.setenv("ADAMAH_GLU_SPLIT", request.param)
    return request.param


@pytest.mark.parametrize("K,ff,act", [(1152, 6912, "geglu"), (4096, 14336, "swiglu"), (2048, 1028, "swiglu"), (512, 36, "geglu"),
                                      (1536, 2050, "swiglu"), (8192, 8192, "swiglu")])
def test_folded_gated_activation_in_both_row_orders(hip, glu_form, K, ff, act):
    """Gate and up rows, and act(gate) * up, from one launch in either form: whole bundles, a last workgroup with few
    rows, fewer bundles than waves, a row count the split form cannot take (ff not a multiple of four), and rows long
    and many enough for workgroups of 16 waves."""
    qt, bases = stacked("q4", (ff, ff), K, ff)
    x = np.random.default_rng(ff).standard_normal(K).astype(np.float32)
    outs, launches = [], None
    for g in (hip, oracle.init()):
        note(f"fused_gateup q4 K={K} ff={ff} act={act} form={glu_form}")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + 3 * ff + 64, x)
        g.batch_begin()
        g.map_fused_gateup_t_xq4_dev(0, 1, up(g, [0]), up(g, [bases[0]]), up(g, [bases[1]]), up(g, [K]), up(g, [K + ff]), K, ff, ff)
        g.map_op2_dev(0, A.OP_GEGLU if act == "geglu" else A.OP_SWIGLU, up(g, K + np.arange(ff)), up(g, K + ff + np.arange(ff)),
                      up(g, K + 2 * ff + np.arange(ff)), ff)
        g.batch_end()
        if g is hip:
            launches = g.get_last_barrier_count()
        outs.append(read(g, 0, K, 3 * ff + 8))
    for part in range(3):
        assert rel_l2(outs[0][part * ff:(part + 1) * ff], outs[1][part * ff:(part + 1) * ff]) < TOL, part
    assert np.array_equal(outs[0][3 * ff:], outs[1][3 * ff:])      # nothing written past the results
    assert launches == 1, launches


@pytest.mark.parametrize("kind,K,ff,act", [("q4", 1152, 6912, "geglu"), ("q4", 4096, 14336, "swiglu"), ("q4", 4096, 1024, None),
                                           ("q8", 1152, 512, None)])
def test_fused_gateup_and_folded_activation(hip, kind, K, ff, act):
    qt, bases = stacked(kind, (ff, ff), K, ff)
    x = np.random.default_rng(2).standard_normal(K).astype(np.float32)
    outs, launches = [], None
    for g in (hip, oracle.init()):
        note(f"fused_gateup {kind} K={K} ff={ff} act={act}")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + 3 * ff + 64, x)
        fn = g.map_fused_gateup_t_xq4_dev if kind == "q4" else g.map_fused_gateup_t_xq8_dev
        g.batch_begin()
        fn(0, 1, up(g, [0]), up(g, [bases[0]]), up(g, [bases[1]]), up(g, [K]), up(g, [K + ff]), K, ff, ff)
        if act:
            g.map_op2_dev(0, A.OP_GEGLU if act == "geglu" else A.OP_SWIGLU, up(g, K + np.arange(ff)), up(g, K + ff + np.arange(ff)),
                          up(g, K + 2 * ff + np.arange(ff)), ff)
        g.batch_end()
        if g is hip:
            launches = g.get_last_barrier_count()
        outs.append(read(g, 0, K, 3 * ff))
    assert rel_l2(outs[0][:ff], outs[1][:ff]) < TOL and rel_l2(outs[0][ff:2 * ff], outs[1][ff:2 * ff]) < TOL
    if act:
        assert rel_l2(outs[0][2 * ff:], outs[1][2 * ff:]) < TOL
    if kind == "q4":
        assert launches == 1, launches


def test_fused_gateup_act_q8(hip):
    rng = np.random.default_rng(4)
    K, ff = 1152, 700
    qt, bases = stacked("q8", (ff, ff), K, 9)
    x = rng.standard_normal(K).astype(np.float32)
    outs = []
    for g in (hip, oracle.init()):
        note("fused_gateup_act q8")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + ff + 64, x)
        g.map_fused_gateup_act_t_xq8_dev(0, 1, up(g, [0]), up(g, [bases[0]]), up(g, [bases[1]]), up(g, [K]), K, ff)
        outs.append(read(g, 0, K, ff))
    assert rel_l2(outs[0], outs[1]) < TOL


def test_errors(hip):
    note("fused projections: errors")
    qt = quant.quantize_q4_0(np.ones((8, 32), np.float32))
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, 256, np.ones(32, np.float32))
    a, b, c = up(hip, [0]), up(hip, [0]), up(hip, [64])
    hip.map_fused_qkv_t_xq4_dev(0, 1, a, b, b, b, c, c, c, 32, 0, 0, 0)                # no rows: nothing to do
    with pytest.raises(RuntimeError):
        hip.map_fused_qkv_t_xq4_dev(0, 1, a, b, b, 987654, c, c, c, 32, 4, 0, 0)       # a missing handle, even unused
    with pytest.raises(RuntimeError):
        hip.map_fused_qkv_t_xq8_dev(0, 1, a, b, b, b, c, c, c, 32, 4, 0, 0)            # Q8 entry on a Q4 map
    with pytest.raises(RuntimeError):
        hip.map_fused_gateup_t_xq4_dev(0, 1, a, b, b, c, up(hip, [250]), 32, 4, 8)     # result past the map
    with pytest.raises(RuntimeError):
        hip.map_fused_gateup_act_t_xq8_dev(0, 1, a, b, b, c, 32, 4)                    # Q8 only


def test_fused_projection_kinds_in_a_decode_plan(hip):
    """Decode-plan kinds 26..30 (adamah.c:10318-10334; the Q/K/V forms carry their seventh handle in u0) replay
    the fused entry points: same words as the direct calls."""
    K, rows, ff = 1152, (1024, 256, 256), 768
    x = np.random.default_rng(3).standard_normal(K).astype(np.float32)
    got = {}
    for route in ("direct", "plan"):
        note(f"fused kinds via {route}")
        res = []
        for kind, kq, kg in (("q4", A.DECODE_OP_FUSED_QKV_T_XQ4, A.DECODE_OP_FUSED_GATEUP_T_XQ4),
                             ("q8", A.DECODE_OP_FUSED_QKV_T_XQ8, A.DECODE_OP_FUSED_GATEUP_T_XQ8)):
            qt, bases = stacked(kind, rows + (ff, ff), K, 11)
            load_qtensor(hip, 1, qt)
            f32map(hip, 0, K + sum(rows) + 3 * ff + 64, x)
            cs = np.cumsum((K,) + rows + (ff, ff))
            hb = [up(hip, [b]) for b in bases]
            hc = [up(hip, [int(c)]) for c in cs[:5]]
            a = up(hip, [0])
            if route == "direct":
                hip.batch_begin()
                (hip.map_fused_qkv_t_xq4_dev if kind == "q4" else hip.map_fused_qkv_t_xq8_dev)(0, 1, a, *hb[:3], *hc[:3], K, *rows)
                (hip.map_fused_gateup_t_xq4_dev if kind == "q4" else hip.map_fused_gateup_t_xq8_dev)(0, 1, a, *hb[3:], *hc[3:], K, ff, ff)
                if kind == "q8":
                    hip.map_fused_gateup_act_t_xq8_dev(0, 1, a, hb[3], hb[4], up(hip, [int(cs[5])]), K, ff)
                hip.batch_end()
            else:
                ops = [A.DecodePlanOp(kind=kq, map_id=0, map_id2=1, h0=a, h1=hb[0], h2=hb[1], h3=hb[2], h4=hc[0], h5=hc[1],
                                      u0=hc[2], u1=K, u2=rows[0], u3=rows[1], u4=rows[2]),
                       A.DecodePlanOp(kind=kg, map_id=0, map_id2=1, h0=a, h1=hb[3], h2=hb[4], h3=hc[3], h4=hc[4], u0=K, u1=ff, u2=ff)]
                if kind == "q8":
                    ops.append(A.DecodePlanOp(kind=A.DECODE_OP_FUSED_GATEUP_ACT_T_XQ8, map_id=0, map_id2=1, h0=a, h1=hb[3], h2=hb[4],
                                              h3=up(hip, [int(cs[5])]), u0=K, u1=ff))
                hip.register_decode_plan(5, ops)
                hip.decode_step(5, 0, 1)
                hip.clear_decode_plan(5)
            res.append(read(hip, 0, K, sum(rows) + 3 * ff))
        got[route] = res
    for d, p in zip(got["direct"], got["plan"]):
        assert np.any(d) and np.array_equal(d.view(np.uint32), p.view(np.uint32))


@pytest.mark.parametrize("kind", ["q4", "q8"])
def test_graph_of_a_fused_qkv_plan_is_dropped_when_its_seventh_handle_is_rewritten(hip, kind):
    """The Q/K/V kinds keep the V result's handle in u0.  A graph recorded one step ahead holds that offset by
    value, so re-uploading the handle between two steps must send the next step through the ordinary replay:
    V lands at the new place from that step on, and the old place is no longer written."""
    K, rows = 1152, (256, 64, 64)
    x = np.random.default_rng(5).standard_normal(K).astype(np.float32)
    qt, bases = stacked(kind, rows, K, 17)
    load_qtensor(hip, 1, qt)
    total = K + sum(rows) + rows[2] + 64
    f32map(hip, 0, total, x)
    cs = np.cumsum((K,) + rows)                    # Q, K, V results back to back; a second V place behind them
    v_old, v_new = int(cs[2]), int(cs[3]) + 32
    hb = [up(hip, [b]) for b in bases]
    hq, hk, hv = up(hip, [int(cs[0])]), up(hip, [int(cs[1])]), up(hip, [v_old])
    a = up(hip, [0])
    kq = A.DECODE_OP_FUSED_QKV_T_XQ4 if kind == "q4" else A.DECODE_OP_FUSED_QKV_T_XQ8
    hip.register_decode_plan(6, [A.DecodePlanOp(kind=kq, map_id=0, map_id2=1, h0=a, h1=hb[0], h2=hb[1], h3=hb[2], h4=hq,
                                                h5=hk, u0=hv, u1=K, u2=rows[0], u3=rows[1], u4=rows[2])])
    try:
        want = None
        for step in range(8):
            note(f"fused qkv plan {kind}, step {step}")
            if step == 4:
                hip.upload_dev(np.array([v_new], np.uint32), handle=hv)
            hip.scatter_contiguous(0, K, np.zeros(total - K, np.float32))
            hip.decode_step(6, step, step + 1)
            out = read(hip, 0, K, total - K)
            v_at_old, v_at_new = out[v_old - K: v_old - K + rows[2]], out[v_new - K: v_new - K + rows[2]]
            if want is None:
                want = v_at_old.copy()
                assert np.any(want)
            if step < 4:
                assert np.array_equal(v_at_old, want) and not np.any(v_at_new), step
            else:
                assert np.array_equal(v_at_new, want) and not np.any(v_at_old), step
    finally:
        hip.clear_decode_plan(6)
