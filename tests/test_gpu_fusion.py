"""Ops that the HIP library folds into a neighbouring GEMV launch when they are issued inside a
batch, against the oracle running the same ops one by one (needs an MI355X).

Covered folds: RMSNorm -> GEMV, RMSNorm+residual -> RMSNorm -> GEMV, GEMV -> ADD, GEMV over
[gate; up] rows -> GEGLU/SWIGLU, the combinations of a prologue with an epilogue, RMSNorm ->
GEMV+argmax; sequences of the same ops that are not folded (activation before the GEMV, norm after
it) and sequences that must NOT be folded (aliasing operands).  Every slot an unfused run would
write is compared, because the fused kernels have to leave the maps exactly as the separate ops
would.  Tolerance: 1e-3 relative L2
(the bar for GEMV outputs); the vectors produced by the folded row-wise ops themselves are held
to 1e-5."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd import quant
from gpu_util import note, up, read, rel_l2, load_qtensor, f32map, put

pytestmark = pytest.mark.gpu
TOL = 1e-3


class Slots:
    """Workspace layout shared by the scenarios: named float ranges in map 0, weights in map 1."""

    def __init__(self, K, N):
        self.K, self.N = K, N
        self.off, pos = {}, 0
        for name, n in (("src", K), ("src2", K), ("x", K), ("y", N), ("res", N), ("dst", N), ("nw", K), ("nw2", N),
                        ("resk", K), ("nwk", K), ("idx", 64), ("val", 64), ("tok", 8)):
            self.off[name] = pos
            pos += n + 32          # keep the ranges apart and 32-element aligned
        self.total = pos

    def fill(self, g, rng_seed):
        rng = np.random.default_rng(rng_seed)
        g.set_dtype(A.DTYPE_F32)
        g.map_create(0, 1, self.total)
        vals = {"src": rng.standard_normal(self.K), "src2": rng.standard_normal(self.K),
                "x": rng.standard_normal(self.K), "res": rng.standard_normal(self.N),
                "nw": rng.uniform(0.5, 1.5, self.K), "nw2": rng.uniform(0.5, 1.5, self.N),
                "resk": rng.standard_normal(self.K), "nwk": rng.uniform(0.5, 1.5, self.K)}
        for k, v in vals.items():
            g.scatter_contiguous(0, self.off[k], v.astype(np.float32))

    def h(self, g, name):
        return up(g, [self.off[name]])

    def run(self, g, name, n):
        return up(g, np.arange(self.off[name], self.off[name] + n, dtype=np.uint32))


def make_weights(N, K, seed):
    rng = np.random.default_rng(seed)
    return quant.quantize_q4_0((rng.standard_normal((N, K)) * 0.02).astype(np.float32))


def scenario(g, s, qt, pro, epi, batch=True):
    """pro in (None, 'rms', 'norm2', 'geglu', 'swiglu');
    epi in (None, 'add', 'add_swapped', 'norm_add', 'geglu_after', 'swiglu_after')."""
    K, N = s.K, s.N
    if batch:
        g.batch_begin()
    if pro == 'rms':
        g.map_rmsnorm_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)
    elif pro == 'norm2':
        g.map_rmsnorm_add_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "resk"), s.h(g, "resk"), 1, K, 1e-6)
        g.map_rmsnorm_dev(0, s.h(g, "resk"), s.h(g, "nwk"), s.h(g, "x"), 1, K, 1e-5)
    elif pro in ('geglu', 'swiglu'):
        g.map_op2_dev(0, A.OP_GEGLU if pro == 'geglu' else A.OP_SWIGLU, s.run(g, "src", K), s.run(g, "src2", K),
                      s.run(g, "x", K), K)
    g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "y"), 1, K, N)
    if epi == 'add':
        g.map_op2_dev(0, A.OP_ADD, s.run(g, "res", N), s.run(g, "y", N), s.run(g, "res", N), N)   # in place
    elif epi == 'add_swapped':
        g.map_op2_dev(0, A.OP_ADD, s.run(g, "y", N), s.run(g, "res", N), s.run(g, "dst", N), N)
    elif epi == 'norm_add':
        g.map_rmsnorm_add_dev(0, s.h(g, "y"), s.h(g, "nw2"), s.h(g, "res"), s.h(g, "res"), 1, N, 1e-6)
    elif epi in ('geglu_after', 'swiglu_after'):
        half = N // 2
        g.map_op2_dev(0, A.OP_GEGLU if epi == 'geglu_after' else A.OP_SWIGLU, s.run(g, "y", half),
                      up(g, np.arange(s.off["y"] + half, s.off["y"] + N, dtype=np.uint32)), s.run(g, "dst", half), half)
    if batch:
        g.batch_end()
    return {n: read(g, 0, s.off[n], s.K if n in ("x", "resk") else s.N) for n in ("x", "resk", "y", "res", "dst")}


@pytest.mark.parametrize("K,N", [(1152, 1536), (4096, 4096), (6912, 1152), (2048, 100)])
@pytest.mark.parametrize("pro", [None, 'rms', 'norm2', 'geglu', 'swiglu'])
@pytest.mark.parametrize("epi", [None, 'add', 'add_swapped', 'norm_add', 'geglu_after', 'swiglu_after'])
def test_folded_sequences_match_separate_ops(hip, K, N, pro, epi):
    s = Slots(K, N)
    qt = make_weights(N, K, K + N)
    out = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"fusion {name} K={K} N={N} pro={pro} epi={epi}")
        s.fill(g, 5)
        load_qtensor(g, 1, qt)
        out[name] = scenario(g, s, qt, pro, epi)
    for slot, tol in (("x", 1e-5), ("resk", 1e-5), ("y", TOL), ("res", TOL), ("dst", TOL)):
        assert rel_l2(out["hip"][slot], out["oracle"][slot]) < tol or not np.any(out["oracle"][slot]), slot


def test_folded_equals_unbatched_on_device(hip):
    """The same sequence outside a batch launches the separate kernels; both routes must agree to
    float rounding on every slot."""
    K, N = 4096, 2048
    s = Slots(K, N)
    qt = make_weights(N, K, 3)
    res = []
    for batch in (True, False):
        note(f"fusion batched={batch}")
        s.fill(hip, 9)
        load_qtensor(hip, 1, qt)
        res.append(scenario(hip, s, qt, 'norm2', 'geglu_after', batch=batch))
    for slot in ("x", "resk", "y", "dst"):
        assert rel_l2(res[0][slot], res[1][slot]) < 1e-5, slot


def test_aliasing_sequences_are_not_folded(hip):
    """RMSNorm in place (dst == src) feeding a GEMV, and an ADD whose destination is the GEMV input:
    folding either would race, so they have to run as separate kernels and still be right."""
    K = N = 1024
    s = Slots(K, N)
    qt = make_weights(N, K, 8)
    out = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"fusion aliasing {name}")
        s.fill(g, 13)
        load_qtensor(g, 1, qt)
        g.batch_begin()
        g.map_rmsnorm_dev(0, s.h(g, "x"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)              # in place
        g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "y"), 1, K, N)
        g.map_op2_dev(0, A.OP_ADD, s.run(g, "x", N), s.run(g, "y", N), s.run(g, "x", N), N)   # writes the GEMV input
        g.batch_end()
        out[name] = {n: read(g, 0, s.off[n], K) for n in ("x", "y")}
    assert rel_l2(out["hip"]["y"], out["oracle"]["y"]) < TOL
    assert rel_l2(out["hip"]["x"], out["oracle"]["x"]) < TOL


@pytest.mark.parametrize("case", ["result_on_norm_source", "result_on_residual", "argmax_lists_on_norm_source"])
def test_gemv_result_over_a_prologue_operand_is_not_folded(hip, case):
    """rmsnorm(A -> B); matvec(B -> A): legal as separate ops, but a GEMV that normalised A in every workgroup
    while storing result rows into A would race.  The same for a result that lands on the residual of the
    two-norm prologue, and for partial argmax lists that lie inside the norm's source."""
    K = N = 2048
    s = Slots(K, N)
    qt = make_weights(N, K, 19)
    out = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"fusion aliasing {case} {name}")
        s.fill(g, 17)
        load_qtensor(g, 1, qt)
        g.batch_begin()
        if case == "result_on_norm_source":
            g.map_rmsnorm_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)
            g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "src"), 1, K, N)
        elif case == "result_on_residual":
            g.map_rmsnorm_add_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "resk"), s.h(g, "src2"), 1, K, 1e-6)
            g.map_rmsnorm_dev(0, s.h(g, "src2"), s.h(g, "nwk"), s.h(g, "x"), 1, K, 1e-5)
            g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "resk"), 1, K, N)
        else:
            rpg = 64
            g.map_rmsnorm_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)
            g.map_matvec_argmax_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.run(g, "src", N // rpg),
                                          up(g, np.arange(s.off["src"] + 100, s.off["src"] + 100 + N // rpg, dtype=np.uint32)),
                                          s.h(g, "tok"), K, N, rpg)
        g.batch_end()
        out[name] = {n: read(g, 0, s.off[n], K) for n in ("src", "src2", "x", "resk")}
        out[name]["tok"] = read(g, 0, s.off["tok"], 1)
    for slot in ("src", "src2", "x", "resk"):
        assert rel_l2(out["hip"][slot], out["oracle"][slot]) < TOL, slot
    assert out["hip"]["tok"][0] == out["oracle"]["tok"][0]


@pytest.mark.parametrize("K,N,rpg", [(1152, 4096, 256), (2048, 1000, 64)])
def test_rmsnorm_folded_into_matvec_argmax(hip, K, N, rpg):
    s = Slots(K, N)
    qt = make_weights(N, K, 77)
    n_groups = (N + rpg - 1) // rpg
    assert n_groups <= 64
    tok = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"fusion argmax {name} K={K} N={N}")
        s.fill(g, 21)
        load_qtensor(g, 1, qt)
        g.batch_begin()
        g.map_rmsnorm_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)
        g.map_matvec_argmax_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.run(g, "idx", n_groups), s.run(g, "val", n_groups),
                                      s.h(g, "tok"), K, N, rpg)
        g.batch_end()
        tok[name] = (read(g, 0, s.off["tok"], 1)[0], read(g, 0, s.off["x"], K), read(g, 0, s.off["idx"], n_groups),
                     read(g, 0, s.off["val"], n_groups))
    assert tok["hip"][0] == tok["oracle"][0]
    assert rel_l2(tok["hip"][1], tok["oracle"][1]) < 1e-5
    assert np.array_equal(tok["hip"][2], tok["oracle"][2])
    assert rel_l2(tok["hip"][3], tok["oracle"][3]) < TOL


def test_host_write_between_deferred_ops_keeps_order(hip):
    """A scatter issued between two ops of a batch must land between them (the queue is flushed
    before any other entry point runs)."""
    K, N = 1024, 512
    s = Slots(K, N)
    qt = make_weights(N, K, 4)
    out = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"fusion ordering {name}")
        s.fill(g, 2)
        load_qtensor(g, 1, qt)
        g.batch_begin()
        g.map_rmsnorm_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "x"), 1, K, 1e-6)
        g.scatter_contiguous(0, s.off["x"] + 7, np.array([3.5], np.float32))    # overwrites one normalised value
        g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "y"), 1, K, N)
        g.batch_end()
        out[name] = (read(g, 0, s.off["x"], K), read(g, 0, s.off["y"], N))
    assert out["hip"][0][7] == np.float32(3.5)
    assert rel_l2(out["hip"][0], out["oracle"][0]) < 1e-5
    assert rel_l2(out["hip"][1], out["oracle"][1]) < TOL


@pytest.mark.parametrize("ctx,Hq,Hkv,d,N", [(640, 4, 1, 256, 1152), (3000, 8, 2, 128, 512), (40, 4, 2, 64, 96)])
def test_attention_chain_folded_into_output_projection(hip, ctx, Hq, Hkv, d, N):
    """scores -> softmax.V -> Q4 GEMV over the heads' outputs in one batch: the scores move into the
    softmax.V launch and the merge of the sequence splits into the GEMV's staging.  Raw scores, the
    attention output and the projection are all compared."""
    from gpu_util import f32map, put
    rng = np.random.default_rng(ctx + N)
    q = rng.standard_normal((Hq, d)).astype(np.float32)
    Kc = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    Vc = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    qt = make_weights(N, Hq * d, 31)
    gs = Hq // Hkv
    sc_sz = Hq * ctx
    q_pos, out_pos, y_pos = sc_sz, sc_sz + Hq * d, sc_sz + 2 * Hq * d
    kv_start = (y_pos + N + d - 1) // d * d
    step = ctx * d
    res = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"attention+projection {name} ctx={ctx} {Hq}/{Hkv}x{d} N={N}")
        f32map(g, 0, kv_start + 2 * Hkv * step, None)
        g.kv_cache_fp16(0, kv_start, 2 * Hkv * step)
        put(g, 0, q_pos, q)
        for h in range(Hkv):
            put(g, 0, kv_start + h * step, Kc[h])
            put(g, 0, kv_start + (Hkv + h) * step, Vc[h])
        load_qtensor(g, 1, qt)
        heads = np.arange(Hq) // gs
        s_rows = up(g, np.arange(Hq) * ctx)
        o_rows = up(g, out_pos + np.arange(Hq) * d)
        g.batch_begin()
        g.map_matmul_t_dev(0, up(g, q_pos + np.arange(Hq) * d), up(g, kv_start + heads * step), s_rows, 1, d, ctx, Hq)
        g.map_attn_softmax_value_dev(0, s_rows, up(g, kv_start + (Hkv + heads) * step), o_rows, Hq, ctx, d,
                                     float(1 / np.sqrt(d)), 50.0)
        g.fusion_flush()
        g.map_matmul_t_xq4_dev(0, 1, up(g, [out_pos]), up(g, [0]), up(g, [y_pos]), 1, Hq * d, N)
        g.batch_end()
        res[name] = (read(g, 0, 0, sc_sz), read(g, 0, out_pos, Hq * d), read(g, 0, y_pos, N))
    assert rel_l2(res["hip"][0], res["oracle"][0]) < 1e-5
    assert rel_l2(res["hip"][1], res["oracle"][1]) < TOL
    assert rel_l2(res["hip"][2], res["oracle"][2]) < TOL


# ---- rotation of the new Q / K rows + KV append as one launch ---------------------------------------
def _kv_prep_case(g, style, batch, Hq, Hkv, d, pos, seed, hazard=None):
    """Layout: q | k | v | weights | (gap) | KV cache [K heads | V heads] of `cap` rows each (fp16 mirrored)."""
    cap = 8
    rng = np.random.default_rng(seed)
    qn, kn = Hq * d, Hkv * d
    q = rng.standard_normal(qn).astype(np.float32); k = rng.standard_normal(kn).astype(np.float32)
    v = rng.standard_normal(kn).astype(np.float32)
    wq = rng.uniform(0.5, 1.5, d).astype(np.float32); wk = rng.uniform(0.5, 1.5, d).astype(np.float32)
    q0, k0, v0, w0 = 3, 3 + qn, 3 + qn + kn, 3 + qn + 2 * kn          # odd start: rows need no alignment
    kv_start = (w0 + 2 * d + d - 1) // d * d
    total = kv_start + 2 * Hkv * cap * d
    f32map(g, 0, total, None)
    put(g, 0, q0, np.concatenate([q, k, v, wq, wk]))
    g.kv_cache_fp16(0, kv_start, 2 * Hkv * cap * d)
    spec = []
    for gi in range(Hkv):
        spec += [gi, kv_start // d + gi * cap, gi + Hkv, kv_start // d + (Hkv + gi) * cap]
    hq, hk = up(g, [q0]), up(g, [k0])
    q_rows, k_rows = up(g, q0 + np.arange(Hq) * d), up(g, k0 + np.arange(Hkv) * d)
    hspec, hbase, hdst = up(g, spec), up(g, [k0]), up(g, [q0])
    hwq, hwk = up(g, [w0] * Hq), up(g, [w0 + d] * Hkv)
    if batch:
        g.batch_begin()
    if style == "rope":
        g.map_rope_dev(0, hq, hq, 1, Hq, d, pos, 5e5)
        g.map_rope_dev(0, hk, hk, 1, Hkv, d, pos, 5e5)
    else:
        g.map_qk_norm_rope_x_dev(0, 0, q_rows, hwq, k_rows, hwk, hdst, Hq, d, Hkv, d, pos, 1e6)
    if hazard == "copy_twice":       # second append of the same rows to another position: rides or runs alone
        g.map_row_copy_offset_dev(0, hspec, hbase, pos % cap, 2 * Hkv, d)
        g.map_row_copy_offset_dev(0, hspec, hbase, (pos + 1) % cap, 2 * Hkv, d)
    elif hazard == "rope_after_copy":  # the copy must see the rows before the second rotation
        g.map_row_copy_offset_dev(0, hspec, hbase, pos % cap, 2 * Hkv, d)
        g.map_rope_dev(0, hk, hk, 1, Hkv, d, pos + 1, 5e5)
    elif hazard == "shifted_source":   # source rows straddle two produced rows: no ride
        g.map_row_copy_offset_dev(0, hspec, up(g, [k0 - d // 2]), pos % cap, 2 * Hkv, d)
    else:
        g.map_row_copy_offset_dev(0, hspec, hbase, pos % cap, 2 * Hkv, d)
    launches = None
    if batch:
        g.batch_end()
        launches = g.get_last_barrier_count()
    return read(g, 0, 0, total), launches


@pytest.mark.parametrize("style,Hq,Hkv,d,pos", [("rope", 32, 8, 128, 4095), ("rope", 4, 2, 64, 1), ("qknr", 4, 1, 256, 611),
                                               ("qknr", 8, 4, 128, 77), ("rope", 512, 128, 128, 1030), ("rope", 80, 66, 64, 5)])
@pytest.mark.parametrize("hazard", [None, "copy_twice", "rope_after_copy", "shifted_source"])
def test_kv_prep_run_equals_separate_ops(hip, style, Hq, Hkv, d, pos, hazard):
    """The last two shapes are one token of many sequences at once (the heads of a lockstep batch side by side): more
    rows than a row run holds, taken by the launch that rotates all Q rows, all K rows and appends K and V."""
    note(f"kv prep {style} {Hq}/{Hkv}x{d} pos={pos} hazard={hazard}")
    folded, launches = _kv_prep_case(hip, style, True, Hq, Hkv, d, pos, 11, hazard)
    apart, _ = _kv_prep_case(hip, style, False, Hq, Hkv, d, pos, 11, hazard)
    assert np.array_equal(folded.view(np.uint32), apart.view(np.uint32))
    want, _ = _kv_prep_case(oracle.init(), style, False, Hq, Hkv, d, pos, 11, hazard)
    assert rel_l2(folded, want) < 1e-5
    if hazard is None:
        assert launches == 1          # rotation(s) and append shared one launch
    elif hazard in ("rope_after_copy", "shifted_source"):
        assert launches >= 2          # the dependent op was kept out of the first launch


# ---- the same preparation done by the decode attention launch itself ---------------------------------
def _prep_attn_case(g, style, Hq, Hkv, d, ctx, seed, variant=None, project=False):
    """One decode step's attention inputs, in one batch: rotation of the new Q / K rows (in place), KV append, scores,
    softmax . V (and optionally a Q4 projection of the heads' outputs).  Layout: q | k | v | norm weights | score rows |
    outputs | y | KV cache [K heads | V heads] of ctx + 3 rows each (fp16 mirrored); the cache rows from the new one on
    hold NaN until the append writes them."""
    rng = np.random.default_rng(seed)
    cap, gs, pos, N = ctx + 3, Hq // Hkv, ctx - 1, 256
    qn, kn = Hq * d, Hkv * d
    q0, k0, v0, w0 = 5, 5 + qn, 5 + qn + kn, 5 + qn + 2 * kn
    sc0 = w0 + 2 * d
    out0 = sc0 + Hq * ctx
    y0 = out0 + qn
    kv_start = (y0 + N + d - 1) // d * d
    step = cap * d
    total = kv_start + 2 * Hkv * step
    f32map(g, 0, total, None)
    put(g, 0, q0, np.concatenate([rng.standard_normal(qn + 2 * kn), rng.uniform(0.5, 1.5, 2 * d)]).astype(np.float32))
    g.kv_cache_fp16(0, kv_start, 2 * Hkv * step)
    for h in range(2 * Hkv):
        rows = rng.standard_normal((cap, d)).astype(np.float32)
        rows[pos:] = np.nan
        put(g, 0, kv_start + h * step, rows)
    if project:
        load_qtensor(g, 1, make_weights(N, qn, 41))
    spec = []
    for gi in range(Hkv):
        spec += [gi, kv_start // d + gi * cap, gi + Hkv, kv_start // d + (Hkv + gi) * cap]
    heads = np.arange(Hq) // gs
    hq, hk = up(g, [q0]), up(g, [k0])
    q_rows, k_rows = up(g, q0 + np.arange(Hq) * d), up(g, k0 + np.arange(Hkv) * d)
    s_rows, o_rows = up(g, sc0 + np.arange(Hq) * ctx), up(g, out0 + np.arange(Hq) * d)
    if variant == "scores_over_raw_v":            # the score rows start on the raw V row: the launch must not read it late
        s_rows = up(g, np.concatenate([[v0], sc0 + np.arange(1, Hq) * ctx]))
    g.batch_begin()
    if style == "rope":
        g.map_rope_dev(0, hq, hq, 1, Hq, d, pos, 5e5)
        if variant != "k_not_rotated":
            g.map_rope_dev(0, hk, hk, 1, Hkv, d, pos if variant != "other_position" else pos + 1, 5e5)
    else:
        g.map_qk_norm_rope_x_dev(0, 0, q_rows, up(g, [w0] * Hq), k_rows, up(g, [w0 + d] * Hkv), up(g, [q0]), Hq, d, Hkv, d, pos, 1e6)
    g.map_row_copy_offset_dev(0, up(g, spec), up(g, [k0]), pos, 2 * Hkv, d)
    g.map_matmul_t_dev(0, q_rows, up(g, kv_start + heads * step), s_rows, 1, d, ctx, Hq)
    g.map_attn_softmax_value_dev(0, s_rows, up(g, kv_start + (Hkv + heads) * step), o_rows, Hq, ctx, d, float(1 / np.sqrt(d)), 0.0)
    if project:
        g.map_matmul_t_xq4_dev(0, 1, up(g, [out0]), up(g, [0]), up(g, [y0]), 1, qn, N)
    g.batch_end()
    launches = g.get_last_barrier_count() if hasattr(g, "get_last_barrier_count") else None
    m = read(g, 0, 0, total)
    # the untouched NaN rows of the cache (beyond the new row) stay out of the comparison of values
    keep = np.ones(total, bool)
    for h in range(2 * Hkv):
        keep[kv_start + h * step + (pos + 1) * d: kv_start + (h + 1) * step] = False
    return m, keep, launches


@pytest.mark.parametrize("style,Hq,Hkv,d,ctx,project", [("rope", 32, 8, 128, 4096, False), ("rope", 32, 8, 128, 4096, True),
                                                        ("rope", 8, 2, 128, 17, False), ("rope", 8, 8, 128, 300, True),
                                                        ("qknr", 4, 1, 256, 612, True), ("qknr", 8, 4, 128, 1, False),
                                                        ("qknr", 16, 2, 256, 2500, False)])
def test_kv_prep_inside_the_attention_launch(hip, monkeypatch, style, Hq, Hkv, d, ctx, project):
    note(f"kv prep in attention {style} {Hq}/{Hkv}x{d} ctx={ctx} project={project}")
    inside, keep, n_in = _prep_attn_case(hip, style, Hq, Hkv, d, ctx, 19, project=project)
    monkeypatch.setenv("ADAMAH_ATTN_ROWPREP", "0")
    apart, _, n_out = _prep_attn_case(hip, style, Hq, Hkv, d, ctx, 19, project=project)
    monkeypatch.delenv("ADAMAH_ATTN_ROWPREP")
    assert n_in == n_out - 1                      # the preparation cost no launch of its own
    assert not np.isnan(inside[keep]).any()
    assert np.array_equal(inside.view(np.uint32), apart.view(np.uint32))
    want, _, _ = _prep_attn_case(oracle.init(), style, Hq, Hkv, d, ctx, 19, project=project)
    assert rel_l2(inside[keep], want[keep]) < (TOL if project else 1e-5)
    # a second step on the same stream: the tickets of the first were handed back
    again, _, _ = _prep_attn_case(hip, style, Hq, Hkv, d, ctx, 19, project=project)
    assert np.array_equal(inside.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("variant", ["k_not_rotated", "other_position", "scores_over_raw_v"])
def test_kv_prep_that_is_not_the_attention_s_own_stays_a_launch(hip, monkeypatch, variant):
    """Row ops before the pair that are not exactly the preparation of its operands (or whose rows the pair writes)."""
    note(f"kv prep not folded: {variant}")
    got, keep, n_in = _prep_attn_case(hip, "rope", 8, 2, 128, 200, 23, variant=variant)
    monkeypatch.setenv("ADAMAH_ATTN_ROWPREP", "0")
    apart, _, n_out = _prep_attn_case(hip, "rope", 8, 2, 128, 200, 23, variant=variant)
    monkeypatch.delenv("ADAMAH_ATTN_ROWPREP")
    assert n_in == n_out
    assert np.array_equal(got.view(np.uint32), apart.view(np.uint32))
    want, _, _ = _prep_attn_case(oracle.init(), "rope", 8, 2, 128, 200, 23, variant=variant)
    assert rel_l2(got[keep], want[keep]) < 1e-5


# ---- the in-place row of a folded norm + residual pair, parked until a later GEMV puts it in place ----
def _norm2_then(g, s, qt, then):
    """norm + residual (in place unless then == 'apart'), norm, GEMV in one batch, followed by `then`:
    'gemv': a second GEMV that does not touch the residual (puts the parked row in place);
    'gemv_reads_row': a second GEMV whose activations are that row; 'op_reads_row': an add over it, then the GEMV;
    'apart': the first norm's result goes to its own place; 'nothing': the batch ends."""
    K, N = s.K, s.N
    t_dst = "src2" if then == "apart" else "resk"
    g.batch_begin()
    g.map_rmsnorm_add_dev(0, s.h(g, "src"), s.h(g, "nw"), s.h(g, "resk"), s.h(g, t_dst), 1, K, 1e-6)
    g.map_rmsnorm_dev(0, s.h(g, t_dst), s.h(g, "nwk"), s.h(g, "x"), 1, K, 1e-5)
    g.map_matmul_t_xq4_dev(0, 1, s.h(g, "x"), up(g, [0]), s.h(g, "y"), 1, K, N)
    if then == "op_reads_row":
        g.map_op2_dev(0, A.OP_ADD, s.run(g, "resk", K), s.run(g, "x", K), s.run(g, "src2", K), K)
    if then != "nothing":
        second_x = "resk" if then == "gemv_reads_row" else "x"
        g.map_matmul_t_xq4_dev(0, 1, s.h(g, second_x), up(g, [0]), s.h(g, "dst"), 1, K, N)
    g.batch_end()
    launches = g.get_last_barrier_count() if hasattr(g, "get_last_barrier_count") else None
    return read(g, 0, 0, s.total), launches


@pytest.mark.parametrize("then", ["gemv", "gemv_reads_row", "op_reads_row", "apart", "nothing"])
@pytest.mark.parametrize("K,N", [(1152, 1536), (4096, 1024)])
def test_norm2_row_parked_until_a_later_gemv(hip, monkeypatch, K, N, then):
    s = Slots(K, N)
    qt = make_weights(N, K, 17)
    got = {}
    for name, g in (("park", hip), ("ticket", hip), ("oracle", oracle.init())):
        note(f"norm2 then {then} K={K} N={N} {name}")
        if name == "ticket":
            monkeypatch.setenv("ADAMAH_NORM2_PARK", "0")
        s.fill(g, 29)
        load_qtensor(g, 1, qt)
        got[name] = _norm2_then(g, s, qt, then)
        if name == "ticket":
            monkeypatch.delenv("ADAMAH_NORM2_PARK")
    assert np.array_equal(got["park"][0].view(np.uint32), got["ticket"][0].view(np.uint32))
    assert got["park"][1] == got["ticket"][1]       # parking costs no launch
    assert rel_l2(got["park"][0], got["oracle"][0]) < TOL
    for slot in ("resk", "x", "src2"):
        o = s.off[slot]
        assert rel_l2(got["park"][0][o:o + K], got["oracle"][0][o:o + K]) < 1e-5, slot
