"""GQA decode attention through the two reference entry points (scores, softmax.V): HIP vs oracle.

BASELINE config 3: 32 q heads / 8 kv heads, head_dim 128, fp16 KV cache, contexts 1024 / 4096 /
16384, q/K/V ~N(0,1), scale 1/sqrt(128), fp32 softmax; output compared per head (1e-3 rel L2)."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from gpu_util import note, up, f32map, put, read, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def attention_case(g, q, K, V, ctx, cap_len, kv16, scale, softcap):
    """K, V: [Hkv, ctx, d] float32.  Layout as the harness builds it: score rows at element 0 with
    stride cap_len, then q, out, then the KV region [K heads | V heads], each head cap_len rows."""
    Hq, d = q.shape
    Hkv = K.shape[0]
    gs = Hq // Hkv
    sc_sz = Hq * cap_len
    q_pos, out_pos = sc_sz, sc_sz + Hq * d
    kv_start = (out_pos + Hq * d + d - 1) // d * d
    step = cap_len * d
    total = kv_start + 2 * Hkv * step
    f32map(g, 0, total, None)
    if kv16:
        g.kv_cache_fp16(0, kv_start, 2 * Hkv * step)
    put(g, 0, q_pos, q)
    for h in range(Hkv):
        put(g, 0, kv_start + h * step, K[h])
        put(g, 0, kv_start + (Hkv + h) * step, V[h])
    heads = np.arange(Hq) // gs
    q_rows = up(g, q_pos + np.arange(Hq) * d)
    k_locs = up(g, kv_start + heads * step)
    v_locs = up(g, kv_start + (Hkv + heads) * step)
    s_rows = up(g, np.arange(Hq) * cap_len)
    o_rows = up(g, out_pos + np.arange(Hq) * d)
    g.batch_begin()
    g.map_matmul_t_dev(0, q_rows, k_locs, s_rows, 1, d, ctx, Hq)
    g.map_attn_softmax_value_dev(0, s_rows, v_locs, o_rows, Hq, ctx, d, scale, softcap)
    g.batch_end()
    scores = np.stack([read(g, 0, h * cap_len, ctx) for h in range(0, Hq, max(1, Hq // 4))])
    return read(g, 0, out_pos, Hq * d).reshape(Hq, d), scores


@pytest.mark.parametrize("ctx", [1024, 4096, 16384])
def test_config3_gqa_decode_attention_fp16_kv(hip, ctx):
    Hq, Hkv, d = 32, 8, 128
    rng = np.random.default_rng(ctx)
    q = rng.standard_normal((Hq, d)).astype(np.float32)
    K = rng.standard_normal((Hkv, ctx, d), dtype=np.float32)
    V = rng.standard_normal((Hkv, ctx, d), dtype=np.float32)
    outs = []
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"attention ctx={ctx} on {name}")
        outs.append(attention_case(g, q, K, V, ctx, ctx, True, float(1 / np.sqrt(d)), 0.0))
    for h in range(Hq):
        assert rel_l2(outs[0][0][h], outs[1][0][h]) < TOL, h
    assert rel_l2(outs[0][1], outs[1][1]) < 1e-5          # raw q.k score rows
    # the reference NumPy form (engine.py:2428-2441) on fp16-rounded K/V, independent of the op surface
    K16 = K.astype(np.float16).astype(np.float64); V16 = V.astype(np.float16).astype(np.float64)
    for h in (0, 13, 31):
        s = K16[h // 4] @ q[h].astype(np.float64) / np.sqrt(d)
        p = np.exp(s - s.max()); p /= p.sum()
        assert rel_l2(outs[0][0][h], p @ V16[h // 4]) < TOL


@pytest.mark.parametrize("ctx,kv16,softcap,Hq,Hkv,d", [
    (1, True, 50.0, 4, 1, 256), (640, True, 50.0, 4, 1, 256), (1023, False, 0.0, 8, 2, 64),
    (1025, True, 0.0, 8, 2, 64), (2049, False, 30.0, 4, 4, 128), (300, True, 0.0, 6, 2, 96),
    # the grouped kernel's other shapes: one, two and eight query heads per KV head, tile edges, prefetching form
    (17, True, 0.0, 8, 8, 128), (63, True, 20.0, 16, 2, 64), (64, True, 0.0, 4, 2, 256), (65, True, 0.0, 8, 1, 128),
    (1000, True, 0.0, 16, 2, 128), (5000, True, 0.0, 8, 8, 64), (9000, True, 15.0, 16, 2, 64), (3001, True, 0.0, 6, 3, 128),
    (700, True, 0.0, 68, 17, 64)])
def test_attention_variants(hip, ctx, kv16, softcap, Hq, Hkv, d):
    rng = np.random.default_rng(ctx + d)
    q = rng.standard_normal((Hq, d)).astype(np.float32)
    K = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    V = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    outs = []
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"attention variant ctx={ctx} kv16={kv16} cap={softcap} {Hq}/{Hkv}x{d} on {name}")
        outs.append(attention_case(g, q, K, V, ctx, ctx + 7, kv16, float(1 / np.sqrt(d)), softcap)[0])
    for h in range(Hq):
        assert rel_l2(outs[0][h], outs[1][h]) < TOL, h
    if ctx == 1:   # a single key: the output is the (fp16-rounded) V row exactly
        want = V[:, 0].astype(np.float16).astype(np.float32) if kv16 else V[:, 0]
        for h in range(Hq):
            assert np.array_equal(outs[0][h], want[h // (Hq // Hkv)])


def test_gqa_heads_with_equal_queries_agree(hip):
    Hq, Hkv, d, ctx = 8, 2, 128, 1500
    rng = np.random.default_rng(1)
    q = np.repeat(rng.standard_normal((Hkv, d)).astype(np.float32), Hq // Hkv, axis=0)
    K = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    V = rng.standard_normal((Hkv, ctx, d)).astype(np.float32)
    note("gqa equal queries")
    out, _ = attention_case(hip, q, K, V, ctx, ctx, True, float(1 / np.sqrt(d)), 0.0)
    for g0 in range(Hkv):
        for j in range(1, Hq // Hkv):
            assert np.array_equal(out[g0 * 4], out[g0 * 4 + j])


# a chunk's attention: one causal kernel -- or, on the matrix-core form (taken by itself for chunks that fill the chip:
# ADAMAH_ATTN_PREFILL_MFMA=1, the default; forced with 2, off with 0), the pass that arranges the K / V tiles and then the kernel
CHUNK_LAUNCHES = {"0": 1, "2": 2}


@pytest.fixture(params=["0", "2/1", "2/2"], ids=["vector-pv", "matrix-pv", "matrix-pv-two-waves-per-head"])
def chunk_impl(request, monkeypatch):
    """The chunk's attention on vector multiply-adds, on the matrix cores with one wave per head, and with two waves
    per head sharing the key tiles (by itself the form of launches with at most one workgroup per CU)."""
    impl, _, wph = request.param.partition("/")
    monkeypatch.setenv("ADAMAH_ATTN_PREFILL_MFMA", impl)
    if wph:
        monkeypatch.setenv("ADAMAH_ATTN_PREFILL_WPH", wph)
    return impl


def chunk_case(g, q, K, V, seq0, cap_len, scale, softcap, gap=0, one_call=False):
    """m tokens' (scores, softmax.V) pairs in one batch: q [m, Hq, d]; token t sees seq0 + t cache rows.
    Layout: score rows, q [m][Hq][d], out [m][Hq][d] (+ gap floats between tokens), fp16 KV region."""
    m, Hq, d = q.shape
    Hkv = K.shape[0]
    gs = Hq // Hkv
    sc_sz = Hq * cap_len
    q_pos = sc_sz
    out_pos = q_pos + m * Hq * d
    o_stride = Hq * d + gap
    kv_start = (out_pos + m * o_stride + d - 1) // d * d
    step = cap_len * d
    f32map(g, 0, kv_start + 2 * Hkv * step, None)
    g.kv_cache_fp16(0, kv_start, 2 * Hkv * step)
    put(g, 0, q_pos, q)
    for h in range(Hkv):
        put(g, 0, kv_start + h * step, K[h])
        put(g, 0, kv_start + (Hkv + h) * step, V[h])
    heads = np.arange(Hq) // gs
    k_locs, v_locs = up(g, kv_start + heads * step), up(g, kv_start + (Hkv + heads) * step)
    s_rows = up(g, np.arange(Hq) * cap_len)
    qh = [up(g, q_pos + t * Hq * d + np.arange(Hq) * d) for t in range(m)]
    oh = [up(g, out_pos + t * o_stride + np.arange(Hq) * d) for t in range(m)]
    g.batch_begin()
    if one_call:
        g.attn_causal_rows_dev(0, qh, k_locs, s_rows, v_locs, oh, d, seq0, Hq, d, scale, softcap)
    for t in range(0 if one_call else m):
        g.map_matmul_t_dev(0, qh[t], k_locs, s_rows, 1, d, seq0 + t, Hq)
        g.map_attn_softmax_value_dev(0, s_rows, v_locs, oh[t], Hq, seq0 + t, d, scale, softcap)
    g.batch_end()
    launches = g.get_last_barrier_count() if hasattr(g, "get_last_barrier_count") else None
    out = np.stack([read(g, 0, out_pos + t * o_stride, Hq * d).reshape(Hq, d) for t in range(m)])
    scores = np.stack([read(g, 0, h * cap_len, seq0 + m - 1) for h in range(Hq)])
    return out, scores, launches


@pytest.mark.parametrize("m,seq0,Hq,Hkv,d,softcap,gap", [
    (40, 1, 4, 1, 256, 50.0, 0),        # Gemma-3-1B heads, a prompt from position 0, last tile short
    (64, 200, 32, 8, 128, 0.0, 0),      # Llama-3-8B heads, second chunk of a prompt
    (17, 3, 8, 2, 64, 0.0, 8),          # head size 64, padded output rows
    (2, 5, 4, 4, 128, 30.0, 0),         # the shortest run
    (33, 100, 6, 3, 64, 0.0, 0),        # heads not a multiple of four; a quad of waves straddles two KV heads
    (50, 4000, 8, 2, 128, 0.0, 0),      # a short chunk deep into a long context
])
def test_prefill_chunk_is_one_causal_launch(hip, chunk_impl, m, seq0, Hq, Hkv, d, softcap, gap):
    """The per-token pairs of a prompt chunk, issued in one batch, run as one causal launch (behind the pass that
    lays the visible V rows out in tiles for the matrix cores) and give what the oracle gives token by token: outputs per token and head within 1e-3 relative L2, and the score rows
    hold the last token's raw scores."""
    rng = np.random.default_rng(m * 1000 + seq0)
    cap_len = seq0 + m + 7
    q = rng.standard_normal((m, Hq, d)).astype(np.float32)
    K = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    V = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    scale = float(1.0 / np.sqrt(d))
    note(f"attention chunk m={m} seq0={seq0} {Hq}q/{Hkv}kv d={d}")
    out, scores, launches = chunk_case(hip, q, K, V, seq0, cap_len, scale, softcap, gap)
    ref, ref_scores, _ = chunk_case(oracle.init(), q, K, V, seq0, cap_len, scale, softcap, gap)
    assert launches == CHUNK_LAUNCHES[chunk_impl], launches
    for t in range(m):
        for h in range(Hq):
            assert rel_l2(out[t, h], ref[t, h]) < TOL, (t, h)
    assert rel_l2(scores, ref_scores) < 1e-5


def test_causal_rows_entry_point_equals_the_pairs_issued_one_by_one(hip, chunk_impl):
    """adamah_attn_causal_rows_dev (an extension: m pairs in one native call) leaves the words the 2 m calls
    leave, in as many launches; the oracle's form of it agrees within the attention bar; bad arguments fail."""
    rng = np.random.default_rng(77)
    m, seq0, Hq, Hkv, d = 33, 10, 8, 2, 128
    cap_len = seq0 + m + 3
    q = rng.standard_normal((m, Hq, d)).astype(np.float32)
    K = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    V = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    scale = float(1.0 / np.sqrt(d))
    note("attention causal rows entry point")
    a = chunk_case(hip, q, K, V, seq0, cap_len, scale, 20.0, one_call=True)
    b = chunk_case(hip, q, K, V, seq0, cap_len, scale, 20.0)
    assert a[2] == b[2] == CHUNK_LAUNCHES[chunk_impl]
    assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32)) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
    ref = chunk_case(oracle.init(), q, K, V, seq0, cap_len, scale, 20.0, one_call=True)
    assert rel_l2(a[0], ref[0]) < TOL and rel_l2(a[1], ref[1]) < 1e-5
    hip.attn_causal_rows_dev(0, [], 1, 1, 1, [], d, seq0, Hq, d, scale)           # m = 0: nothing to do
    with pytest.raises(RuntimeError):
        hip.attn_causal_rows_dev(0, [987654], 1, 1, 1, [987655], d, seq0, Hq, d, scale)   # unknown handles


@pytest.mark.parametrize("layout,expect", [("hole", 2), ("irregular", 3)])
def test_prefill_chunk_splits_or_falls_back_when_tokens_do_not_line_up(hip, chunk_impl, layout, expect):
    """A hole in the query rows after the third token: two chunk launches.  No common stride at all: the
    tokens pair up (any two tokens have a stride), three launches.  Same results either way."""
    rng = np.random.default_rng(9)
    m, Hq, Hkv, d, seq0 = 6, 4, 2, 128, 4
    cap_len = 32
    q = rng.standard_normal((m, Hq, d)).astype(np.float32)
    K = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    V = rng.standard_normal((Hkv, cap_len, d)).astype(np.float32)
    outs = []
    for g in (hip, oracle.init()):
        note("attention chunk fallback")
        sc_sz = Hq * cap_len
        q_pos = sc_sz
        out_pos = q_pos + (3 * m) * Hq * d
        kv_start = (out_pos + m * Hq * d + d - 1) // d * d
        step = cap_len * d
        f32map(g, 0, kv_start + 2 * Hkv * step, None)
        g.kv_cache_fp16(0, kv_start, 2 * Hkv * step)
        if layout == "hole":
            qoff = [t * Hq * d + (Hq * d if t >= 3 else 0) for t in range(m)]
        else:
            qoff = [2 * t * Hq * d + 8 * t * t for t in range(m)]
        for t in range(m):
            put(g, 0, q_pos + qoff[t], q[t])
        for h in range(Hkv):
            put(g, 0, kv_start + h * step, K[h]); put(g, 0, kv_start + (Hkv + h) * step, V[h])
        heads = np.arange(Hq) // (Hq // Hkv)
        k_locs, v_locs, s_rows = up(g, kv_start + heads * step), up(g, kv_start + (Hkv + heads) * step), up(g, np.arange(Hq) * cap_len)
        g.batch_begin()
        for t in range(m):
            g.map_matmul_t_dev(0, up(g, q_pos + qoff[t] + np.arange(Hq) * d), k_locs, s_rows, 1, d, seq0 + t, Hq)
            g.map_attn_softmax_value_dev(0, s_rows, v_locs, up(g, out_pos + t * Hq * d + np.arange(Hq) * d), Hq, seq0 + t, d,
                                         0.1, 0.0)
        g.batch_end()
        if g is hip:
            assert g.get_last_barrier_count() == expect * CHUNK_LAUNCHES[chunk_impl]
        outs.append(read(g, 0, out_pos, m * Hq * d))
    assert rel_l2(outs[0], outs[1]) < TOL


@pytest.mark.parametrize("B,ctx,Hq,Hkv,d", [(16, 300, 8, 2, 128), (5, 2000, 32, 8, 128), (3, 40, 4, 1, 256)])
def test_lockstep_merge_writes_the_projection_s_operand(hip, monkeypatch, B, ctx, Hq, Hkv, d):
    """The lockstep pairs followed by the O-projection over the heads' outputs as rows [B, Hq d]: with several slices
    of the sequence the merge launch also writes the matmul's fp16 operand form (attention, merge, matmul: 3 launches;
    ADAMAH_ATTN_MERGE_EMIT=0: merge, conversion: 4), every word of outputs and product the same.  One slice: nothing
    to merge, the conversion stays."""
    from adam_amd import quant
    from gpu_util import load_qtensor
    rng = np.random.default_rng(B + ctx)
    gs, N = Hq // Hkv, 64
    scale = float(1.0 / np.sqrt(d))
    q = rng.standard_normal((B, Hq, d)).astype(np.float32)
    K = rng.standard_normal((B, Hkv, ctx, d)).astype(np.float32)
    V = rng.standard_normal((B, Hkv, ctx, d)).astype(np.float32)
    qt = quant.quantize_q4_0(rng.standard_normal((N, Hq * d), dtype=np.float32) * np.float32(0.05))

    def go(g):
        sc_sz = Hq * ctx
        q_pos, out_pos = sc_sz, sc_sz + B * Hq * d
        y_pos = out_pos + B * Hq * d
        kv_start = (y_pos + B * N + d - 1) // d * d
        step = ctx * d
        per_seq = 2 * Hkv * step
        load_qtensor(g, 1, qt)
        f32map(g, 0, kv_start + B * per_seq, None)
        g.kv_cache_fp16(0, kv_start, B * per_seq)
        put(g, 0, q_pos, q)
        for b in range(B):
            put(g, 0, kv_start + b * per_seq, K[b]); put(g, 0, kv_start + b * per_seq + Hkv * step, V[b])
        heads = np.arange(Hq) // gs
        s_rows = up(g, np.arange(Hq) * ctx)
        hs = [(up(g, q_pos + b * Hq * d + np.arange(Hq) * d), up(g, kv_start + b * per_seq + heads * step),
               up(g, kv_start + b * per_seq + (Hkv + heads) * step), up(g, out_pos + b * Hq * d + np.arange(Hq) * d)) for b in range(B)]
        a, w, c = up(g, [out_pos]), up(g, [0]), up(g, [y_pos])
        g.batch_begin()
        for hq, hk, hv, ho in hs:
            g.map_matmul_t_dev(0, hq, hk, s_rows, 1, d, ctx, Hq)
            g.map_attn_softmax_value_dev(0, s_rows, hv, ho, Hq, ctx, d, scale, 0.0)
        g.map_matmul_t_xq4_dev(0, 1, a, w, c, B, Hq * d, N, 1)
        g.batch_end()
        return read(g, 0, out_pos, B * Hq * d + B * N), (g.get_last_barrier_count() if g is hip else None)

    note(f"lockstep merge + projection B={B} ctx={ctx} {Hq}q/{Hkv}kv d={d}")
    fused, n_fused = go(hip)
    monkeypatch.setenv("ADAMAH_ATTN_MERGE_EMIT", "0")
    apart, n_apart = go(hip)
    monkeypatch.delenv("ADAMAH_ATTN_MERGE_EMIT")
    assert np.array_equal(fused.view(np.uint32), apart.view(np.uint32))
    assert (n_fused, n_apart) == ((3, 4) if ctx >= 300 else (3, 3))
    want, _ = go(oracle.init())
    assert rel_l2(fused[:B * Hq * d], want[:B * Hq * d]) < TOL
    assert rel_l2(fused[B * Hq * d:], want[B * Hq * d:]) < TOL


@pytest.mark.parametrize("B,ctx,Hq,Hkv,d,softcap", [(16, 300, 8, 2, 128, 0.0), (3, 40, 4, 1, 256, 50.0), (5, 2000, 32, 8, 128, 0.0)])
def test_lockstep_sequences_are_one_launch(hip, B, ctx, Hq, Hkv, d, softcap):
    """One (scores, softmax.V) pair per sequence of a batch, own queries / outputs / KV cache each, shared
    score rows: on the HIP library one attention launch (plus the merge of the slices when the context
    is long) with the oracle's per-sequence results; the score rows end up holding the last sequence's."""
    rng = np.random.default_rng(B * 100 + ctx)
    gs = Hq // Hkv
    scale = float(1.0 / np.sqrt(d))
    q = rng.standard_normal((B, Hq, d)).astype(np.float32)
    K = rng.standard_normal((B, Hkv, ctx, d)).astype(np.float32)
    V = rng.standard_normal((B, Hkv, ctx, d)).astype(np.float32)
    res = []
    for g in (hip, oracle.init()):
        note(f"attention lockstep B={B} ctx={ctx} {Hq}q/{Hkv}kv d={d}")
        sc_sz = Hq * ctx
        q_pos, out_pos = sc_sz, sc_sz + B * Hq * d
        kv_start = (out_pos + B * Hq * d + d - 1) // d * d
        step = ctx * d
        per_seq = 2 * Hkv * step
        f32map(g, 0, kv_start + B * per_seq, None)
        g.kv_cache_fp16(0, kv_start, B * per_seq)
        put(g, 0, q_pos, q)
        for b in range(B):
            put(g, 0, kv_start + b * per_seq, K[b]); put(g, 0, kv_start + b * per_seq + Hkv * step, V[b])
        heads = np.arange(Hq) // gs
        s_rows = up(g, np.arange(Hq) * ctx)
        g.batch_begin()
        for b in range(B):
            kb = kv_start + b * per_seq
            g.map_matmul_t_dev(0, up(g, q_pos + b * Hq * d + np.arange(Hq) * d), up(g, kb + heads * step), s_rows, 1, d, ctx, Hq)
            g.map_attn_softmax_value_dev(0, s_rows, up(g, kb + (Hkv + heads) * step), up(g, out_pos + b * Hq * d + np.arange(Hq) * d),
                                         Hq, ctx, d, scale, softcap)
        g.batch_end()
        launches = g.get_last_barrier_count() if g is hip else None
        res.append((read(g, 0, out_pos, B * Hq * d).reshape(B, Hq, d), read(g, 0, 0, sc_sz), launches))
    assert res[0][2] in (1, 2), res[0][2]
    for b in range(B):
        for h in range(Hq):
            assert rel_l2(res[0][0][b, h], res[1][0][b, h]) < TOL, (b, h)
    assert rel_l2(res[0][1], res[1][1]) < 1e-5
