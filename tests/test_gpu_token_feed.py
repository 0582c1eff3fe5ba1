"""Token feedback without a host round trip (needs an MI355X): the device-side embedding lookup, the ring tokens
reach the host through, and the greedy loops that run one step ahead of the read-back.

The lookup is checked against the host arithmetic of the dequantising gather (float32 code * scale + zero point,
reference shaders/src/q4/map_gather.comp) times the embedding scale, and against the library's own
gather + scatter + multiply path; the loops against the engine's read-then-issue loops, which in turn are checked
against the oracle elsewhere: same tokens, bit for bit."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd import quant, synth
from gpu_util import note, up, f32map, read, put, load_qtensor

pytestmark = pytest.mark.gpu

ACT, SRC = 8, 9


def _table(kind, V, E, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((V, E), dtype=np.float32)
    if kind == "f32":
        return w, w
    qt = (quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0)(w)
    s, z = qt.qparams()
    codes = qt.codes
    if kind == "q4":
        codes = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(-1)
    deq = (codes.astype(np.float32).reshape(-1, 32) * s[:, None].astype(np.float32) + z[:, None].astype(np.float32))
    return qt, deq.reshape(V, E).astype(np.float32)


@pytest.mark.parametrize("kind", ["f32", "q4", "q8"])
@pytest.mark.parametrize("V,E,m,scale", [(300, 256, 1, 1.0), (300, 256, 5, 16.0), (77, 96, 3, 0.125), (1000, 1152, 16, 33.941125)])
def test_embed_tokens_matches_the_host_lookup(hip, kind, V, E, m, scale):
    note(f"embed_tokens {kind} V={V} E={E} m={m} scale={scale}")
    g = hip
    src, table = _table(kind, V, E, seed=V + E + m)
    row0 = 64                                       # the table does not start at element 0 of its map
    if kind == "f32":
        f32map(g, SRC, row0 + V * E + 32)
        put(g, SRC, row0, src)
    else:
        load_qtensor(g, SRC, src, offset=row0, total=row0 + V * E + 32)
    n_act = 4096 + m * E
    f32map(g, ACT, n_act, np.full(n_act, 7.0, np.float32))
    rng = np.random.default_rng(m)
    toks = rng.integers(0, V, m)
    toks[-1] = V - 1
    # token slots: a run of consecutive elements, and a scattered list (looked up on the device)
    for slots in (np.arange(10, 10 + m), 10 + 3 * rng.permutation(m)):
        put(g, ACT, 0, np.full(4096, 7.0, np.float32))
        for s_, t in zip(slots, toks):
            put(g, ACT, int(s_), np.array([t], np.float32))
        h = up(g, slots)
        dst = 4096
        g.batch_begin()
        g.embed_tokens_dev(ACT, SRC, h, row0, dst, m, E, V, scale)
        g.batch_end()
        got = read(g, ACT, dst, m * E).reshape(m, E)
        want = table[toks] * np.float32(scale)
        assert np.array_equal(got, want)
        assert np.all(read(g, ACT, 0, 10) == 7.0)
        # the form that also hands the token values to the host: same rows, and the tokens under its ticket
        put(g, ACT, dst, np.zeros(m * E, np.float32))
        g.batch_begin()
        ticket = g.embed_post_tokens_dev(ACT, SRC, h, row0, dst, m, E, V, scale)
        g.batch_end()
        assert g.token_wait(ticket, m).tolist() == [float(t) for t in toks]
        assert np.array_equal(read(g, ACT, dst, m * E).reshape(m, E), want)
    # the library's own three-op path leaves the same bits
    locs = (row0 + toks[:, None] * E + np.arange(E)[None, :]).astype(np.uint32).reshape(-1)
    lh = up(g, locs)
    dh = up(g, np.arange(4096, 4096 + m * E))
    put(g, ACT, 100, np.array([scale], np.float32))
    sh = up(g, np.full(m * E, 100))
    put(g, ACT, 4096, np.zeros(m * E, np.float32))
    g.batch_begin()
    src_h, _, _, _ = g.map_gather_dev(SRC, lh, m * E)
    g.map_scatter_dev(ACT, dh, m * E, src_h)
    g.map_broadcast_dev(ACT, A.OP_MUL, dh, sh, dh, m * E)
    g.batch_end()
    assert np.array_equal(read(g, ACT, 4096, m * E).reshape(m, E), got)
    g.map_destroy(ACT); g.map_destroy(SRC)


def test_embed_tokens_out_of_range_token_gives_zeros_and_bad_ranges_are_refused(hip):
    note("embed_tokens: token ids outside the table, destinations outside the map")
    g = hip
    V, E = 50, 64
    w = np.random.default_rng(1).standard_normal((V, E), dtype=np.float32)
    f32map(g, SRC, V * E, w)
    f32map(g, ACT, 1024, np.ones(1024, np.float32))
    put(g, ACT, 0, np.array([-1.0, 50.0, 49.0, 1e9], np.float32))
    h = up(g, [0, 1, 2, 3])
    g.embed_tokens_dev(ACT, SRC, h, 0, 512, 4, E, V, 1.0)
    got = read(g, ACT, 512, 4 * E).reshape(4, E)
    assert np.all(got[0] == 0) and np.all(got[1] == 0) and np.all(got[3] == 0)
    assert np.array_equal(got[2], w[49])
    with pytest.raises(RuntimeError):
        g.embed_tokens_dev(ACT, SRC, h, 0, 1024 - 100, 4, E, V, 1.0)      # rows would end outside map_act
    with pytest.raises(RuntimeError):
        g.embed_tokens_dev(ACT, SRC, h, 64, 512, 4, E, V, 1.0)            # table would end outside map_src
    g.kv_cache_fp16(ACT, 512, 256)
    with pytest.raises(RuntimeError):
        g.embed_tokens_dev(ACT, SRC, h, 0, 512, 4, E, V, 1.0)             # an fp16 KV range cannot take the rows
    g.map_destroy(ACT); g.map_destroy(SRC)


def test_token_ring_hands_over_values_in_order_without_a_stream_sync(hip):
    note("token_post / token_wait")
    g = hip
    f32map(g, ACT, 256, np.arange(256, dtype=np.float32))
    one, many = up(g, [17]), up(g, [200, 3, 99, 100, 101])
    t0 = g.token_post(ACT, one, 1)
    t1 = g.token_post(ACT, many, 5)
    put(g, ACT, 17, np.array([-4.0], np.float32))      # stream order: the first post saw 17.0
    t2 = g.token_post(ACT, one, 1)
    assert (t1, t2) == (t0 + 1, t0 + 2)
    assert g.token_wait(t0, 1).tolist() == [17.0]
    assert g.token_wait(t1, 5).tolist() == [200.0, 3.0, 99.0, 100.0, 101.0]
    assert g.token_wait(t2, 1).tolist() == [-4.0]
    assert g.token_wait(t1, 3).tolist() == [200.0, 3.0, 99.0]      # a slot keeps its values until it is reused
    with pytest.raises(RuntimeError):
        g.token_wait(t2 + 1, 1)                         # not posted: reported once the stream has drained
    with pytest.raises(RuntimeError):
        g.token_wait(t2, 2)                             # more values than were posted
    ts = [g.token_post(ACT, one, 1) for _ in range(9)]  # nine posts: the first one's slot is taken again
    g.sync()                                            # (once all nine have run)
    with pytest.raises(RuntimeError):
        g.token_wait(ts[0], 1)
    assert g.token_wait(ts[8], 1).tolist() == [-4.0]
    with pytest.raises(RuntimeError):
        g.token_post(ACT, many, 63)                     # at most 62 values a post
    g.map_destroy(ACT)


@pytest.mark.parametrize("arch", ["llama", "gemma3"])
def test_greedy_loops_one_step_ahead_give_the_same_tokens(hip, arch):
    note(f"lookahead loops {arch}")
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=11, sigma=0.1)
    rng = np.random.default_rng(2)
    prompt = [int(t) for t in rng.integers(0, 1000, 12)]
    prompts = [[int(t) for t in rng.integers(0, 1000, 9)] for _ in range(4)]
    ora = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=80, kv_fp16=True)
    want, _ = ora.generate(prompt, GenerationConfig(max_tokens=40))
    res = {}
    for la in (False, True):
        eng = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=80, kv_fp16=True, fusion_scheduler_mode="level_batched",
                           prefill_chunk=16, batch=4, lookahead=la)
        assert eng._lookahead == la
        one, st = eng.generate(prompt, GenerationConfig(max_tokens=40))
        # a second run on the same engine
        again, _ = eng.generate(prompt, GenerationConfig(max_tokens=40))
        stop = one[7]
        cut, _ = eng.generate(prompt, GenerationConfig(max_tokens=40, eos_token_ids=(stop,)))
        many, _ = eng.generate_batch(prompts, 24)
        gc = GenerationConfig(max_tokens=24, temperature=2.0, top_k=40, top_p=0.95, repeat_penalty=1.3, seed=5)
        drawn, _ = eng.generate(prompt, gc)          # sampled: the layers run ahead, the LM head waits for the token
        drawn_cut, _ = eng.generate(prompt, GenerationConfig(max_tokens=24, temperature=2.0, top_k=40, top_p=0.95,
                                                             repeat_penalty=1.3, seed=5, eos_token_ids=(drawn[5],)))
        assert drawn_cut == drawn[:drawn.index(drawn[5])]
        res[la] = (one, again, cut, many, drawn)
        assert st["n_gen"] == 40
        assert cut == one[:one.index(stop)]
        del eng
    assert res[True] == res[False]
    assert res[True][0] == res[True][1]
    agree = sum(a == b for a, b in zip(res[True][0], want))
    assert agree >= 39, (agree, res[True][0], want)     # the oracle's loop, up to one rounding-level tie
