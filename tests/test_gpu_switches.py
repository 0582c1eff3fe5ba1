"""Every behaviour switch the library reads from the environment, both ways (needs an MI355X).

A switch selects between two code paths that must leave the same results (a folded launch or separate ones, the
grouped attention kernel or the per-head ones, one pass over the LM head for a batch or one per row, ...).  For
each value the whole path runs on a small model of either family -- token-by-token decode from the registered
plan, a prompt in chunks, four sequences in lockstep, and sampled decoding -- against the reference forward pass
and the oracle, to the bars of the default path: tokens equal wherever the reference's own top-two margin is not
at rounding level (1e-4), hidden state within 1e-3 relative L2.  Switches that pick the M = 1 product's kernel
are also run on Llama-3-8B-sized matrices against the oracle."""
import numpy as np
import pytest

import oracle
from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd.quant import QTensor
from adam_amd import quant, synth
from gpu_util import note, rel_l2, up, f32map, read, load_qtensor

pytestmark = pytest.mark.gpu

SWITCHES = [("ADAMAH_NO_FUSE", "1"), ("ADAMAH_PLAN_GRAPH", "0"), ("ADAMAH_GEMV_IMPL", "0"), ("ADAMAH_GEMV_IMPL", "1"), ("ADAMAH_GEMV_IMPL", "3"),
            ("ADAMAH_GLU_SPLIT", "0"), ("ADAMAH_GLU_SPLIT", "2"), ("ADAMAH_GEMM_IMPL", "0"), ("ADAMAH_GEMM_MERGE", "0"), ("ADAMAH_GEMM_SPLITK", "0"), ("ADAMAH_GEMM_EPI", "0"), ("ADAMAH_GEMM_REUSE", "0"), ("ADAMAH_GLU_EMIT", "0"), ("ADAMAH_GEMM_ROWS16", "0"),
            ("ADAMAH_RMSNORM_EMIT", "0"), ("ADAMAH_RMSNORM_ROWS", "0"), ("ADAMAH_ARGMAX_RUN", "0"),
            ("ADAMAH_ATTN_CHUNK", "0"), ("ADAMAH_ATTN_PREFILL_MFMA", "0"), ("ADAMAH_ATTN_PREFILL_MFMA", "2"), ("ADAMAH_ATTN_PREFILL_WPH", "1"), ("ADAMAH_ATTN_PREFILL_WPH", "2"), ("ADAMAH_ATTN_HEADSPLIT", "0"), ("ADAMAH_ATTN_HEADSPLIT", "2"), ("ADAMAH_ATTN_BATCH", "0"), ("ADAMAH_ATTN_MERGE_EMIT", "0"), ("ADAMAH_ATTN_IMPL", "0"), ("ADAMAH_ATTN_ROWPREP", "0"), ("ADAMAH_ROWS_WIDE", "0"), ("ADAMAH_NORM2_PARK", "0"), ("ADAMAH_TOPK_RANK", "0"),
            ("ADAMAH_TOPK_RANK", "1"), ("ADAMAH_TOPK_SELECT", "0"), ("ADAMAH_TOPK_BLOCK", "0")]

_REF = {}


def _reference(arch):
    """Reference runs of the small model, made once per family."""
    if arch not in _REF:
        cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
        tensors = synth.make_model(cfg, seed=5, sigma=0.1)
        deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
        rng = np.random.default_rng(3)
        prompt = [int(t) for t in rng.integers(0, 1000, 40)]
        prompts = [[int(t) for t in rng.integers(0, 1000, 20)] for _ in range(4)]
        one = CpuModel(cfg, deq, kv_cap=96, kv_fp16=True).generate(prompt, 10)
        many = [CpuModel(cfg, deq, kv_cap=64, kv_fp16=True).generate(p, 8) for p in prompts]
        ora = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=96, kv_fp16=True, gpu_fused_rows_per_group=128)
        ora.prefill(prompt)
        gc = GenerationConfig(max_tokens=8, temperature=3.0, top_k=40, top_p=0.97, repeat_penalty=1.3, seed=7)
        sampled, _ = ora.generate(prompt[:6], gc)
        ora.prefill(prompt)
        _REF[arch] = dict(cfg=cfg, tensors=tensors, prompt=prompt, prompts=prompts, one=one, many=many,
                          hidden=ora.read_slot('hidden'), gc=gc, sampled=sampled)
    return _REF[arch]


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("switch,value", SWITCHES)
def test_small_model_paths_with_switch(hip, monkeypatch, arch, switch, value):
    r = _reference(arch)
    monkeypatch.setenv(switch, value)
    note(f"switch {switch}={value} {arch}: decode from the plan")
    cfg, tensors = r["cfg"], r["tensors"]
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=96, kv_fp16=True, gpu_fused_rows_per_group=128)
    dev.prefill(r["prompt"])
    assert rel_l2(dev.read_slot('hidden'), r["hidden"]) < 1e-3
    tok, _ = dev.generate(r["prompt"], GenerationConfig(max_tokens=10), forced=r["one"][0])
    for i in range(10):
        assert tok[i] == r["one"][0][i] or r["one"][1][i] < 1e-4, (i, tok[i], r["one"][0][i], r["one"][1][i])
    note(f"switch {switch}={value} {arch}: sampled")
    stok, _ = dev.generate(r["prompt"][:6], r["gc"], forced=r["sampled"])
    assert stok == r["sampled"]
    note(f"switch {switch}={value} {arch}: prompt in chunks, lockstep batch")
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=96, kv_fp16=True, prefill_chunk=16, batch=4)
    dev.prefill(r["prompt"])
    assert rel_l2(dev.read_slot('hidden'), r["hidden"]) < 1e-3
    out, _ = dev.generate_batch(r["prompts"], 8, forced=[m[0] for m in r["many"]])
    for sq in range(4):
        for i in range(8):
            assert out[sq][i] == r["many"][sq][0][i] or r["many"][sq][1][i] < 1e-4, (sq, i)


@pytest.mark.parametrize("impl", ["0", "1", "3"])
@pytest.mark.parametrize("kind,N,K", [("q4", 4096, 4096), ("q4", 512, 14336), ("q4", 64, 16384), ("q8", 1024, 4096),
                                      ("q8", 256, 14336)])
def test_m1_product_kernels_at_full_row_lengths(hip, monkeypatch, impl, kind, N, K):
    """ADAMAH_GEMV_IMPL picks the kernel of the M = 1 product: activations in LDS (0), in registers (1, the form
    rows longer than 16000 weights take by default), int8 matrix instruction (3, Q4 only: a Q8 map keeps its
    float32 form).  Product and GEMV + argmax against the oracle, inside a batch and outside."""
    monkeypatch.setenv("ADAMAH_GEMV_IMPL", impl)
    rng = np.random.default_rng(N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    qt = quant.quantize_q4_0(w) if kind == "q4" else quant.quantize_q8_0(w)
    x = rng.standard_normal(K).astype(np.float32)
    rpg = 64
    res = {}
    for name, g in (("hip", hip), ("oracle", oracle.init())):
        note(f"GEMV_IMPL={impl} {kind} {N}x{K} on {name}")
        load_qtensor(g, 1, qt)
        f32map(g, 0, K + 2 * N + 3 * (N // rpg) + 8, x)
        mm = g.map_matmul_t_xq4_dev if kind == "q4" else g.map_matmul_t_xq8_dev
        am = g.map_matvec_argmax_t_xq4_dev if kind == "q4" else g.map_matvec_argmax_t_xq8_dev
        ng = N // rpg
        li, lv, lt = K + 2 * N, K + 2 * N + ng, K + 2 * N + 2 * ng
        mm(0, 1, up(g, [0]), up(g, [0]), up(g, [K]), 1, K, N)
        g.batch_begin()
        mm(0, 1, up(g, [0]), up(g, [0]), up(g, [K + N]), 1, K, N)
        am(0, 1, up(g, [0]), up(g, [0]), up(g, np.arange(li, li + ng)), up(g, np.arange(lv, lv + ng)), up(g, [lt]), K, N, rpg)
        g.batch_end()
        res[name] = (read(g, 0, K, N), read(g, 0, K + N, N), read(g, 0, lt, 1)[0], read(g, 0, lv, ng))
    assert rel_l2(res["hip"][0], res["oracle"][0]) < 1e-3
    assert rel_l2(res["hip"][1], res["oracle"][1]) < 1e-3
    assert res["hip"][2] == res["oracle"][2]
    assert rel_l2(res["hip"][3], res["oracle"][3]) < 1e-3


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_row_preparation_and_parked_row_on_a_model_with_wide_heads(hip, monkeypatch, arch):
    """The decode attention launch takes over the token's rotation and KV append only for head sizes 128 and 256, and
    a folded norm pair parks its in-place row only when a later GEMV can put it in place: a small model with 128-wide
    heads decodes the same tokens and ends on the same hidden state (bit for bit) with either turned off, and
    agrees with the reference forward pass."""
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=128, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=6, sigma=0.1)
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    rng = np.random.default_rng(4)
    prompt = [int(t) for t in rng.integers(0, 1000, 37)]
    want = CpuModel(cfg, deq, kv_cap=96, kv_fp16=True).generate(prompt, 10)
    got = {}
    for name, env in (("default", None), ("no_rowprep", "ADAMAH_ATTN_ROWPREP"), ("no_park", "ADAMAH_NORM2_PARK")):
        note(f"wide heads {arch}: {name}")
        if env:
            monkeypatch.setenv(env, "0")
        dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=96, kv_fp16=True, gpu_fused_rows_per_group=128)
        tok, _ = dev.generate(prompt, GenerationConfig(max_tokens=10), forced=want[0])
        got[name] = (tok, dev.read_slot('hidden'), hip.get_last_barrier_count())
        if env:
            monkeypatch.delenv(env)
        for i in range(10):
            assert tok[i] == want[0][i] or want[1][i] < 1e-4, (name, i)
    for name in ("no_rowprep", "no_park"):
        assert got[name][0] == got["default"][0]
        assert np.array_equal(got[name][1].view(np.uint32), got["default"][1].view(np.uint32)), name
    assert got["no_rowprep"][2] == got["default"][2] + cfg.n_layer      # one launch per layer more
