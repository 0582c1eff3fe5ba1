"""Whole decode steps at the contexts and widths the benchmark configurations name, against the restated
reference forward pass (oracle/forward_cpu.py, which never touches the op surface).

The KV caches of both sides are preloaded with the same seeded fp16-exact K / V rows, so a step at position
4095 (bs = 1) or 1023 (16 sequences in lockstep) costs the CPU side one forward pass instead of thousands.
Layer count and, for the batched case, vocabulary are reduced; every matrix keeps the Llama-3-8B width.
Bars: hidden state and full logits within 1e-3 relative L2, greedy token equal unless the reference's own
top-two margin is below 1e-4."""
import numpy as np
import pytest

from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine
from adam_amd.quant import QTensor
from adam_amd import synth
from gpu_util import note, rel_l2

pytestmark = pytest.mark.gpu


def device_logits(eng, src_h=None):
    """Full logits of the vector in the `normed` slot (or at handle src_h) through the ordinary M = 1 product."""
    c, g = eng.cfg, eng.gpu
    fn = g.map_matmul_t_xq8_dev if eng._kind[eng._lm_name] == 'q8' else g.map_matmul_t_xq4_dev
    fn(eng.WS_MAP, eng._map_of[eng._lm_name], src_h or eng._ws['normed'][0], eng._wh[eng._lm_name], eng._ws['logits'][0],
       1, c.n_embd, c.n_vocab)
    return eng.read_slot('logits')


def preload_kv(eng, cpu, n_rows, seed, seq=0):
    """The same fp16-exact N(0, 1) rows at positions 0 .. n_rows-1 of every layer's K and V cache on both sides."""
    c = eng.cfg
    rng = np.random.default_rng(seed)
    for L in range(c.n_layer):
        for which, base in (("k", eng._k_base_s[seq][L]), ("v", eng._v_base_s[seq][L])):
            rows = rng.standard_normal((c.n_head_kv, n_rows, c.head_dim_kv)).astype(np.float16).astype(np.float32)
            (cpu.k_cache if which == "k" else cpu.v_cache)[L, :, :n_rows, :] = rows
            for h in range(c.n_head_kv):
                eng.gpu.scatter_contiguous(eng.WS_MAP, base + h * eng._kv_step, np.ascontiguousarray(rows[h]).reshape(-1))


def dequantised(tensors):
    return {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}


def check_step(dev_hidden, dev_logits, dev_token, cpu, cpu_logits):
    assert rel_l2(dev_hidden, cpu.last_hidden) < 1e-3
    assert rel_l2(dev_logits, cpu.last_raw_logits) < 1e-3
    top2 = np.partition(cpu_logits, -2)[-2:]
    assert dev_token == int(np.argmax(cpu_logits)) or float(top2[1] - top2[0]) < 1e-4


def test_llama3_8b_shape_decode_step_at_position_4095(hip):
    """BASELINE config 4's context: bs = 1 step over 4095 cached positions -- the sequence is split over
    slices, the slice merge is folded into the O-projection, the head is Q8_0 over the full vocabulary."""
    cfg = synth.llama3_8b_config()
    cfg.n_layer = 2
    tensors = synth.make_model(cfg, seed=3, sigma=0.02)
    cpu = CpuModel(cfg, dequantised(tensors), kv_cap=4100, kv_fp16=True)
    note("llama-3-8b width, 2 layers, bs=1 step at position 4095")
    eng = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=4100, kv_fp16=True, fusion_scheduler_mode="level_batched")
    preload_kv(eng, cpu, 4095, seed=7)
    tok = 1234
    cpu_logits = cpu.forward(tok, 4095)
    eng._forward(tok, 4095)
    check_step(eng.read_slot('hidden'), device_logits(eng), eng.read_token(), cpu, cpu_logits)
    # the op-by-op path (no decode plan: what an unchanged reference engine issues) gives the same step
    eng2 = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=4100, kv_fp16=True, decode_plan=False)
    cpu2 = CpuModel(cfg, cpu.t, kv_cap=4100, kv_fp16=True)
    preload_kv(eng2, cpu2, 4095, seed=7)
    eng2._forward(tok, 4095)
    check_step(eng2.read_slot('hidden'), device_logits(eng2), eng2.read_token(), cpu, cpu_logits)
    # the next step fed from the device (the token the LM head just left in its slot, its embedding row gathered
    # from the table on the device, the token handed to the host by that launch) against the same step fed from the
    # host: same token reported, same hidden state, same choice
    nt = eng2.read_token()
    note("the step at position 4096 fed from the device")
    eng2._forward(None, 4096, from_device=True)
    assert eng2._wait_tokens(eng2._feed_ticket) == [nt]
    h_dev, t_dev = eng2.read_slot('hidden'), eng2.read_token()
    eng2._forward(nt, 4096)
    assert np.array_equal(h_dev, eng2.read_slot('hidden'))
    assert t_dev == eng2.read_token()


def _full_depth_step(hip, cfg, ctx, seed, tok):
    """One decode step of the full-size model at position `ctx` over preloaded caches: from the decode plan (the
    launches the benchmark times) and again with every op issued by itself, each against the reference forward."""
    tensors = synth.make_model(cfg, seed=seed, sigma=0.02)
    cpu = CpuModel(cfg, dequantised(tensors), kv_cap=ctx + 4, kv_fp16=True, acc64=False)
    eng = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=ctx + 4, kv_fp16=True, fusion_scheduler_mode="level_batched")
    assert eng._plan_id is not None
    preload_kv(eng, cpu, ctx, seed=seed + 4)
    cpu_logits = cpu.forward(tok, ctx)
    eng._forward(tok, ctx)
    check_step(eng.read_slot('hidden'), device_logits(eng), eng.read_token(), cpu, cpu_logits)
    plan_id, eng._plan_id = eng._plan_id, None          # the same step op by op (rows of position ctx written again)
    try:
        note("... the same step op by op")
        eng._forward(tok, ctx)
        check_step(eng.read_slot('hidden'), device_logits(eng), eng.read_token(), cpu, cpu_logits)
    finally:
        eng._plan_id = plan_id


def test_llama3_8b_all_32_layers_at_position_4095(hip):
    """BASELINE config 4 at full depth and full context together: 32 layers of slice merges over 4095 cached
    positions, Q8_0 head over the whole vocabulary, one reference pass on the CPU."""
    note("llama-3-8b shape, all 32 layers, bs=1 step at position 4095")
    _full_depth_step(hip, synth.llama3_8b_config(), 4095, seed=6, tok=4321)


def test_gemma3_1b_all_26_layers_at_position_639(hip):
    """BASELINE config 2's last position (512-token prompt + 128 tokens): 26 layers, one KV head of 256, attention
    soft-cap on, tied Q4_0 head over 262144 rows."""
    note("gemma-3-1b shape, all 26 layers, bs=1 step at position 639")
    _full_depth_step(hip, synth.gemma3_1b_config(), 639, seed=8, tok=98765)


def test_llama3_8b_shape_chunk_of_512_rows_and_16_sequences_in_lockstep(hip):
    """BASELINE config 5 at full width, one layer: a 512-token prompt chunk (projections as [512, K] matmuls,
    one causal attention launch) against 512 token-by-token reference passes, then one lockstep step of 16
    sequences at position 1023 over their own preloaded caches against 16 reference passes."""
    cfg = synth.llama3_8b_config()
    cfg.n_layer, cfg.n_vocab = 1, 16384
    tensors = synth.make_model(cfg, seed=4, sigma=0.02)
    deq = dequantised(tensors)
    B, ctx = 16, 1023
    eng = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=1032, kv_fp16=True, fusion_scheduler_mode="level_batched",
                       prefill_chunk=512, batch=B)
    # --- the chunk
    rng = np.random.default_rng(11)
    prompt = [int(t) for t in rng.integers(0, cfg.n_vocab, 512)]
    cpu = CpuModel(cfg, deq, kv_cap=520, kv_fp16=True, acc64=False)      # float32 BLAS: 512 passes in seconds
    for i, t in enumerate(prompt):
        cpu_logits = cpu.forward(t, i)
    note("llama-3-8b width, 1 layer, 512-row chunk")
    eng.reset()
    eng._forward_chunk(prompt, 0)
    check_step(eng.read_slot('hidden'), device_logits(eng), eng.read_token(), cpu, cpu_logits)
    # --- 16 sequences, one step at position 1023
    cpus = []
    for sq in range(B):
        m = CpuModel(cfg, deq, kv_cap=1032, kv_fp16=True)
        preload_kv(eng, m, ctx, seed=100 + sq, seq=sq)
        cpus.append(m)
    feed = [int(t) for t in rng.integers(0, cfg.n_vocab, B)]
    want = [m.forward(feed[sq], ctx) for sq, m in enumerate(cpus)]
    note("llama-3-8b width, 1 layer, 16 sequences in lockstep at position 1023")
    eng._forward_chunk(feed, ctx, lockstep=True)
    toks = eng.read_tokens(B)
    E = cfg.n_embd
    hid = hip.gather(eng.WS_MAP, np.arange(eng._cp['hidden'], eng._cp['hidden'] + B * E, dtype=np.uint32)).view(np.float32)
    for sq in range(B):
        logits = device_logits(eng, eng._c_n1[sq])
        check_step(hid[sq * E:(sq + 1) * E], logits, toks[sq], cpus[sq], want[sq])
