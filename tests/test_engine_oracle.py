"""Harness wiring: the decode harness driving the NumPy op-surface oracle must reproduce the
restated reference forward pass (which never touches the op surface) -- CPU only."""
import numpy as np
import pytest

import oracle
from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd.quant import QTensor
from adam_amd import synth


def dequant_tensors(tensors):
    out = {}
    for n, v in tensors.items():
        out[n] = v.dequant() if isinstance(v, QTensor) else v
    return out


@pytest.mark.parametrize("arch,sched,kv16", [("gemma3", "legacy", False), ("llama", "legacy", True),
                                             ("llama", "level_batched", False), ("gemma3", "level_batched", True)])
def test_engine_matches_forward_cpu(arch, sched, kv16):
    cfg = synth.tiny_config(arch, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    tensors = synth.make_model(cfg, seed=3, sigma=0.3)
    g = oracle.init()
    eng = DecodeEngine(g, cfg, tensors, A=A, kv_cap=32, kv_fp16=kv16, fusion_scheduler_mode=sched,
                       gpu_fused_rows_per_group=64)
    ref = CpuModel(cfg, dequant_tensors(tensors), kv_cap=32, kv_fp16=kv16)
    prompt = [5, 17, 3, 101, 64]
    n_gen = 8
    ref_tokens, margins = ref.generate(prompt, n_gen)
    out, stats = eng.generate(prompt, GenerationConfig(max_tokens=n_gen), forced=ref_tokens)
    # teacher-forced: every step must agree unless the reference's own top-2 margin is at rounding level
    for i, (a, b) in enumerate(zip(out, ref_tokens)):
        assert a == b or margins[i] < 1e-5, (i, a, b, margins[i])
    assert stats['n_gen'] == n_gen and stats['sampling_mode'] == 'gpu_matvec_argmax'
    # last hidden state of the harness vs the reference forward
    hid = eng.read_slot('hidden')
    rel = np.linalg.norm(hid - ref.last_hidden) / np.linalg.norm(ref.last_hidden)
    assert rel < 1e-4, rel


def test_multi_map_split_equals_single_map():
    cfg = synth.tiny_config("llama", n_layer=3, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    tensors = synth.make_model(cfg, seed=4, sigma=0.3)
    outs = []
    for limit in ((1 << 32) - 64, 40000):
        eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=16, q4_map_elem_limit=limit)
        out, _ = eng.generate([1, 2, 3], GenerationConfig(max_tokens=4))
        outs.append((out, len(eng._q4_sizes)))
    assert outs[0][1] == 1 and outs[1][1] > 1
    assert outs[0][0] == outs[1][0]


def test_kv_cap_guard():
    cfg = synth.tiny_config("llama", n_layer=1, n_embd=64, n_head=2, n_head_kv=1, head_dim=32, n_ff=64, n_vocab=64)
    eng = DecodeEngine(oracle.init(), cfg, synth.make_model(cfg, seed=1, sigma=0.3), A=A, kv_cap=8)
    with pytest.raises(RuntimeError, match="KV cache too small"):
        eng.generate([1, 2, 3, 4, 5], GenerationConfig(max_tokens=4))


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_sampled_generation_draws_from_the_top_k_of_the_reference_logits(arch):
    """temperature / top-k / top-p / repeat penalty on the op surface: every drawn token lies in the top k
    of the restated reference forward's logits (after the same penalty), the run is reproducible from
    its seed, and a different seed gives a different continuation."""
    cfg = synth.tiny_config(arch, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    tensors = synth.make_model(cfg, seed=6, sigma=0.3)
    gc = GenerationConfig(max_tokens=10, temperature=4.0, top_k=8, top_p=0.98, repeat_penalty=1.2, seed=123)
    prompt = [5, 17, 3, 101]
    runs = []
    for seed in (123, 123, 7):
        gc.seed = seed
        eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=32, gpu_fused_rows_per_group=32)
        out, stats = eng.generate(prompt, gc)
        assert stats['sampling_mode'] == 'gpu_fused_topk' and len(out) == 10
        runs.append(out)
    assert runs[0] == runs[1] and runs[0] != runs[2]
    ref = CpuModel(cfg, dequant_tensors(tensors), kv_cap=32)
    hist = []                                  # the penalty looks at the generated tokens (repeat_on_prompt is off)
    logits = None
    for i, t in enumerate(prompt):
        logits = ref.forward(int(t), i)
    for step, tok in enumerate(runs[0]):
        lg = np.array(logits, np.float32)
        for r in set(hist[-64:]):
            lg[r] = lg[r] / np.float32(1.2) if lg[r] > 0 else lg[r] * np.float32(1.2)
        top = np.argsort(-lg, kind="stable")[:8]
        assert tok in top, (step, tok, top)
        hist.append(tok)
        logits = ref.forward(tok, len(prompt) + step)


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("chunk", [3, 7, 16])
def test_chunked_prefill_equals_token_by_token(arch, chunk):
    """The prompt run as [m, K] matmuls and m-row norms with attention token by token leaves the same
    KV cache and hidden state as m single-token steps (exactly, on the oracle), also when the last chunk
    is short and when the chunk is longer than the prompt."""
    cfg = synth.tiny_config(arch, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    tensors = synth.make_model(cfg, seed=3, sigma=0.3)
    prompt = [5, 17, 3, 101, 64, 9, 33]
    outs = []
    for m in (0, chunk):
        eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=32, kv_fp16=True, prefill_chunk=m)
        out, _ = eng.generate(prompt, GenerationConfig(max_tokens=6))
        kv = eng.gpu.gather(0, np.arange(eng._kv_start, eng._kv_start + cfg.n_layer * eng._kv_per_layer, dtype=np.uint32))
        outs.append((out, eng.read_slot('hidden'), kv))
    assert outs[0][0] == outs[1][0]
    assert np.array_equal(outs[0][1], outs[1][1]) and np.array_equal(outs[0][2], outs[1][2])


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_batched_lockstep_decode_equals_independent_sequences(arch):
    """Several sequences decoded in lockstep (rows of one [B, K] matmul, own KV cache each) give, on the
    oracle, exactly the tokens of the same prompts decoded one sequence at a time; a batch engine still
    decodes a single sequence."""
    cfg = synth.tiny_config(arch, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    tensors = synth.make_model(cfg, seed=3, sigma=0.3)
    prompts = [[5, 17, 3, 101, 64], [9, 33, 2, 8, 150], [1, 1, 1, 1, 1]]
    singles = []
    for pr in prompts:
        eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=32, kv_fp16=True)
        singles.append(eng.generate(pr, GenerationConfig(max_tokens=6))[0])
    eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=32, kv_fp16=True, batch=4, prefill_chunk=3)
    out, stats = eng.generate_batch(prompts, 6)
    assert out == singles and stats['n_seq'] == 3
    assert eng.generate(prompts[1], GenerationConfig(max_tokens=6))[0] == singles[1]
    with pytest.raises(RuntimeError):
        eng.generate_batch([[1, 2], [3]], 2)
