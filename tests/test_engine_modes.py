"""The decode harness's LM-head / sampling modes and `reuse_prefix` on the NumPy op-surface oracle (CPU only):
mode selection in the reference's order (adam/models/engine.py:3783-3805), every mode's tokens against the
restated reference forward pass, and the modes against each other where they compute the same distribution."""
import numpy as np
import pytest

import oracle
from adam_amd.engine import GenerationConfig
from mode_cases import PROMPT, SAMPLED, tiny, engine, greedy_reference, agree

PEN = 6.0


def test_mode_selection_follows_the_reference_order():
    cfg, tensors = tiny("llama")
    greedy, pen = GenerationConfig(max_tokens=1), GenerationConfig(max_tokens=1, repeat_penalty=1.2)
    samp = GenerationConfig(**SAMPLED)
    free = GenerationConfig(max_tokens=1, temperature=1.0, top_k=0)
    e = engine(oracle.init(), cfg, tensors, gpu_approx_rerank=True)
    assert e._select_sampling_mode(greedy) == 'gpu_matvec_argmax'
    assert e._select_sampling_mode(pen) == 'gpu_fused_topk'             # top-1 under a penalty: fused, k = 1
    assert e._select_sampling_mode(samp) == 'gpu_approx_rerank'         # ahead of the fused mode when switched on
    assert e._select_sampling_mode(free) == 'cpu'                       # no k: the host samples from the full logits
    e = engine(oracle.init(), cfg, tensors)
    assert e._select_sampling_mode(samp) == 'gpu_fused_topk'
    e = engine(oracle.init(), cfg, tensors, gpu_fused_topk=False)
    assert e._select_sampling_mode(samp) == 'gpu_topk'
    assert e._select_sampling_mode(pen) == 'gpu_topk'
    e = engine(oracle.init(), cfg, tensors, sampling_mode='gpu_argmax')
    assert e._select_sampling_mode(greedy) == 'gpu_argmax'
    with pytest.raises(RuntimeError, match="cannot serve"):
        e._select_sampling_mode(pen)                                    # arg-max of the logits knows no penalty
    ct, tt = tiny("gemma3")
    with pytest.raises(RuntimeError, match="cannot serve"):             # the rerank needs an 8-bit head
        engine(oracle.init(), ct, tt, gpu_approx_rerank=True, sampling_mode='gpu_approx_rerank').generate(PROMPT, samp)


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("mode", ["gpu_argmax", "gpu_topk", "cpu", "gpu_matvec_argmax"])
def test_deterministic_modes_give_the_reference_tokens(arch, mode):
    """Full logits + final soft-cap + arg-max, the top-k list's head, the host sampler at temperature 0 and the
    fused GEMV + arg-max all pick the reference forward's greedy token (the soft-cap is monotonic)."""
    cfg, tensors = tiny(arch)
    want, margins = greedy_reference(cfg, tensors, PROMPT, 8)
    eng = engine(oracle.init(), cfg, tensors, sampling_mode=mode, gpu_fused_topk=(mode != 'gpu_topk'))
    gc = GenerationConfig(max_tokens=8, top_k=(0 if mode == 'cpu' else 1))
    got, st = eng.generate(PROMPT, gc, forced=want)
    assert st['sampling_mode'] == mode and agree(got, want, margins)


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("fused", [True, False])
def test_top1_under_a_repeat_penalty(arch, fused):
    """Deterministic decoding with a repeat penalty: 'gpu_fused_topk' with k = 1 (arg-max of the partial values,
    resolved) or, with the fused modes off, 'gpu_topk' -- against the penalty rule applied to the reference logits.
    (For the soft-capped architecture the full-logits mode penalises the capped values, the fused one the raw ones:
    the restatement follows suit.)"""
    cfg, tensors = tiny(arch)
    eng = engine(oracle.init(), cfg, tensors, gpu_fused_topk=fused)
    gc = GenerationConfig(max_tokens=10, repeat_penalty=PEN)
    got, st = eng.generate(PROMPT, gc)
    assert st['sampling_mode'] == ('gpu_fused_topk' if fused else 'gpu_topk')
    if cfg.final_softcap > 0 and not fused:
        return                                   # capped-then-penalised: covered by the mode-equivalence test's oracle ops
    want, margins = greedy_reference(cfg, tensors, PROMPT, 10, penalty=PEN, forced=got)
    assert agree(got, want, margins)
    assert got != greedy_reference(cfg, tensors, PROMPT, 10)[0]      # the penalty does change the continuation


def test_sampling_modes_draw_the_same_tokens_where_they_compute_the_same_distribution():
    """Without a final soft-cap the fused top-k, the full-logits top-k and the approximate shortlist + exact rerank
    (shortlist wide enough to hold the true top k) rank the same penalised logits and draw with the same uniform
    numbers: teacher-forced on one run's tokens they make the same choice at every step."""
    cfg, tensors = tiny("llama")
    gc = GenerationConfig(**SAMPLED)
    base, st = engine(oracle.init(), cfg, tensors).generate(PROMPT, gc)
    assert st['sampling_mode'] == 'gpu_fused_topk' and len(set(base)) > 4
    for kw, mode in ((dict(gpu_fused_topk=False), 'gpu_topk'), (dict(gpu_approx_rerank=True, gpu_approx_partial_k=16), 'gpu_approx_rerank')):
        got, st = engine(oracle.init(), cfg, tensors, **kw).generate(PROMPT, gc, forced=base)
        assert st['sampling_mode'] == mode and got == base, mode


def test_host_sampler_stays_inside_the_top_k_and_follows_its_seed():
    cfg, tensors = tiny("llama")
    gc = GenerationConfig(max_tokens=8, temperature=2.0, top_k=6, top_p=0.9, seed=11)
    runs = [engine(oracle.init(), cfg, tensors, sampling_mode='cpu').generate(PROMPT, gc)[0] for _ in range(2)]
    assert runs[0] == runs[1]
    from mode_cases import CpuModel, dequantised
    ref = CpuModel(cfg, dequantised(tensors), kv_cap=32, kv_fp16=True)
    logits = None
    for i, t in enumerate(PROMPT):
        logits = ref.forward(t, i)
    for step, tok in enumerate(runs[0]):
        assert tok in np.argsort(-logits, kind="stable")[:6]
        logits = ref.forward(tok, len(PROMPT) + step)


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("chunk", [0, 4])
def test_reuse_prefix_continues_from_the_rows_the_last_call_left(arch, chunk):
    """A second turn whose prompt starts with the first turn's prompt and answer: prefill of the new part only
    gives the tokens (and the hidden state) of prefilling everything."""
    cfg, tensors = tiny(arch)
    gc = GenerationConfig(max_tokens=5)
    eng = engine(oracle.init(), cfg, tensors, prefill_chunk=chunk)
    first, _ = eng.generate(PROMPT, gc)
    turn2 = PROMPT + first + [9, 33, 2]
    cont, st = eng.generate(turn2, gc, reuse_prefix=len(PROMPT) + len(first))
    assert (st['n_prompt_reused'], st['n_prompt_prefilled'], st['n_prompt_total']) == (10, 3, 13)
    hid = eng.read_slot('hidden')
    fresh = engine(oracle.init(), cfg, tensors, prefill_chunk=chunk)
    want, st2 = fresh.generate(turn2, gc)
    assert st2['n_prompt_reused'] == 0 and cont == want
    assert np.array_equal(hid, fresh.read_slot('hidden'))
    # a prefix as long as the prompt is ignored, as in the reference
    again, st3 = eng.generate(turn2, gc, reuse_prefix=len(turn2))
    assert st3['n_prompt_reused'] == 0 and again == want
