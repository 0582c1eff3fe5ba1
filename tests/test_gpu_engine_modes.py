"""The decode harness's LM-head / sampling modes and `reuse_prefix` on the HIP library (needs an MI355X): every mode
teacher-forced on the run of the same mode on the NumPy op-surface oracle makes the oracle's choice at every step."""
import numpy as np
import pytest

import oracle
from adam_amd.engine import GenerationConfig
from gpu_util import note, rel_l2
from mode_cases import PROMPT, SAMPLED, tiny, engine

pytestmark = pytest.mark.gpu


def both(hip, cfg, tensors, gc, **kw):
    want, st = engine(oracle.init(), cfg, tensors, **kw).generate(PROMPT, gc)
    dev = engine(hip, cfg, tensors, **kw)
    got, st_dev = dev.generate(PROMPT, gc, forced=want)
    assert st_dev['sampling_mode'] == st['sampling_mode']
    return want, got, st['sampling_mode'], dev


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("mode", ["gpu_argmax", "gpu_topk", "cpu"])
def test_deterministic_modes(hip, arch, mode):
    cfg, tensors = tiny(arch)
    note(f"engine mode {mode} {arch}")
    gc = GenerationConfig(max_tokens=8, top_k=(0 if mode == 'cpu' else 1))
    want, got, m, dev = both(hip, cfg, tensors, gc, sampling_mode=mode, gpu_fused_topk=(mode != 'gpu_topk'))
    assert m == mode and got == want
    # the full logits of the last step (final soft-cap applied) against the oracle engine's
    ref = engine(oracle.init(), cfg, tensors, sampling_mode=mode, gpu_fused_topk=(mode != 'gpu_topk'))
    ref.generate(PROMPT, gc, forced=want)
    assert rel_l2(dev.read_slot('logits'), ref.read_slot('logits')) < 1e-3


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("fused", [True, False])
def test_top1_under_a_repeat_penalty(hip, arch, fused):
    cfg, tensors = tiny(arch)
    note(f"engine top-1 with penalty {arch} fused={fused}")
    want, got, m, _ = both(hip, cfg, tensors, GenerationConfig(max_tokens=10, repeat_penalty=6.0), gpu_fused_topk=fused)
    assert m == ('gpu_fused_topk' if fused else 'gpu_topk') and got == want


@pytest.mark.parametrize("arch,kw", [("llama", dict(gpu_fused_topk=False)), ("gemma3", dict(gpu_fused_topk=False)),
                                     ("llama", dict(gpu_approx_rerank=True, gpu_approx_partial_k=16)),
                                     ("llama", dict(gpu_approx_rerank=True, gpu_approx_partial_k=16, lookahead=False))])
def test_sampled_modes(hip, arch, kw):
    """'gpu_topk' (full logits, penalty, top-k, top-p and the draw in the forward batch) and 'gpu_approx_rerank'
    (partial top-k over the 4-bit copy of the head, shortlist on the host, exact rows over the 8-bit head)."""
    cfg, tensors = tiny(arch)
    note(f"engine sampled {arch} {kw}")
    want, got, m, _ = both(hip, cfg, tensors, GenerationConfig(**SAMPLED), **kw)
    assert m == ('gpu_approx_rerank' if kw.get('gpu_approx_rerank') else 'gpu_topk')
    assert len(set(want)) > 4 and got == want


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
@pytest.mark.parametrize("chunk", [0, 4])
def test_reuse_prefix(hip, arch, chunk):
    cfg, tensors = tiny(arch)
    note(f"engine reuse_prefix {arch} chunk={chunk}")
    gc = GenerationConfig(max_tokens=5)
    eng = engine(hip, cfg, tensors, prefill_chunk=chunk)
    first, _ = eng.generate(PROMPT, gc)
    turn2 = PROMPT + first + [9, 33, 2]
    cont, st = eng.generate(turn2, gc, reuse_prefix=len(PROMPT) + len(first))
    assert (st['n_prompt_reused'], st['n_prompt_prefilled']) == (10, 3)
    hid = eng.read_slot('hidden')
    want, _ = eng.generate(turn2, gc)                      # everything prefilled again
    assert cont == want
    # token-by-token prefill writes the very rows a decode step wrote: same bits; the chunked prefill computes the
    # prompt's rows on the matrix cores, so the two hidden states agree to its tolerance
    h2 = eng.read_slot('hidden')
    assert np.array_equal(hid, h2) if chunk == 0 else rel_l2(hid, h2) < 1e-3
    ref, _ = engine(oracle.init(), cfg, tensors, prefill_chunk=chunk).generate(turn2, gc)
    assert cont == ref
