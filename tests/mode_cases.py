"""Shared by the CPU and the GPU tests of the decode harness's LM-head / sampling modes: the cases, and the
independent restatements they are checked against (the reference forward pass on the dequantised weights,
`oracle/forward_cpu.py`, plus the reference's penalty rule typed out here)."""
import numpy as np

from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd.quant import QTensor
from adam_amd import synth

PROMPT = [5, 17, 3, 101, 64]


def tiny(arch, seed=6):
    cfg = synth.tiny_config(arch, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, n_vocab=160)
    return cfg, synth.make_model(cfg, seed=seed, sigma=0.3)


def dequantised(tensors):
    return {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}


def engine(gpu, cfg, tensors, **kw):
    kw.setdefault("kv_cap", 48)
    kw.setdefault("kv_fp16", True)
    kw.setdefault("gpu_fused_rows_per_group", 32)
    return DecodeEngine(gpu, cfg, tensors, A=A, **kw)


def penalised(logits, generated, penalty):
    """The reference's repeat penalty (engine.py:1960-1967, map_repeat_penalty.comp): the distinct ids among the last
    64 generated tokens; positive logits divided, the others multiplied."""
    lg = np.array(logits, np.float32)
    for t in sorted(set(generated[-64:])):
        lg[t] = lg[t] / np.float32(penalty) if lg[t] > 0 else lg[t] * np.float32(penalty)
    return lg


def greedy_reference(cfg, tensors, prompt, n_gen, penalty=1.0, forced=None):
    """Deterministic decoding restated on the reference forward pass: (tokens, top-two margins)."""
    ref = CpuModel(cfg, dequantised(tensors), kv_cap=len(prompt) + n_gen + 2, kv_fp16=True)
    logits = None
    for i, t in enumerate(prompt):
        logits = ref.forward(int(t), i)
    out, margins, fed = [], [], []
    for step in range(n_gen):
        lg = penalised(logits, fed, penalty) if penalty != 1.0 else np.array(logits, np.float32)
        top2 = np.partition(lg, -2)[-2:]
        out.append(int(np.argmax(lg))); margins.append(float(top2[1] - top2[0]))
        fed.append(out[-1] if forced is None else int(forced[step]))
        logits = ref.forward(fed[-1], len(prompt) + step)
    return out, margins


def agree(got, want, margins, tol=1e-5):
    return all(a == b or m < tol for a, b, m in zip(got, want, margins)) and len(got) == len(want)


SAMPLED = dict(max_tokens=12, temperature=3.0, top_k=8, top_p=0.97, repeat_penalty=1.25, seed=321)
