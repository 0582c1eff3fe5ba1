"""Whole decode steps: the harness on the HIP library vs the same harness on the oracle."""
import numpy as np
import pytest

import oracle
from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd.quant import QTensor
from adam_amd import synth
from gpu_util import note, rel_l2

pytestmark = pytest.mark.gpu


def run_pair(hip, cfg, tensors, prompt, n_gen, kv_cap, kv16, sched, rpg=256):
    ref = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=kv_cap, kv_fp16=kv16,
                       fusion_scheduler_mode=sched, gpu_fused_rows_per_group=rpg)
    ref_tok, _ = ref.generate(prompt, GenerationConfig(max_tokens=n_gen))
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=kv_cap, kv_fp16=kv16,
                       fusion_scheduler_mode=sched, gpu_fused_rows_per_group=rpg)
    free_tok, _ = dev.generate(prompt, GenerationConfig(max_tokens=n_gen))
    forced_tok, stats = dev.generate(prompt, GenerationConfig(max_tokens=n_gen), forced=ref_tok)
    return ref, dev, ref_tok, free_tok, forced_tok, stats


@pytest.mark.parametrize("arch,sched,kv16", [("gemma3", "legacy", True), ("llama", "legacy", True),
                                             ("llama", "level_batched", False), ("gemma3", "level_batched", True)])
def test_tiny_models_match_oracle(hip, arch, sched, kv16):
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=5, sigma=0.1)
    note(f"engine tiny {arch} {sched} kv16={kv16}")
    ref, dev, ref_tok, free_tok, forced_tok, stats = run_pair(hip, cfg, tensors, [3, 99, 512, 7, 640, 31], 24, 64,
                                                             kv16, sched, rpg=128)
    assert forced_tok == ref_tok          # teacher-forced: same choice at every step
    assert free_tok == ref_tok            # and free-running on a model with healthy logit gaps
    assert rel_l2(dev.read_slot('hidden'), ref.read_slot('hidden')) < 1e-3
    assert stats['n_gen'] == 24


def test_gemma_shape_two_layers_full_width(hip):
    """Real Gemma-3-1B layer shapes (E=1152, 4/1 heads of 256, FF 6912) with a reduced depth and
    vocabulary so the oracle finishes in seconds."""
    cfg = synth.gemma3_1b_config()
    cfg.n_layer, cfg.n_vocab = 2, 8192
    tensors = synth.make_model(cfg, seed=0, sigma=0.02)
    note("engine gemma-shape 2 layers")
    prompt = list(np.random.default_rng(0).integers(0, cfg.n_vocab, 12))
    ref, dev, ref_tok, free_tok, forced_tok, _ = run_pair(hip, cfg, tensors, prompt, 6, 32, True, "legacy")
    assert rel_l2(dev.read_slot('hidden'), ref.read_slot('hidden')) < 1e-3
    assert forced_tok == ref_tok
    # and against the reference NumPy forward (no op surface involved)
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    cpu = CpuModel(cfg, deq, kv_cap=32, kv_fp16=True)
    cpu_tok, margins = cpu.generate(prompt, 6, forced=ref_tok)
    for i in range(6):
        assert cpu_tok[i] == forced_tok[i] or margins[i] < 1e-5


def test_llama_shape_one_layer_full_width(hip):
    cfg = synth.llama3_8b_config()
    cfg.n_layer, cfg.n_vocab = 1, 4096
    tensors = synth.make_model(cfg, seed=0, sigma=0.02)
    note("engine llama-shape 1 layer")
    prompt = list(np.random.default_rng(1).integers(0, cfg.n_vocab, 8))
    ref, dev, ref_tok, free_tok, forced_tok, _ = run_pair(hip, cfg, tensors, prompt, 4, 16, True, "level_batched")
    assert rel_l2(dev.read_slot('hidden'), ref.read_slot('hidden')) < 1e-3
    assert forced_tok == ref_tok


def test_many_tokens_do_not_exhaust_handles(hip):
    """The tied-embedding fetch creates one gather handle per token (as in the reference, which stops
    after 2048); the library's table is larger so long runs keep working."""
    cfg = synth.tiny_config("gemma3", n_layer=1, n_embd=64, n_head=2, n_head_kv=1, head_dim=32, n_ff=64, n_vocab=64)
    eng = DecodeEngine(hip, cfg, synth.make_model(cfg, seed=2, sigma=0.2), A=A, kv_cap=2600)
    note("2500 decode steps")
    out, _ = eng.generate([1, 2], GenerationConfig(max_tokens=2500))
    assert len(out) == 2500


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_decode_plan_replay_equals_op_by_op(hip, arch):
    """The engine registers its per-token op list as a native decode plan; replaying it must give
    the tokens and the hidden state of issuing the ops one by one."""
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=9, sigma=0.1)
    res = []
    for plan in (True, False):
        note(f"engine {arch} decode_plan={plan}")
        eng = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=64, kv_fp16=True, fusion_scheduler_mode="level_batched",
                           gpu_fused_rows_per_group=128, decode_plan=plan)
        assert (eng._plan_id is not None) == plan
        tok, _ = eng.generate([5, 17, 900, 2], GenerationConfig(max_tokens=16))
        res.append((tok, eng.read_slot('hidden')))
    assert res[0][0] == res[1][0]
    assert np.array_equal(res[0][1], res[1][1])


def _full_model_vs_cpu(hip, cfg, n_prompt, n_gen, seed):
    """Full-size random-init model on the GPU against the reference NumPy forward pass (which never touches
    the op surface): teacher-forced greedy tokens agree wherever the reference's top-two logit gap is
    not at rounding level, and the last step's hidden state and full logits are within 1e-3 relative L2."""
    tensors = synth.make_model(cfg, seed=seed, sigma=0.02)
    prompt = [int(t) for t in np.random.default_rng(seed).integers(0, cfg.n_vocab, n_prompt)]
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    cpu = CpuModel(cfg, deq, kv_cap=n_prompt + n_gen + 2, kv_fp16=True, acc64=False)
    cpu_tok, margins = cpu.generate(prompt, n_gen)
    cpu_hidden, cpu_logits = cpu.last_hidden, cpu.last_raw_logits      # of the last pass (fed the last token)
    del deq, cpu
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=n_prompt + n_gen + 2, kv_fp16=True)
    forced_tok, stats = dev.generate(prompt, GenerationConfig(max_tokens=n_gen), forced=cpu_tok)
    assert stats['n_gen'] == n_gen
    # hidden state and full logits of the last step (the LM head as an ordinary M = 1 product over `normed`)
    fn = hip.map_matmul_t_xq8_dev if dev._kind[dev._lm_name] == 'q8' else hip.map_matmul_t_xq4_dev
    fn(dev.WS_MAP, dev._map_of[dev._lm_name], dev._ws['normed'][0], dev._wh[dev._lm_name], dev._ws['logits'][0], 1,
       cfg.n_embd, cfg.n_vocab)
    assert rel_l2(dev.read_slot('hidden'), cpu_hidden) < 1e-3
    assert rel_l2(dev.read_slot('logits'), cpu_logits) < 1e-3
    agree = [a == b or m < 1e-4 for a, b, m in zip(forced_tok, cpu_tok, margins)]
    assert all(agree), (forced_tok, cpu_tok, margins)
    assert sum(a == b for a, b in zip(forced_tok, cpu_tok)) >= n_gen - 1


def test_gemma3_1b_full_model_tokens_match_reference_forward(hip):
    note("engine gemma-3-1b shape, all 26 layers, vocabulary 262144")
    _full_model_vs_cpu(hip, synth.gemma3_1b_config(), 12, 8, 0)


def test_llama3_8b_full_model_tokens_match_reference_forward(hip):
    note("engine llama-3-8b shape, all 32 layers, Q8_0 head")
    _full_model_vs_cpu(hip, synth.llama3_8b_config(), 4, 3, 0)


@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("arch", ["llama", "gemma3"])
def test_model_read_from_a_gguf_file(hip, arch, mixed, tmp_path):
    """Q4_K, Q4_0 and Q8_0 blocks of a file uploaded in map form (nothing re-quantised) -- and, mixed, a file that
    also holds Q5_0 (as signed 8-bit codes), Q6_K, F16, BF16 and F32 matrices (through the 4-bit map's own
    quantiser, as the reference sends them): the harness on the HIP library follows the harness on the oracle,
    and the restated reference forward over the dequantised weights."""
    from adam_amd import gguf
    from test_gguf_loader import _model_file
    p = tmp_path / f"{arch}.gguf"
    _model_file(str(p), arch, np.random.default_rng(11), mixed=mixed)
    cfg, tensors = gguf.load_model(str(p))
    note(f"engine from gguf {arch}")
    prompt = [5, 17, 3, 90, 44]
    ref, dev, ref_tok, free_tok, forced_tok, _ = run_pair(hip, cfg, tensors, prompt, 8, 32, True, "legacy", rpg=32)
    assert rel_l2(dev.read_slot('hidden'), ref.read_slot('hidden')) < 1e-3
    assert forced_tok == ref_tok
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    cpu = CpuModel(cfg, deq, kv_cap=32, kv_fp16=True)
    cpu_tok, margins = cpu.generate(prompt, 8, forced=ref_tok)
    for i in range(8):
        assert cpu_tok[i] == forced_tok[i] or margins[i] < 1e-5


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_sampled_generation_follows_the_oracle(hip, arch):
    """Sampled decoding (partial top-k with repeat penalty, top-k, soft-cap, top-p, categorical draw, all on
    the device): teacher-forced on the oracle run's tokens and with the same seed, the HIP run draws the
    same token at every step."""
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=5, sigma=0.1)
    gc = GenerationConfig(max_tokens=16, temperature=3.0, top_k=40, top_p=0.97, repeat_penalty=1.3, seed=99)
    prompt = [3, 99, 512, 7, 640, 31]
    ref = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=64, kv_fp16=True, gpu_fused_rows_per_group=128)
    ref_tok, st = ref.generate(prompt, gc)
    assert st['sampling_mode'] == 'gpu_fused_topk' and len(set(ref_tok)) > 4      # not a degenerate distribution
    note(f"engine sampled {arch}")
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=64, kv_fp16=True, gpu_fused_rows_per_group=128)
    dev_tok, _ = dev.generate(prompt, gc, forced=ref_tok)
    assert dev_tok == ref_tok
    for name in ('sample_topk_prob',):
        assert np.allclose(dev.read_slot(name), ref.read_slot(name), atol=1e-4)


@pytest.mark.parametrize("arch,chunk", [("gemma3", 32), ("llama", 32), ("llama", 5)])
def test_chunked_prefill_on_the_matrix_cores(hip, arch, chunk):
    """Prompt in chunks (projections on the fp16 matrix-core matmul, two-term operands) vs the token-by-token
    oracle run: hidden state of the last prompt token within 1e-3 relative L2, then teacher-forced decoding
    agrees wherever the reference's own top-2 margin is not at rounding level."""
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=5, sigma=0.1)
    prompt = [int(t) for t in np.random.default_rng(2).integers(0, 1000, 70)]
    ref = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=96, kv_fp16=True)
    ref.prefill(prompt)
    ref_hidden = ref.read_slot('hidden')
    note(f"engine chunked prefill {arch} chunk={chunk}")
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=96, kv_fp16=True, prefill_chunk=chunk)
    dev.prefill(prompt)
    assert rel_l2(dev.read_slot('hidden'), ref_hidden) < 1e-3
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    cpu = CpuModel(cfg, deq, kv_cap=96, kv_fp16=True)
    ref_tok, margins = cpu.generate(prompt, 8)
    dev_tok, _ = dev.generate(prompt, GenerationConfig(max_tokens=8), forced=ref_tok)
    for i in range(8):
        assert dev_tok[i] == ref_tok[i] or margins[i] < 1e-4, (i, dev_tok[i], ref_tok[i], margins[i])


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_batched_lockstep_decode(hip, arch):
    """Four sequences in lockstep on the HIP library (projections as [4, K] matmuls on the matrix cores,
    attention per sequence): teacher-forced on the reference forward's tokens, every sequence agrees at
    every step unless the reference's own top-2 margin is at rounding level (1e-4, as for bs = 1)."""
    cfg = synth.tiny_config(arch, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
    tensors = synth.make_model(cfg, seed=5, sigma=0.1)
    rng = np.random.default_rng(3)
    prompts = [[int(t) for t in rng.integers(0, 1000, 20)] for _ in range(4)]
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    refs = [CpuModel(cfg, deq, kv_cap=64, kv_fp16=True).generate(p, 10) for p in prompts]
    note(f"engine batched decode {arch}")
    dev = DecodeEngine(hip, cfg, tensors, A=A, kv_cap=64, kv_fp16=True, batch=4, prefill_chunk=16)
    out, stats = dev.generate_batch(prompts, 10, forced=[r[0] for r in refs])
    assert stats['n_seq'] == 4
    for sq in range(4):
        for i in range(10):
            assert out[sq][i] == refs[sq][0][i] or refs[sq][1][i] < 1e-4, (sq, i, out[sq][i], refs[sq][0][i], refs[sq][1][i])


_GRAPH_SNIPPET = """
import sys, json
sys.path.insert(0, {root!r})
import numpy as np
from adam_amd import adamah as A, synth
from adam_amd.engine import DecodeEngine, GenerationConfig
cfg = synth.tiny_config({arch!r}, n_layer=3, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=1000)
tensors = synth.make_model(cfg, seed=5, sigma=0.1)
gpu = A.init()
eng = DecodeEngine(gpu, cfg, tensors, A=A, kv_cap=96, kv_fp16=True)
out = []
for prompt in ([3, 99, 512, 7, 640, 31], [5, 6]):          # a second prompt: the step sequence restarts
    toks, _ = eng.generate(prompt, GenerationConfig(max_tokens=40))
    out.append([int(t) for t in toks])
hid = eng.read_slot('hidden')
gpu.shutdown()
print(json.dumps({{"tokens": out, "hidden": [float(v) for v in hid[:64]]}}))
"""


@pytest.mark.parametrize("arch", ["gemma3", "llama"])
def test_decode_plan_from_recorded_graphs_gives_the_same_tokens(arch):
    """The plan's launches for the next position are recorded into a HIP graph while the current step runs and
    replayed by the next call (ADAMAH_PLAN_GRAPH=0: never).  Two generations (80 graph replays with the token read
    and the embedding upload between them) give the tokens and the final hidden state, bit for bit, of the
    ordinary replay.  Each mode runs in a process of its own, so the library's exit report can be read."""
    import json, os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = {}
    for mode in ("0", "1"):
        note(f"decode plan graphs {arch} mode {mode}")
        env = dict(os.environ, ADAMAH_PLAN_GRAPH=mode, ADAMAH_DEBUG="1")
        p = subprocess.run([sys.executable, "-c", _GRAPH_SNIPPET.format(root=root, arch=arch)], env=env, capture_output=True,
                           text=True, timeout=110)
        assert p.returncode == 0, p.stderr[-2000:]
        res[mode] = json.loads(p.stdout.strip().split("\n")[-1])
        if mode == "1":
            line = [l for l in p.stderr.split("\n") if "steps from graphs" in l]
            assert line and "given up" not in line[-1], p.stderr[-1000:]
            assert int(line[-1].split(":")[1].split()[0]) >= 60, line[-1]       # most steps came from graphs
    assert res["0"]["tokens"] == res["1"]["tokens"]
    assert res["0"]["hidden"] == res["1"]["hidden"]


_GRAPH_STALE_SNIPPET = """
import sys, json
sys.path.insert(0, {root!r})
import numpy as np
from adam_amd import adamah as A
gpu = A.init()
n = 4096
gpu.set_dtype(A.DTYPE_F32)
gpu.map_create(0, 1, 4 * n)
rng = np.random.default_rng(0)
vals = rng.standard_normal(3 * n).astype(np.float32)
gpu.scatter_contiguous(0, 0, vals)
run = lambda lo: np.arange(lo, lo + n, dtype=np.uint32)
a_h, b_h, c_h = (gpu.upload_dev(run(lo))[0] for lo in (0, n, 3 * n))
gpu.register_decode_plan(3, [A.DecodePlanOp(kind=A.DECODE_OP_OP2, map_id=0, op_code=A.OP_ADD, h0=a_h, h1=b_h, h2=c_h, u0=n)])
out = []
for step in range(8):
    if step == 4:
        gpu.upload_dev(run(2 * n), handle=b_h)          # the recorded graph of step 4 still holds the old offset
    if step == 6:
        gpu.map_create(5, 1, 1024)                      # an unrelated map appears: recorded graphs are dropped
    gpu.decode_step(3, step, step + 1)
    got = gpu.gather(0, run(3 * n)).view(np.float32)
    want = vals[:n] + (vals[n:2 * n] if step < 4 else vals[2 * n:])
    out.append(bool(np.array_equal(got, want)))
gpu.shutdown()
print(json.dumps(out))
"""


def test_recorded_graph_is_dropped_when_a_plan_handle_is_rewritten():
    """A graph recorded one step ahead holds operand offsets by value: re-uploading a handle of the plan (or any
    event that may move device buffers) between the recording and the launch must send that step through the
    ordinary replay.  Every step's result is checked."""
    import json, os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    note("decode plan graphs: handle rewritten between record and launch")
    env = dict(os.environ, ADAMAH_PLAN_GRAPH="1", ADAMAH_DEBUG="1")
    p = subprocess.run([sys.executable, "-c", _GRAPH_STALE_SNIPPET.format(root=root)], env=env, capture_output=True, text=True,
                       timeout=110)
    assert p.returncode == 0, p.stderr[-2000:]
    assert json.loads(p.stdout.strip().split("\n")[-1]) == [True] * 8, p.stdout
    line = [l for l in p.stderr.split("\n") if "steps from graphs" in l]
    assert line and int(line[-1].split(":")[1].split()[0]) >= 2, p.stderr[-1000:]      # graphs were in use at all


_GRAPH_SAME_STEP_SNIPPET = """
import sys, json
sys.path.insert(0, {root!r})
import numpy as np
from adam_amd import adamah as A
gpu = A.init()
n = 4096
gpu.set_dtype(A.DTYPE_F32)
gpu.map_create(0, 1, 3 * n)
vals = np.random.default_rng(0).standard_normal(2 * n).astype(np.float32)
gpu.scatter_contiguous(0, 0, vals)
run = lambda lo: np.arange(lo, lo + n, dtype=np.uint32)
a_h, b_h, c_h = (gpu.upload_dev(run(lo))[0] for lo in (0, n, 2 * n))
gpu.register_decode_plan(3, [A.DecodePlanOp(kind=A.DECODE_OP_OP2, map_id=0, op_code=A.OP_ADD, h0=a_h, h1=b_h, h2=c_h, u0=n)])
ok = []
for step in (5, 5, 5, 5, 5, 5, 9, 2, 2):          # a benchmark loop, not a decode loop
    gpu.decode_step(3, step, step + 1)
    ok.append(bool(np.array_equal(gpu.gather(0, run(2 * n)).view(np.float32), vals[:n] + vals[n:])))
gpu.shutdown()
print(json.dumps(ok))
"""


def test_a_plan_called_with_the_same_step_is_not_recorded():
    """Graphs are recorded one step ahead for a caller that walks through positions.  A plan that is called with the same
    (or an unrelated) step every time -- the kernel benchmarks do that -- must not pay for recordings it never uses."""
    import json, os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    note("decode plan graphs: the same step again and again")
    env = dict(os.environ, ADAMAH_DEBUG="1")
    env.pop("ADAMAH_PLAN_GRAPH", None)
    p = subprocess.run([sys.executable, "-c", _GRAPH_SAME_STEP_SNIPPET.format(root=root)], env=env, capture_output=True, text=True,
                       timeout=110)
    assert p.returncode == 0, p.stderr[-2000:]
    assert json.loads(p.stdout.strip().split("\n")[-1]) == [True] * 9, p.stdout
    line = [l for l in p.stderr.split("\n") if "steps from graphs" in l]
    assert line and " 0 steps from graphs" in line[-1] and " 0 instantiations" in line[-1], p.stderr[-1000:]
