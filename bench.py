#!/usr/bin/env python3
"""Benchmark of the quantized decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b|gemma3-1b] [--only LEG]

A "step" is one bs=1 greedy decode step (embedding fetch, all layers, fused LM-head GEMV+argmax,
token read-back) of a random-init Q4_0 model of the named architecture, issued through the
ADAMAH op surface exactly as the decode harness does.  The default workload is the Llama-3-8B
shape with a Q8_0 output head; its prompt is sized so that the last timed step runs at context
4096.  W untimed steps follow the prompt prefill, then exactly K steps are timed between two
device synchronisations; weights, KV cache and activations are resident in HBM before the timed
region starts.  The timed region is run three times over the same positions and the median run is
reported (the reference's protocol: one cold run, one warm-up, median of three steady runs).

One JSON line is printed.  Besides the contract keys it carries
  op_by_op      the same decode with every op of a step issued as its own call (no decode plan):
                what an engine that never registers a plan gets from this library
  config2_gemma3_1b  the Gemma-3-1B-shape decode (128 steps after a 512-token prompt), plan and op by op
  config5_batched    16 prompts of 1024 tokens prefilled in chunks of 512, then 128 lockstep steps
  gemm_q4_0     the batched Q4_0 matmul (M = 16, 512) at the Llama-3-8B shapes
  roofline      the Q4_0 GEMV kernel at the Llama-3-8B gate+up shape (28672x4096), timed with HIP
                events on the library's stream while cycling through > 1 GB of distinct weights
  gemv_shapes   the same measurement for the other Llama-3-8B GEMV shapes
  attention_32q8kv_d128  GQA decode attention over an fp16 KV cache at context 1024 / 4096 / 16384
  cpu_baseline  the NumPy restatement of the reference forward pass (float32 BLAS, pre-dequantised
                weights) timed on this host on a bounded sample of the same workload: a few steps at
                the GPU leg's context over caches preloaded with random rows
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
LLAMA_GEMV_SHAPES = [(28672, 4096), (14336, 4096), (6144, 4096), (4096, 4096), (4096, 14336)]
CONFIG1_GEMV_SHAPE = (6912, 1152)      # BASELINE config 1 (Gemma-3-1B FFN up): launch-bound, reported beside the others
# HBM bytes per 28672x4096 Q4_0 GEMV launch from rocprofv3 --pmc (profiles/gemv_q4_0_llama_shapes_pmc_
# fetch_write.txt): FETCH_SIZE 33,535.3 counts x 1.999 KiB (factor from a plain read kernel of known
# size) + WRITE_SIZE 112.2 counts x 1.000 KiB (factor from a plain copy kernel).
GEMV_TRAFFIC_BYTES = int(33535.3 * 1.999 * 1024 + 112.2 * 1.000 * 1024)
GEMV_TRAFFIC_SOURCE = ("profiles/gemv_q4_0_llama_shapes_pmc_fetch_write.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                       "`bench.py --only gemv`, scaled by the same counters of `bench.py --only probe`; a figure of that "
                       "profile, not of this run")
METRIC = "decode tok/s at bs=1 + Q4 GEMV achieved HBM GB/s (% of MI355X peak)"


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def gemv_bytes(N, K):
    """Algorithmic bytes of one Q4_0 GEMV launch: 18 B per 32 weights + x + y."""
    return N * K * 18 // 32 + 4 * K + 4 * N


def measure_gemv(gpu, A, shapes, rounds=6):
    """HBM GB/s of the Q4_0 GEMV at each shape.  A 1.88 G-element Q4 map (1.06 GB of codes + scales)
    is carved into as many distinct [N, K] matrices as fit; each round launches every one of them
    once through a registered decode plan (one host call per round), so consecutive launches
    never touch the same weights and the 256 MB last-level cache cannot serve them."""
    wmap, amap, plan_id = 3, 5, 7
    total = 16 * 28672 * 4096
    rng = np.random.default_rng(123)
    gpu.map_create_typed(wmap, A.DTYPE_Q4, 1, total, 32)
    s = rng.uniform(0.001, 0.01, total // 32).astype(np.float16).astype(np.float32)
    gpu.set_qparams(wmap, s, np.float32(-8.0) * s)
    chunk = 1 << 26
    for b in range(0, total // 2, chunk):
        n = min(chunk, total // 2 - b)
        gpu.scatter_q4_packed_contiguous(wmap, 2 * b, rng.integers(0, 256, n, dtype=np.uint8), n_locs=2 * n)
    assert gpu.map_layout(wmap) == 1
    kmax = max(k for _, k in shapes); nmax = max(n for n, _ in shapes)
    gpu.set_dtype(A.DTYPE_F32)
    gpu.map_create(amap, 1, kmax + nmax)
    gpu.scatter_contiguous(amap, 0, rng.standard_normal(kmax).astype(np.float32))
    a_h = gpu.upload_dev(np.array([0], np.uint32))[0]
    c_h = gpu.upload_dev(np.array([kmax], np.uint32))[0]
    out = {}
    for N, K in shapes:
        n_mats = total // (N * K)
        ops = []
        for i in range(n_mats):
            b_h = gpu.upload_dev(np.array([i * N * K], np.uint32))[0]
            ops.append(A.DecodePlanOp(kind=A.DECODE_OP_MATMUL_T_XQ4, map_id=amap, map_id2=wmap,
                                      h0=a_h, h1=b_h, h2=c_h, u0=1, u1=K, u2=N, u3=1))
        gpu.register_decode_plan(plan_id, ops)
        gpu.decode_step(plan_id, 0, 0)
        gpu.sync()
        gpu.timer_begin()
        for _ in range(rounds):
            gpu.decode_step(plan_id, 0, 0)
        ms = gpu.timer_end()
        gpu.clear_decode_plan(plan_id)
        us = ms * 1e3 / (rounds * n_mats)
        gbps = gemv_bytes(N, K) / (us * 1e-6) / 1e9
        out[f"{N}x{K}"] = {"us_per_launch": round(us, 3), "GB/s": round(gbps, 1),
                           "frac": round(gbps / HBM_PEAK_GBPS, 4), "launches": rounds * n_mats,
                           "distinct_MB": round(n_mats * N * K * 18 / 32 / 1e6)}
        log(f"gemv {N}x{K}: {us:.2f} us/launch, {gbps:.0f} GB/s ({100 * gbps / HBM_PEAK_GBPS:.1f}% of peak)")
    gpu.map_destroy(wmap)
    gpu.map_destroy(amap)
    return out


def measure_attention(gpu, A, ctxs=(1024, 4096, 16384), Hq=32, Hkv=8, d=128):
    """GQA decode attention (scores + softmax.V issued as the decode loop does, inside a batch) over an fp16
    KV cache: microseconds per attention and KV bytes per second.  Several distinct KV instances
    (> 256 MB together where they fit 600 MB) are cycled so the last-level cache cannot serve them."""
    up = lambda v: gpu.upload_dev(np.asarray(v, np.uint32))[0]
    out = {}
    for ctx in ctxs:
        n_inst = max(2, min(32, (600 << 20) // (2 * Hkv * ctx * d * 2)))
        step, sc_sz = ctx * d, Hq * ctx
        q_pos, out_pos = sc_sz + 1, sc_sz + 1 + Hq * d          # odd: query rows need no alignment
        kv_start = (out_pos + Hq * d + d - 1) // d * d
        gpu.set_dtype(A.DTYPE_F32)
        gpu.map_create(0, 1, kv_start + n_inst * 2 * Hkv * step)
        gpu.kv_cache_fp16(0, kv_start, n_inst * 2 * Hkv * step)
        rng = np.random.default_rng(ctx)
        gpu.scatter_contiguous(0, q_pos, rng.standard_normal(Hq * d).astype(np.float32))
        blk = rng.standard_normal(2 * Hkv * step).astype(np.float32)
        for i in range(n_inst):
            gpu.scatter_contiguous(0, kv_start + i * 2 * Hkv * step, blk)
        heads = np.arange(Hq) // (Hq // Hkv)
        q_rows, s_rows, o_rows = up(q_pos + np.arange(Hq) * d), up(np.arange(Hq) * ctx), up(out_pos + np.arange(Hq) * d)
        ops = []
        for i in range(n_inst):
            base = kv_start + i * 2 * Hkv * step
            ops.append(A.DecodePlanOp(kind=A.DECODE_OP_MATMUL_T, map_id=0, h0=q_rows, h1=up(base + heads * step),
                                      h2=s_rows, u0=1, u1=d, u2=ctx, u3=Hq))
            ops.append(A.DecodePlanOp(kind=A.DECODE_OP_ATTN_SOFTMAX_VALUE, map_id=0, h0=s_rows,
                                      h1=up(base + (Hkv + heads) * step), h2=o_rows, u0=Hq, u1=ctx, u2=d,
                                      f0=float(1 / np.sqrt(d)), f1=0.0))
            ops.append(A.DecodePlanOp(kind=A.DECODE_OP_FUSION_FLUSH))
        gpu.register_decode_plan(7, ops)
        gpu.decode_step(7, 0, 0)
        gpu.sync()
        rounds = 4
        gpu.timer_begin()
        for _ in range(rounds):
            gpu.decode_step(7, 0, 0)
        us = gpu.timer_end() * 1e3 / (rounds * n_inst)
        kvb = 2 * Hkv * ctx * d * 2
        out[str(ctx)] = {"us": round(us, 2), "kv_MB": round(kvb / 1e6, 2), "GB/s": round(kvb / us / 1e3, 1),
                         "frac": round(kvb / us / 1e3 / HBM_PEAK_GBPS, 4), "instances": n_inst}
        log(f"attention {Hq}q/{Hkv}kv x{d} ctx {ctx}: {us:.2f} us, {kvb / us / 1e3:.0f} GB/s of KV")
        gpu.clear_decode_plan(7)
        gpu.map_destroy(0)
    return out


def measure_gemm(gpu, A, Ms=(16, 512), shapes=((28672, 4096), (4096, 4096), (4096, 14336))):
    """Batched Q4_0 matmul C[M, N] = X[M, K] . W[N, K]^T (prefill chunk M = 512, batched decode M = 16) on
    the fp16 matrix cores: microseconds per call, dense TFLOP/s and the rate at which weights stream."""
    total = 4 * 28672 * 4096
    rng = np.random.default_rng(5)
    gpu.map_create_typed(3, A.DTYPE_Q4, 1, total, 32)
    s = rng.uniform(0.001, 0.01, total // 32).astype(np.float16).astype(np.float32)
    gpu.set_qparams(3, s, np.float32(-8.0) * s)
    chunk = 1 << 26
    for b in range(0, total // 2, chunk):
        n = min(chunk, total // 2 - b)
        gpu.scatter_q4_packed_contiguous(3, 2 * b, rng.integers(0, 256, n, dtype=np.uint8), n_locs=2 * n)
    out = {}
    for M in Ms:
        for N, K in shapes:
            gpu.set_dtype(A.DTYPE_F32)
            gpu.map_create(5, 1, M * (2 * K + N))
            gpu.scatter_contiguous(5, 0, rng.standard_normal(2 * M * K).astype(np.float32))
            # two copies of the rows, alternated: every call converts its rows to fp16 (a lone matmul's cost);
            # with one copy the calls after the first find them converted (K and V after Q, up after gate)
            a2 = [gpu.upload_dev(np.array([i * M * K], np.uint32))[0] for i in range(2)]
            c = gpu.upload_dev(np.array([2 * M * K], np.uint32))[0]
            n_mats = total // (N * K)
            bs = [gpu.upload_dev(np.array([i * N * K], np.uint32))[0] for i in range(n_mats)]
            rounds = 3
            t = {}
            for mode in ("alone", "shared"):
                pick = (lambda i: a2[i & 1]) if mode == "alone" else (lambda i: a2[0])
                for i, b in enumerate(bs):
                    gpu.map_matmul_t_xq4_dev(5, 3, pick(i), b, c, M, K, N, 1)
                gpu.sync()
                gpu.timer_begin()
                for r in range(rounds):
                    for i, b in enumerate(bs):
                        gpu.map_matmul_t_xq4_dev(5, 3, pick(i + r * n_mats), b, c, M, K, N, 1)
                t[mode] = gpu.timer_end() * 1e3 / (rounds * n_mats)
            us = t["alone"]
            out[f"M{M}_{N}x{K}"] = {"us": round(us, 2), "us_rows_already_converted": round(t["shared"], 2),
                                   "TFLOP/s": round(2 * M * N * K / us / 1e6, 1),
                                   "frac_fp16_mfma_peak": round(2 * M * N * K / us / 1e6 / 2500.0, 4),
                                   "weights_GB/s": round(N * K * 18 / 32 / us / 1e3, 1)}
            log(f"gemm M={M} {N}x{K}: {us:.1f} us, {2 * M * N * K / us / 1e6:.1f} TFLOP/s")
            gpu.map_destroy(5)
    gpu.map_destroy(3)
    return out


def blas_info():
    """Vendor, version, threading layer and thread count of the BLAS NumPy runs on (threadpoolctl)."""
    try:
        from threadpoolctl import threadpool_info
        pools = [p for p in threadpool_info() if p.get("user_api") == "blas"] or threadpool_info()
        return [{k: p.get(k) for k in ("internal_api", "version", "threading_layer", "architecture", "num_threads")}
                for p in pools]
    except Exception as e:                                  # noqa: BLE001 -- a missing helper must not cost the line
        return [{"error": repr(e)[:120]}]


def cpu_baseline(cfg, tensors, ctx_end, n_steps):
    """The oracle's NumPy forward pass (reference forward_cpu restated) on this host's cores, at the context the
    GPU leg is timed at: the K / V caches hold random fp16-exact rows for positions 0 .. ctx_end - n_steps - 1 (what
    a prompt of that length leaves behind costs hours on the CPU and changes nothing about a step's work), then
    n_steps greedy steps are timed, the last one at context ctx_end."""
    from oracle.forward_cpu import CpuModel
    from adam_amd.quant import QTensor
    blas = blas_info()
    threads = max([int(p.get("num_threads") or 1) for p in blas] or [1])
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    m = CpuModel(cfg, deq, kv_cap=ctx_end + 1, kv_fp16=True, acc64=False)
    start = max(0, ctx_end - n_steps - 1)
    rng = np.random.default_rng(4)
    for L in range(cfg.n_layer):
        shape = (cfg.n_head_kv, start, cfg.head_dim_kv)
        m.k_cache[L, :, :start, :] = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
        m.v_cache[L, :, :start, :] = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    logits = m.forward(1, start)                            # untimed: first touch of every matrix
    t0 = time.perf_counter()
    for s in range(n_steps):
        nt = int(np.argmax(logits))
        logits = m.forward(nt, start + 1 + s)
    dt = time.perf_counter() - t0
    out = {"value": round(n_steps / dt, 3), "unit": "tok/s", "cores": int(threads), "kind": "port",
           "sample": f"{n_steps} greedy decode steps at context {start + 2}..{start + 1 + n_steps} over caches "
                     f"preloaded with random rows, same model, NumPy float32 BLAS on pre-dequantised weights "
                     f"({os.cpu_count()} logical CPUs visible)",
           "blas": blas}
    out.update(cpu_kernels())
    return out


def cpu_kernels():
    """The two kernels of the path alone, restated in NumPy (oracle/blocks.py; the attention form of the
    reference's engine.py:2428-2441): BASELINE config 1 GEMV and config 3 attention at context 4096."""
    from oracle import blocks
    rng = np.random.default_rng(0)
    N, K = CONFIG1_GEMV_SHAPE
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    d, codes = blocks.quantize_q4_0(w)
    wd = blocks.dequant_q4_0(d, codes).reshape(N, K)

    def best(fn, secs=1.0):
        fn(); t_end, b = time.perf_counter() + secs, 1e9
        while time.perf_counter() < t_end:
            t0 = time.perf_counter(); fn(); b = min(b, time.perf_counter() - t0)
        return b
    t_pre = best(lambda: wd @ x)
    t_deq = best(lambda: blocks.dequant_q4_0(d, codes).reshape(N, K) @ x)
    Hq, Hkv, dd, ctx = 32, 8, 128, 4096
    q = rng.standard_normal((Hq, dd)).astype(np.float32)
    Kc = rng.standard_normal((Hkv, ctx, dd)).astype(np.float16); Vc = rng.standard_normal((Hkv, ctx, dd)).astype(np.float16)

    def attn():
        o = np.empty((Hq, dd), np.float32)
        for h in range(Hq):
            kh, vh = Kc[h // (Hq // Hkv)].astype(np.float32), Vc[h // (Hq // Hkv)].astype(np.float32)
            sc = kh @ q[h] * np.float32(1 / np.sqrt(dd))
            p = np.exp(sc - sc.max()); p /= p.sum()
            o[h] = p @ vh
        return o
    t_att = best(attn)
    return {"gemv_6912x1152_us": {"pre_dequantised": round(t_pre * 1e6, 1), "dequant_and_gemv": round(t_deq * 1e6, 1)},
            "attention_32q8kv_d128_ctx4096_us": round(t_att * 1e6, 1)}


def measure_model_batched(args, A, synth, DecodeEngine):
    """Whole-model legs beyond bs = 1 decode: the prompt as one chunk, and lockstep decoding of a batch."""
    cfg = synth.gemma3_1b_config() if args.workload == "gemma3-1b" else synth.llama3_8b_config()
    tensors = synth.make_model(cfg, seed=0, sigma=0.02)
    gpu = A.init()
    rng = np.random.default_rng(0)
    out = {"workload": args.workload}
    if args.only == "prefill":
        n_prompt = args.prompt or 512
        prompt = [int(t) for t in rng.integers(0, cfg.n_vocab, n_prompt)]
        ref = None
        big = args.prefill_chunk or n_prompt
        for chunk in ((big,) if args.skip_reference else (0, big)):
            eng = DecodeEngine(gpu, cfg, tensors, A=A, kv_cap=n_prompt + 16, kv_fp16=True, fusion_scheduler_mode=args.scheduler,
                               prefill_chunk=chunk)
            eng.reset()
            eng.prefill(prompt); gpu.sync()                                  # warm-up (allocations, code objects)
            gpu.reset_native_stats()
            t0 = time.perf_counter(); eng.prefill(prompt); gpu.sync(); dt = time.perf_counter() - t0
            hid, tok = eng.read_slot('hidden'), eng.read_token()
            ref = ref if ref is not None else (hid, tok)
            key = "token_by_token" if chunk == 0 else f"chunk_{chunk}"
            out[key] = {"ms": round(dt * 1e3, 2), "tok/s": round(n_prompt / dt, 1),
                        "launches": gpu.get_native_stats()["dispatch_count"]}
            if not args.skip_reference:
                out[key].update({"hidden_rel_l2_vs_token_by_token": float(np.linalg.norm(hid - ref[0]) / np.linalg.norm(ref[0])),
                                 "first_token_same": bool(tok == ref[1])})
            log(f"prefill {n_prompt} tokens {key}: {dt * 1e3:.1f} ms")
    else:
        B, P = args.batch, args.prompt or 1024
        eng = DecodeEngine(gpu, cfg, tensors, A=A, kv_cap=P + args.steps + 8, kv_fp16=True,
                           fusion_scheduler_mode=args.scheduler, prefill_chunk=512, batch=B)
        prompts = [[int(t) for t in rng.integers(0, cfg.n_vocab, P)] for _ in range(B)]
        _, st = eng.generate_batch(prompts, args.steps)
        out.update({"batch": B, "prompt": P, "steps": args.steps, "prefill_tok/s": round(B * P / st["prefill_s"], 1),
                    "decode_tok/s_aggregate": round(st["decode_tps"], 1), "ms_per_step": round(st["decode_s"] / args.steps * 1e3, 3)})
    gpu.shutdown()
    return out


def step_bytes_of(cfg, tensors, ctx_mid):
    """Algorithmic HBM bytes of one bs=1 decode step: every weight block once + the KV rows of the context."""
    q4_w = sum(v.size for v in tensors.values() if getattr(v, "kind", "") == "q4_0")
    q8_w = sum(v.size for v in tensors.values() if getattr(v, "kind", "") == "q8_0")
    kv_b = 2 * cfg.n_layer * cfg.n_head_kv * cfg.head_dim_kv * 2 * ctx_mid
    return q4_w * 18 // 32 + q8_w * 34 // 32 + kv_b


def measure_decode(gpu, A, DecodeEngine, cfg, tensors, prompt, steps, warmup, scheduler, prefill_chunk, decode_plan=True,
                   lookahead=True, repeats=3):
    """bs=1 greedy decode: the prompt, `warmup` untimed steps, then exactly `steps` timed steps (token id read back
    every step) between two device synchronisations, `repeats` times over; the median run is the result.  decode_plan=False issues every op of a step as a call of its own
    through the op surface, which is what the unchanged reference engine does (adam/models/engine.py:2971-3706).
    lookahead (the engine's default greedy loop): every step takes its input token from the device slot the previous
    step's LM head wrote and is issued before the host has read that token; the host reads every token, in order, one
    issue late.  lookahead=False: read the token, then issue the step that consumes it, as the reference's loop does."""
    n_prompt = len(prompt)
    eng = DecodeEngine(gpu, cfg, tensors, A=A, kv_cap=n_prompt + warmup + steps + 8, kv_fp16=True,
                       fusion_scheduler_mode=scheduler, prefill_chunk=prefill_chunk, decode_plan=decode_plan,
                       lookahead=lookahead)
    lookahead = lookahead and eng._lookahead and eng._token_feed() is not None
    gpu.sync()
    eng.reset()
    t0 = time.perf_counter()
    eng.prefill(prompt)
    gpu.sync()
    prefill_s = time.perf_counter() - t0
    tokens, pos = [], n_prompt

    def run(n):
        nonlocal pos
        for _ in range(n):
            if lookahead:
                eng._forward(None, pos, from_device=True)
                nt = eng._wait_tokens(eng._feed_ticket)[0]      # the token that step consumes
            else:
                nt = eng.read_token()
                eng._forward(nt, pos)
            tokens.append(nt)
            pos += 1

    run(warmup)
    gpu.sync()
    # The reference's protocol (adam/tools/benchmark.py:56-61,874): one cold run, one warm-up, then the median of
    # three steady runs.  Prefill and the warm-up steps stand for the first two; the timed region -- exactly `steps`
    # steps between two device synchronisations -- is run `repeats` times over the same positions (the position is
    # wound back, the cache rows of those positions are written again) and the median run is reported.
    start, runs, dev_runs, launches, first = pos, [], [], 0, None
    for r in range(repeats):
        pos = start
        n_before = len(tokens)
        gpu.sync()
        gpu.reset_native_stats()
        gpu.timer_begin()
        t0 = time.perf_counter()
        run(steps)
        gpu.sync()
        runs.append(time.perf_counter() - t0)
        dev_runs.append(gpu.timer_end())
        launches = gpu.get_native_stats()["dispatch_count"]
        first = first if first is not None else tokens[n_before:]
    order = sorted(range(repeats), key=lambda i: runs[i])
    wall, dev_ms = runs[order[repeats // 2]], dev_runs[order[repeats // 2]]
    sb = step_bytes_of(cfg, tensors, n_prompt + warmup + steps // 2)
    ceiling = HBM_PEAK_GBPS * 1e9 / sb
    feed_bytes, feed_s = eng.feed_table_bytes, eng.feed_table_upload_s
    del eng
    return {"tok_s": steps / wall, "ms_per_step": 1e3 * wall / steps, "device_ms_per_step": dev_ms / steps,
            "tok_s_runs": [round(steps / t, 2) for t in runs],
            "launches_per_token": launches / max(1, steps), "prefill_s": prefill_s, "n_prompt": n_prompt,
            "end_pos": pos, "tokens": first, "step_bytes": int(sb), "ceiling": ceiling,
            "feed_table_bytes": int(feed_bytes), "feed_table_upload_s": round(feed_s, 3),
            # the reference's stat keys (adam/models/engine.py:3922-3944)
            "stats": {"n_prompt": n_prompt, "n_gen": steps, "prefill_tps": round(n_prompt / prefill_s, 1),
                      "decode_tps": round(steps / wall, 2), "avg_ms": round(1e3 * wall / steps, 4),
                      "sampling_mode": "gpu_matvec_argmax"}}


def measure_lockstep(gpu, A, DecodeEngine, cfg, tensors, batch, n_prompt, steps, scheduler):
    """BASELINE config 5: `batch` independent random prompts prefilled in chunks of 512 tokens on the matrix cores,
    then `steps` lockstep decode steps."""
    rng = np.random.default_rng(1)
    eng = DecodeEngine(gpu, cfg, tensors, A=A, kv_cap=n_prompt + steps + 8, kv_fp16=True,
                       fusion_scheduler_mode=scheduler, prefill_chunk=512, batch=batch)
    prompts = [[int(t) for t in rng.integers(0, cfg.n_vocab, n_prompt)] for _ in range(batch)]
    _, st = eng.generate_batch(prompts, steps)
    del eng
    return {"batch": batch, "prompt_tokens_per_sequence": n_prompt, "prefill_chunk": 512, "steps": steps,
            "prefill_tok/s": round(batch * n_prompt / st["prefill_s"], 1),
            "decode_tok/s_aggregate": round(st["decode_tps"], 1),
            "ms_per_step": round(st["decode_s"] / steps * 1e3, 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="llama3-8b", choices=["gemma3-1b", "llama3-8b"])
    ap.add_argument("--prompt", type=int, default=None,
                    help="prompt length (default: llama3-8b 4096 - warmup - steps, so that the last timed step runs at "
                         "context 4096; gemma3-1b 512)")
    ap.add_argument("--scheduler", default="level_batched", choices=["legacy", "level_batched"])
    ap.add_argument("--prefill-chunk", type=int, default=None,
                    help="prompt in chunks of this many tokens on the matrix-core matmul (0: token by token, as the "
                         "reference does; default 512 for llama3-8b, 0 for gemma3-1b); the timed region is the decode "
                         "loop either way")
    ap.add_argument("--batch", type=int, default=16, help="sequences decoded in lockstep (config 5 leg, --only batch)")
    ap.add_argument("--only", default=None, choices=["roofline", "gemv", "probe", "attention", "gemm", "prefill", "batch"],
                    help="roofline: just the 28672x4096 GEMV (one kernel row in a rocprofv3 --stats table); "
                         "gemv: that shape, 4096x4096 and 4096x14336; probe: plain read/copy kernels of known "
                         "size (reference points for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE); attention: GQA "
                         "decode attention 32q/8kv x128 at ctx 1024/4096/16384; gemm: batched Q4_0 matmul at "
                         "M = 16 and 512 on the Llama-3-8B shapes; prefill: a 512-token prompt of --workload token "
                         "by token and in one chunk (matrix-core matmuls, causal attention in one launch per "
                         "layer); batch: --batch random prompts of --prompt (default 1024) tokens prefilled in "
                         "chunks of 512, then --steps lockstep decode steps of --workload")
    ap.add_argument("--skip-reference", action="store_true",
                    help="--only prefill: time the chunked prompt alone (chunks of --prefill-chunk, default the whole "
                         "prompt), without the token-by-token run it is otherwise compared with")
    ap.add_argument("--no-roofline", action="store_true", help="skip the kernel legs (GEMV shapes, attention, matmul)")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the other configurations (op-by-op decode, Gemma-3-1B shape, lockstep batch)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    from adam_amd import adamah as A, synth
    from adam_amd.engine import DecodeEngine

    if args.only in ("prefill", "batch"):
        if args.only == "batch" and args.steps == 256:
            args.steps = 128
        print(json.dumps(measure_model_batched(args, A, synth, DecodeEngine)), flush=True)
        return
    if args.only:
        gpu = A.init()
        if args.only == "roofline":
            out = {"gemv_shapes": measure_gemv(gpu, A, LLAMA_GEMV_SHAPES[:1], rounds=8)}
        elif args.only == "gemv":
            out = {"gemv_shapes": measure_gemv(gpu, A, LLAMA_GEMV_SHAPES, rounds=3)}
        elif args.only == "attention":
            out = {"attention": measure_attention(gpu, A)}
        elif args.only == "gemm":
            out = {"gemm": measure_gemm(gpu, A)}
        else:
            nbytes = gemv_bytes(28672, 4096) // 4096 * 4096
            pool = nbytes * 16
            out = {"probe_bytes_per_launch": nbytes,
                   "read_us": round(gpu.stream_probe(nbytes, pool, 0, 32, 48), 3),
                   "copy_us": round(gpu.stream_probe(nbytes, pool, 1, 4, 48), 3)}
            out["read_GB/s"] = round(nbytes / out["read_us"] / 1e3, 1)
            out["copy_GB/s"] = round(2 * nbytes / out["copy_us"] / 1e3, 1)
        gpu.shutdown()
        print(json.dumps(out), flush=True)
        return

    gemma = args.workload == "gemma3-1b"
    cfg = synth.gemma3_1b_config() if gemma else synth.llama3_8b_config()
    if args.prompt is not None:
        n_prompt = args.prompt
    else:
        n_prompt = 512 if gemma else max(16, 4096 - args.warmup - args.steps)
    chunk = args.prefill_chunk if args.prefill_chunk is not None else (0 if gemma else 512)
    t0 = time.perf_counter()
    tensors = synth.make_model(cfg, seed=0, sigma=0.02)
    log(f"synthesised {args.workload} weights in {time.perf_counter() - t0:.1f}s")

    gpu = A.init()
    rng = np.random.default_rng(0)
    prompt = [int(t) for t in rng.integers(0, cfg.n_vocab, n_prompt)]
    t0 = time.perf_counter()
    m = measure_decode(gpu, A, DecodeEngine, cfg, tensors, prompt, args.steps, args.warmup, args.scheduler, chunk)
    log(f"{args.workload}: {m['tok_s']:.1f} tok/s, {m['ms_per_step']:.3f} ms/step, prefill {m['prefill_s']:.2f}s "
        f"({time.perf_counter() - t0:.1f}s for the leg)")

    res = {
        "metric": METRIC, "value": round(m["tok_s"], 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(m["ms_per_step"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}-shape Q4_0 random-init"
                               + ("" if gemma else " (Q8_0 output head)") + ", bs=1 greedy decode, "
                               f"{n_prompt}-token random prompt "
                               f"({'chunks of ' + str(chunk) if chunk else 'token by token'}), fp16 KV, "
                               f"timed steps at context {m['end_pos'] - args.steps + 1}..{m['end_pos']}",
                   "baseline_config": 2 if gemma else 4,
                   "scheduler": args.scheduler, "launches_per_token": round(m["launches_per_token"], 1),
                   "issue": "one native decode_step call per token (registered decode plan, launched from HIP graphs "
                            "recorded one step ahead); every token id is read back, in order, but the step that consumes "
                            "token n takes it from the device and is issued before the host has read it (one step of "
                            "lookahead; 'read_then_issue' is the same loop without it)"},
        "timed_runs": {"protocol": "prefill (cold) and the warm-up steps, then the timed region of exactly `steps` steps "
                                   "three times over the same positions; value = the median run "
                                   "(adam/tools/benchmark.py:56-61,874)",
                       "tok/s": m["tok_s_runs"], "min": min(m["tok_s_runs"]), "max": max(m["tok_s_runs"])},
        "device_ms_per_step": round(m["device_ms_per_step"], 4),
        "token_feed_table": {"device_bytes": m["feed_table_bytes"], "upload_s": m["feed_table_upload_s"],
                             "note": "float32 [V, E] copy of an untied embedding table from which the device gathers the "
                                     "row of a token it still holds (0 for tied models: they read the LM head's rows); "
                                     "uploaded before the timed region"},
        "algorithmic_bytes_per_token": m["step_bytes"],
        "tok_s_at_hbm_peak": round(m["ceiling"], 1), "frac_of_hbm_roofline": round(m["tok_s"] / m["ceiling"], 4),
        "prefill_tok_s": round(n_prompt / m["prefill_s"], 1), "first_tokens": m["tokens"][:8],
        "stats": m["stats"],
    }

    def leg(name, fn):
        """An extra leg never costs the headline line: its failure is reported in its own object."""
        t0 = time.perf_counter()
        try:
            res[name] = fn()
        except Exception as e:
            res[name] = {"error": repr(e)[:300]}
        log(f"{name}: {time.perf_counter() - t0:.1f}s")

    if not args.no_extra:
        n_obo = min(args.steps, 32)

        def op_by_op(cfg_, tensors_, prompt_, chunk_, ref_tokens):
            o = measure_decode(gpu, A, DecodeEngine, cfg_, tensors_, prompt_, n_obo, args.warmup, args.scheduler,
                               chunk_, decode_plan=False, lookahead=False, repeats=1)
            return {"tok/s": round(o["tok_s"], 2), "ms_per_step": round(o["ms_per_step"], 4), "steps": n_obo,
                    "launches_per_token": round(o["launches_per_token"], 1),
                    "issue": "every op of the step as its own call through ctypes, as the reference engine issues them",
                    "tokens_same_as_plan_replay": bool(o["tokens"][:8] == ref_tokens[:8])}
        leg("op_by_op", lambda: op_by_op(cfg, tensors, prompt, chunk, m["tokens"]))

        def read_then_issue():
            o = measure_decode(gpu, A, DecodeEngine, cfg, tensors, prompt, args.steps, args.warmup, args.scheduler, chunk,
                               lookahead=False)
            return {"tok/s": round(o["tok_s"], 2), "ms_per_step": round(o["ms_per_step"], 4), "steps": args.steps,
                    "tok/s_runs": o["tok_s_runs"],
                    "issue": "the headline loop without lookahead: the host reads token n, then issues the step that "
                             "consumes it (embedding row looked up with host-made locations), as the reference's loop does",
                    "tokens_same_as_headline": bool(o["tokens"] == m["tokens"])}
        leg("read_then_issue", read_then_issue)

        def other_shape():
            g2 = not gemma
            cfg2 = synth.gemma3_1b_config() if g2 else synth.llama3_8b_config()
            t2 = synth.make_model(cfg2, seed=0, sigma=0.02)
            st2 = min(args.steps, 128) if g2 else args.steps
            np2 = 512 if g2 else max(16, 4096 - args.warmup - st2)
            p2 = [int(t) for t in np.random.default_rng(0).integers(0, cfg2.n_vocab, np2)]
            o = measure_decode(gpu, A, DecodeEngine, cfg2, t2, p2, st2, args.warmup, args.scheduler, 0 if g2 else 512)
            out = {"workload": ("gemma3-1b" if g2 else "llama3-8b") + f"-shape Q4_0 random-init, bs=1 greedy decode, "
                               f"{np2}-token random prompt, fp16 KV, timed steps at context "
                               f"{o['end_pos'] - st2 + 1}..{o['end_pos']}",
                   "tok/s": round(o["tok_s"], 2), "tok/s_runs": o["tok_s_runs"], "ms_per_step": round(o["ms_per_step"], 4),
                   "steps": st2,
                   "launches_per_token": round(o["launches_per_token"], 1),
                   "tok_s_at_hbm_peak": round(o["ceiling"], 1), "frac_of_hbm_roofline": round(o["tok_s"] / o["ceiling"], 4),
                   "prefill_tok_s": round(np2 / o["prefill_s"], 1), "stats": o["stats"]}
            ob = measure_decode(gpu, A, DecodeEngine, cfg2, t2, p2, n_obo, args.warmup, args.scheduler, 0 if g2 else 512,
                                decode_plan=False, lookahead=False, repeats=1)
            out["op_by_op_tok/s"] = round(ob["tok_s"], 2)
            rt = measure_decode(gpu, A, DecodeEngine, cfg2, t2, p2, st2, args.warmup, args.scheduler, 0 if g2 else 512,
                                lookahead=False)
            out["read_then_issue_tok/s"] = round(rt["tok_s"], 2)
            return out
        leg("config2_gemma3_1b" if not gemma else "config4_llama3_8b", other_shape)

        if not gemma:
            leg("config5_batched", lambda: dict(
                measure_lockstep(gpu, A, DecodeEngine, cfg, tensors, args.batch, 1024, 128, args.scheduler),
                mfma_busy_source="profiles/gemm_q4_0_m16_m512_mfma_busy.txt"))

    if not args.no_roofline:
        shapes = measure_gemv(gpu, A, LLAMA_GEMV_SHAPES + [CONFIG1_GEMV_SHAPE])
        top = shapes["28672x4096"]
        # what a plain read kernel of the same number of bytes reaches in this run on this box: kernel vs achievable
        nbytes = gemv_bytes(28672, 4096) // 4096 * 4096
        try:
            probe_us = min(gpu.stream_probe(nbytes, nbytes * 16, 0, wg, 48) for wg in (8, 16, 32))
            probe = {"probe_us": round(probe_us, 3), "probe_frac": round(nbytes / probe_us / 1e3 / HBM_PEAK_GBPS, 4)}
        except RuntimeError as e:
            probe = {"probe_error": repr(e)[:200]}
        res["roofline"] = {"bound": "hbm", "achieved": top["GB/s"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": top["frac"], "traffic": GEMV_TRAFFIC_BYTES, **probe,
                           "probe": "plain 16-byte-per-lane read of the same bytes per launch over 16 distinct buffers "
                                    "(adamah_hip_stream_probe), best of 8 / 16 / 32 workgroups per CU",
                           "traffic_source": GEMV_TRAFFIC_SOURCE,
                           "kernel": "k_gemv_mfma<Q4_0 block16, store> 28672x4096, "
                                     f"{gemv_bytes(28672, 4096)} algorithmic B/launch"}
        res["gemv_shapes"] = shapes
        leg("attention_32q8kv_d128", lambda: measure_attention(gpu, A))
        if not args.no_extra:
            leg("gemm_q4_0", lambda: measure_gemm(gpu, A))
    gpu.shutdown()

    if not args.no_cpu_baseline:
        t0 = time.perf_counter()
        res["cpu_baseline"] = cpu_baseline(cfg, tensors, m["end_pos"], n_steps=48 if gemma else 6)
        log(f"cpu baseline {res['cpu_baseline']['value']} tok/s ({time.perf_counter() - t0:.1f}s incl. dequant)")

    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
