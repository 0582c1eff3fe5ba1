"""GGUF reader and block -> map-form conversion (CPU only).

The files are written by this test from the published layout (header, typed metadata, tensor
descriptors, aligned data; ggml block formats Q4_0, Q8_0, Q4_K), with random bit patterns in every
block field.  Expected values come from element-by-element decoders written here in the ggml
formulation -- w = d (q - 8), w = d q, w = d sc q - dmin m with the 6-bit (sc, m) unpacking -- and not
from the code under test.  Bars: metadata round trip exact; map-form codes / scales / zero points such
that dequantisation is bit-exact against those decoders in float32; a tiny model of either family read
from a file and decoded through the op-surface oracle gives the tokens of the restated reference
forward pass over the same dequantised weights."""
import struct

import numpy as np
import pytest

import oracle
from oracle.forward_cpu import CpuModel
from adam_amd import adamah as A
from adam_amd import gguf
from adam_amd.engine import DecodeEngine, GenerationConfig
from adam_amd.quant import QTensor


# ------------------------------------------------------------------ writer (test side)
def _s(x):
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _kv(key, value):
    if isinstance(value, bool):
        return _s(key) + struct.pack("<I?", 7, value)
    if isinstance(value, str):
        return _s(key) + struct.pack("<I", 8) + _s(value)
    if isinstance(value, float):
        return _s(key) + struct.pack("<If", 6, value)
    if isinstance(value, int):
        return _s(key) + struct.pack("<II", 4, value)
    if isinstance(value, list) and value and isinstance(value[0], str):
        return _s(key) + struct.pack("<IIQ", 9, 8, len(value)) + b"".join(_s(v) for v in value)
    if isinstance(value, list):
        return _s(key) + struct.pack("<IIQ", 9, 5, len(value)) + struct.pack(f"<{len(value)}i", *value)
    raise TypeError(value)


def write_gguf(path, metadata, tensors, align=32, version=3):
    """tensors: list of (name, shape rows-first, ggml type, raw bytes)."""
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(metadata) + 1)
    head += _s("general.alignment") + struct.pack("<II", 4, align)
    for k, v in metadata.items():
        head += _kv(k, v)
    off, infos, blobs = 0, b"", []
    for name, shape, gtype, raw in tensors:
        dims = tuple(reversed(shape))
        infos += _s(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims) + struct.pack("<IQ", gtype, off)
        pad = (-len(raw)) % align
        blobs.append(raw + b"\0" * pad)
        off += len(raw) + pad
    body = head + infos
    body += b"\0" * ((-len(body)) % align)
    with open(path, "wb") as f:
        f.write(body + b"".join(blobs))


def rand_f16(rng, n, lo=0.001, hi=0.05):
    return rng.uniform(lo, hi, n).astype(np.float16)


def make_q4_0(rng, n_blocks):
    b = np.empty((n_blocks, 18), np.uint8)
    b[:, 0:2] = rand_f16(rng, n_blocks).view(np.uint8).reshape(n_blocks, 2)
    b[:, 2:] = rng.integers(0, 256, (n_blocks, 16), dtype=np.uint8)
    return b.tobytes()


def make_q8_0(rng, n_blocks):
    b = np.empty((n_blocks, 34), np.uint8)
    b[:, 0:2] = rand_f16(rng, n_blocks).view(np.uint8).reshape(n_blocks, 2)
    b[:, 2:] = rng.integers(0, 256, (n_blocks, 32), dtype=np.uint8)
    return b.tobytes()


def make_q4_k(rng, n_blocks):
    b = np.empty((n_blocks, 144), np.uint8)
    b[:, 0:2] = rand_f16(rng, n_blocks, 0.0005, 0.003).view(np.uint8).reshape(n_blocks, 2)
    b[:, 2:4] = rand_f16(rng, n_blocks, 0.0005, 0.003).view(np.uint8).reshape(n_blocks, 2)
    b[:, 4:] = rng.integers(0, 256, (n_blocks, 140), dtype=np.uint8)      # every scale / minimum bit pattern
    return b.tobytes()


# ------------------------------------------------------------------ independent decoders (ggml formulation)
def dec_q4_0(raw):
    out = []
    for i in range(0, len(raw), 18):
        d = np.frombuffer(raw[i:i + 2], np.float16)[0].astype(np.float32)
        qs = raw[i + 2:i + 18]
        out += [d * np.float32((q & 15) - 8) for q in qs] + [d * np.float32((q >> 4) - 8) for q in qs]
    return np.array(out, np.float32)


def dec_q8_0(raw):
    out = []
    for i in range(0, len(raw), 34):
        d = np.frombuffer(raw[i:i + 2], np.float16)[0].astype(np.float32)
        out += [d * np.float32(q) for q in np.frombuffer(raw[i + 2:i + 34], np.int8)]
    return np.array(out, np.float32)


def dec_q4_k(raw):
    out = []
    for i in range(0, len(raw), 144):
        d = np.frombuffer(raw[i:i + 2], np.float16)[0].astype(np.float32)
        dmin = np.frombuffer(raw[i + 2:i + 4], np.float16)[0].astype(np.float32)
        sc = raw[i + 4:i + 16]
        qs = raw[i + 16:i + 144]

        def scale_min(j):
            if j < 4:
                return sc[j] & 63, sc[j + 4] & 63
            return (sc[j + 4] & 15) | ((sc[j - 4] >> 6) << 4), (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)

        for c in range(4):                                 # 64 weights per 32 bytes
            s1, m1 = scale_min(2 * c)
            s2, m2 = scale_min(2 * c + 1)
            d1, n1 = d * np.float32(s1), dmin * np.float32(m1)
            d2, n2 = d * np.float32(s2), dmin * np.float32(m2)
            out += [d1 * np.float32(q & 15) - n1 for q in qs[32 * c:32 * c + 32]]
            out += [d2 * np.float32(q >> 4) - n2 for q in qs[32 * c:32 * c + 32]]
    return np.array(out, np.float32)


# ------------------------------------------------------------------ tests
def test_header_metadata_and_block_conversions(tmp_path):
    rng = np.random.default_rng(1)
    raws = {"a.weight": (gguf.GGML_Q4_0, (6, 64), make_q4_0(rng, 12)),
            "b.weight": (gguf.GGML_Q8_0, (4, 96), make_q8_0(rng, 12)),
            "c.weight": (gguf.GGML_Q4_K, (3, 512), make_q4_k(rng, 6)),
            "n.weight": (gguf.GGML_F32, (40,), rng.standard_normal(40).astype(np.float32).tobytes()),
            "h.weight": (gguf.GGML_F16, (2, 8), rng.standard_normal(16).astype(np.float16).tobytes())}
    md = {"general.architecture": "llama", "llama.block_count": 3, "llama.rope.freq_base": 500000.0,
          "some.flag": True, "tokenizer.ggml.tokens": ["<a>", "b", "çé"], "tokenizer.ggml.token_type": [1, 2, -3]}
    p = tmp_path / "t.gguf"
    for align, version in ((32, 3), (64, 2)):
        write_gguf(p, md, [(n, s, t, r) for n, (t, s, r) in raws.items()], align=align, version=version)
        f = gguf.GGUFFile(str(p))
        assert f.version == version and f.metadata["general.alignment"] == align
        for k, v in md.items():
            got = f.metadata[k]
            assert got == pytest.approx(v) if isinstance(v, float) else got == v
        assert {n: (s, t) for n, (s, t, _) in f.tensors.items()} == {n: (s, t) for n, (t, s, _) in raws.items()}
        for name, dec in (("a.weight", dec_q4_0), ("b.weight", dec_q8_0), ("c.weight", dec_q4_k)):
            t = f.tensor(name)
            assert isinstance(t, QTensor) and t.shape == raws[name][1]
            exp = dec(raws[name][2]).reshape(t.shape)
            if name == "c.weight":
                # scale * q + zp rounds twice exactly as d sc q - dmin m does (two products, one sum)
                assert t.kind == 'q4_aff' and t.d is None
            assert np.array_equal(t.dequant().view(np.uint32), exp.view(np.uint32)), name
            assert np.array_equal(t.dequant_rows(1, 2), exp[1:3])
        assert np.array_equal(f.tensor("n.weight"), np.frombuffer(raws["n.weight"][2], np.float32))
        assert np.array_equal(f.tensor("h.weight"), np.frombuffer(raws["h.weight"][2], np.float16).astype(np.float32).reshape(2, 8))
        f.close()


def test_q4_k_map_form_goes_through_the_op_surface_bit_exactly(tmp_path):
    """Uploaded as packed nibbles + qparams and multiplied by an identity matrix: the values of the ggml
    decoder come back (one non-zero product per sum, so nothing rounds)."""
    rng = np.random.default_rng(2)
    raw = make_q4_k(rng, 4)
    N, K = 2, 512
    t = gguf.from_gguf_q4_k(np.frombuffer(raw, np.uint8), (N, K))
    g = oracle.init()
    g.map_create_typed(1, A.DTYPE_Q4, 1, N * K, 32)
    g.set_qparams(1, *t.qparams())
    g.scatter_q4_packed_contiguous(1, 0, t.codes)
    g.set_dtype(A.DTYPE_F32)
    g.map_create(0, 1, K * K + K * N)
    g.scatter_contiguous(0, 0, np.eye(K, dtype=np.float32).reshape(-1))
    up = lambda a: g.upload_dev(np.asarray(a, np.uint32))[0]
    g.map_matmul_t_xq4_dev(0, 1, up([0]), up([0]), up([K * K]), K, K, N)
    got = g.gather(0, np.arange(K * K, K * K + K * N, dtype=np.uint32)).view(np.float32).reshape(K, N).T
    assert np.array_equal(got, dec_q4_k(raw).reshape(N, K))


def test_rejects_bad_files(tmp_path):
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(ValueError, match="not a GGUF"):
        gguf.GGUFFile(str(p))
    rng = np.random.default_rng(3)
    write_gguf(p, {"general.architecture": "llama"}, [("x.weight", (2, 64), 14, b"\0" * 210)])     # Q6_K
    f = gguf.GGUFFile(str(p))
    with pytest.raises(NotImplementedError, match="x.weight"):
        f.tensor("x.weight")
    f.close()
    write_gguf(p, {"general.architecture": "llama"}, [("y.weight", (2, 64), gguf.GGML_Q4_0, make_q4_0(rng, 2))])   # too short
    f = gguf.GGUFFile(str(p))
    with pytest.raises(ValueError, match="past the end"):
        f.tensor("y.weight")
    f.close()


def _model_file(path, arch, rng):
    L, E, H, KV, D, FF, V = 2, 256, 4, 2, 64, 512, 96
    md = {"general.architecture": arch, f"{arch}.block_count": L, f"{arch}.embedding_length": E,
          f"{arch}.feed_forward_length": FF, f"{arch}.attention.head_count": H, f"{arch}.attention.head_count_kv": KV,
          f"{arch}.attention.key_length": D, f"{arch}.attention.value_length": D, f"{arch}.context_length": 64,
          f"{arch}.attention.layer_norm_rms_epsilon": 1e-5, f"{arch}.rope.freq_base": 10000.0, f"{arch}.vocab_size": V}
    ts = []
    norm = lambda n: rng.uniform(0.5, 1.5, n).astype(np.float32).tobytes()
    for i in range(L):
        p = f"blk.{i}"
        # a mix of the three block formats, as quantised files have
        ts += [(f"{p}.attn_q.weight", (H * D, E), gguf.GGML_Q4_K, make_q4_k(rng, H * D * E // 256)),
               (f"{p}.attn_k.weight", (KV * D, E), gguf.GGML_Q4_0, make_q4_0(rng, KV * D * E // 32)),
               (f"{p}.attn_v.weight", (KV * D, E), gguf.GGML_Q4_K, make_q4_k(rng, KV * D * E // 256)),
               (f"{p}.attn_output.weight", (E, H * D), gguf.GGML_Q4_K, make_q4_k(rng, E * H * D // 256)),
               (f"{p}.ffn_gate.weight", (FF, E), gguf.GGML_Q4_K, make_q4_k(rng, FF * E // 256)),
               (f"{p}.ffn_up.weight", (FF, E), gguf.GGML_Q4_K, make_q4_k(rng, FF * E // 256)),
               (f"{p}.ffn_down.weight", (E, FF), gguf.GGML_Q4_0, make_q4_0(rng, E * FF // 32)),
               (f"{p}.attn_norm.weight", (E,), gguf.GGML_F32, norm(E)), (f"{p}.ffn_norm.weight", (E,), gguf.GGML_F32, norm(E))]
        if arch == "gemma3":
            ts += [(f"{p}.attn_q_norm.weight", (D,), gguf.GGML_F32, norm(D)), (f"{p}.attn_k_norm.weight", (D,), gguf.GGML_F32, norm(D)),
                   (f"{p}.post_attention_norm.weight", (E,), gguf.GGML_F32, norm(E)),
                   (f"{p}.post_ffw_norm.weight", (E,), gguf.GGML_F32, norm(E))]
    ts.append(("output_norm.weight", (E,), gguf.GGML_F32, norm(E)))
    ts.append(("token_embd.weight", (V, E), gguf.GGML_Q4_K if arch == "gemma3" else gguf.GGML_Q8_0,
               make_q4_k(rng, V * E // 256) if arch == "gemma3" else make_q8_0(rng, V * E // 32)))
    if arch == "llama":
        ts.append(("output.weight", (V, E), gguf.GGML_Q8_0, make_q8_0(rng, V * E // 32)))
        ts.append(("rope_freqs.weight", (D // 2,), gguf.GGML_F32, np.ones(D // 2, np.float32).tobytes()))
    write_gguf(path, md, ts)


@pytest.mark.parametrize("arch", ["llama", "gemma3"])
def test_model_from_file_decodes_like_the_reference_forward(tmp_path, arch):
    p = tmp_path / f"{arch}.gguf"
    _model_file(str(p), arch, np.random.default_rng(7))
    cfg, tensors = gguf.load_model(str(p))
    assert (cfg.arch, cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.n_head_kv, cfg.head_dim, cfg.n_ff, cfg.n_vocab) == \
        (arch, 2, 256, 4, 2, 64, 512, 96)
    assert cfg.ffn_act == ("gelu" if arch == "gemma3" else "silu") and (cfg.attn_softcap == 50.0) == (arch == "gemma3")
    assert "rope_freqs.weight" not in tensors
    deq = {n: (v.dequant() if isinstance(v, QTensor) else v) for n, v in tensors.items()}
    ref = CpuModel(cfg, deq, kv_cap=32, kv_fp16=False)
    prompt, n_gen = [5, 17, 3, 90], 6
    ref_tokens, margins = ref.generate(prompt, n_gen)
    eng = DecodeEngine(oracle.init(), cfg, tensors, A=A, kv_cap=32, gpu_fused_rows_per_group=32)
    out, _ = eng.generate(prompt, GenerationConfig(max_tokens=n_gen), forced=ref_tokens)
    for i, (a, b) in enumerate(zip(out, ref_tokens)):
        assert a == b or margins[i] < 1e-5, (i, a, b, margins[i])
    hid = eng.read_slot('hidden')
    assert np.linalg.norm(hid - ref.last_hidden) / np.linalg.norm(ref.last_hidden) < 1e-4
