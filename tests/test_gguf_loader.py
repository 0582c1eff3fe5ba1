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
from adam_amd import gguf, quant
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


def make_q5_0(rng, n_blocks):
    b = np.empty((n_blocks, 22), np.uint8)
    d = rand_f16(rng, n_blocks)
    d[::3] = -d[::3]                                   # negative scales occur in real files
    if n_blocks > 4:
        d[4] = 0
    b[:, 0:2] = d.view(np.uint8).reshape(n_blocks, 2)
    b[:, 2:] = rng.integers(0, 256, (n_blocks, 20), dtype=np.uint8)
    return b.tobytes()


def make_q6_k(rng, n_blocks):
    b = np.empty((n_blocks, 210), np.uint8)
    b[:, 0:208] = rng.integers(0, 256, (n_blocks, 208), dtype=np.uint8)     # every nibble, bit pair and int8 scale
    b[:, 208:210] = rand_f16(rng, n_blocks, 0.00002, 0.0002).view(np.uint8).reshape(n_blocks, 2)
    return b.tobytes()


# ------------------------------------------------------------------ independent decoders (ggml formulation)
def dec_q5_0(raw):
    """w[j] = d * ((nibble j | bit j of qh << 4) - 16); nibbles: low halves are weights 0..15, high 16..31."""
    out = []
    for i in range(0, len(raw), 22):
        d = np.frombuffer(raw[i:i + 2], np.float16)[0].astype(np.float32)
        qh = struct.unpack("<I", raw[i + 2:i + 6])[0]
        qs = raw[i + 6:i + 22]
        for j in range(32):
            nib = (qs[j] & 15) if j < 16 else (qs[j - 16] >> 4)
            out.append(d * np.float32((nib | (((qh >> j) & 1) << 4)) - 16))
    return np.array(out, np.float32)


def dec_q6_k(raw):
    """Per 128 weights: weight 32 j + l (j = 0..3, l = 0..31) has its low nibble in ql[l + 32 (j & 1)] (low half for
    j < 2, high half else), its upper two bits at bit 2 j of qh[l], and the int8 scale 2 j + l // 16 of the half;
    w = d * scale * (q - 32), left to right in float32."""
    out = []
    for i in range(0, len(raw), 210):
        ql, qh = raw[i:i + 128], raw[i + 128:i + 192]
        sc = np.frombuffer(raw[i + 192:i + 208], np.int8)
        d = np.frombuffer(raw[i + 208:i + 210], np.float16)[0].astype(np.float32)
        for half in range(2):
            for j in range(4):
                for l in range(32):
                    byte = ql[64 * half + l + 32 * (j & 1)]
                    low = (byte & 15) if j < 2 else (byte >> 4)
                    q = low | (((qh[32 * half + l] >> (2 * j)) & 3) << 4)
                    out.append(d * np.float32(sc[8 * half + 2 * j + l // 16]) * np.float32(q - 32))
    return np.array(out, np.float32)

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
    write_gguf(p, {"general.architecture": "llama"}, [("x.weight", (2, 128), 10, b"\0" * 84)])     # Q2_K: not read
    f = gguf.GGUFFile(str(p))
    with pytest.raises(NotImplementedError, match="x.weight"):
        f.tensor("x.weight")
    f.close()
    write_gguf(p, {"general.architecture": "llama"}, [("y.weight", (2, 64), gguf.GGML_Q4_0, make_q4_0(rng, 2))])   # too short
    f = gguf.GGUFFile(str(p))
    with pytest.raises(ValueError, match="past the end"):
        f.tensor("y.weight")
    f.close()


def _float_matrix(rng, gtype, n):
    w = (rng.standard_normal(n) * 0.05).astype(np.float32)
    if gtype == gguf.GGML_F16:
        return w.astype(np.float16).tobytes()
    if gtype == gguf.GGML_BF16:
        return (w.view(np.uint32) >> 16).astype(np.uint16).tobytes()
    return w.tobytes()


def _model_file(path, arch, rng, mixed=False):
    """mixed: the tensor types of a Q4_K_M-style file and of float exports -- Q6_K for V, down and the output /
    tied embedding matrix, Q5_0 for K, F16 / BF16 / F32 matrices for O, up and gate of the second layer."""
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
        if mixed:
            repl = {f"{p}.attn_k.weight": (gguf.GGML_Q5_0, make_q5_0(rng, KV * D * E // 32)),
                    f"{p}.attn_v.weight": (gguf.GGML_Q6_K, make_q6_k(rng, KV * D * E // 256)),
                    f"{p}.ffn_down.weight": (gguf.GGML_Q6_K, make_q6_k(rng, E * FF // 256)),
                    f"{p}.attn_output.weight": (gguf.GGML_F16, _float_matrix(rng, gguf.GGML_F16, E * H * D)),
                    f"{p}.ffn_up.weight": (gguf.GGML_BF16, _float_matrix(rng, gguf.GGML_BF16, FF * E))}
            if i == 1:
                repl[f"{p}.ffn_gate.weight"] = (gguf.GGML_F32, _float_matrix(rng, gguf.GGML_F32, FF * E))
            ts[-9:] = [(n, sh, *repl[n]) if n in repl else (n, sh, gt, raw) for n, sh, gt, raw in ts[-9:]]
        if arch == "gemma3":
            ts += [(f"{p}.attn_q_norm.weight", (D,), gguf.GGML_F32, norm(D)), (f"{p}.attn_k_norm.weight", (D,), gguf.GGML_F32, norm(D)),
                   (f"{p}.post_attention_norm.weight", (E,), gguf.GGML_F32, norm(E)),
                   (f"{p}.post_ffw_norm.weight", (E,), gguf.GGML_F32, norm(E))]
    ts.append(("output_norm.weight", (E,), gguf.GGML_F32, norm(E)))
    if mixed:      # tied: Q6_K embedding = LM head; untied: F16 embedding rows on the host, Q6_K output matrix
        ts.append(("token_embd.weight", (V, E), gguf.GGML_Q6_K, make_q6_k(rng, V * E // 256)) if arch == "gemma3" else
                  ("token_embd.weight", (V, E), gguf.GGML_F16, _float_matrix(rng, gguf.GGML_F16, V * E)))
    else:
        ts.append(("token_embd.weight", (V, E), gguf.GGML_Q4_K if arch == "gemma3" else gguf.GGML_Q8_0,
                   make_q4_k(rng, V * E // 256) if arch == "gemma3" else make_q8_0(rng, V * E // 32)))
    if arch == "llama":
        ts.append(("output.weight", (V, E), gguf.GGML_Q6_K, make_q6_k(rng, V * E // 256)) if mixed else
                  ("output.weight", (V, E), gguf.GGML_Q8_0, make_q8_0(rng, V * E // 32)))
        ts.append(("rope_freqs.weight", (D // 2,), gguf.GGML_F32, np.ones(D // 2, np.float32).tobytes()))
    write_gguf(path, md, ts)


@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("arch", ["llama", "gemma3"])
def test_model_from_file_decodes_like_the_reference_forward(tmp_path, arch, mixed):
    p = tmp_path / f"{arch}.gguf"
    _model_file(str(p), arch, np.random.default_rng(7), mixed=mixed)
    cfg, tensors = gguf.load_model(str(p))
    if mixed:
        kinds = {n: getattr(v, "kind", None) for n, v in tensors.items()}
        assert kinds["blk.0.attn_k.weight"] == 'q8_0' and kinds["blk.1.ffn_gate.weight"] == 'q4_req'
        assert kinds["blk.0.attn_v.weight"] == kinds["blk.0.attn_output.weight"] == kinds["blk.1.ffn_up.weight"] == 'q4_req'
        assert kinds["output.weight" if arch == "llama" else "token_embd.weight"] == 'q4_req' 
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


def test_q5_0_q6_k_bf16_decoders_and_requantised_upload(tmp_path):
    """Q5_0 -> signed 8-bit codes with scale |d|: bit-exact against the ggml form, negative and zero scales
    included.  Q6_K and BF16 decode bit-exactly; as weight matrices they (and F16 / F32 matrices) come back from
    load_model in the reference's re-quantised form -- scale = (max - min) / 15, zero point = min per 32 weights,
    codes from the map's quantiser -- and what the op surface then holds equals QTensor.dequant()."""
    rng = np.random.default_rng(5)
    r5, r6 = make_q5_0(rng, 16), make_q6_k(rng, 4)
    bf = (rng.standard_normal(128).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    f16 = rng.standard_normal(128).astype(np.float16)
    f32 = rng.standard_normal(128).astype(np.float32)
    p = tmp_path / "m.gguf"
    write_gguf(p, {"general.architecture": "llama", "llama.vocab_size": 8},
               [("blk.0.a.weight", (8, 64), gguf.GGML_Q5_0, r5), ("blk.0.b.weight", (4, 256), gguf.GGML_Q6_K, r6),
                ("blk.0.c.weight", (2, 64), gguf.GGML_BF16, bf.tobytes()), ("blk.0.d.weight", (2, 64), gguf.GGML_F16, f16.tobytes()),
                ("blk.0.e.weight", (4, 32), gguf.GGML_F32, f32.tobytes()), ("blk.0.n.weight", (128,), gguf.GGML_BF16, bf.tobytes())])
    f = gguf.GGUFFile(str(p))
    t5 = f.tensor("blk.0.a.weight")
    # default: the codes of the reference's default path, round(w / |d|) clipped to [-16, 15] (engine.py:1171-1179) --
    # the ggml values except for q = 0 under a negative d, whose +16 becomes 15
    w5 = dec_q5_0(r5).reshape(-1, 32)
    d5 = np.abs(np.frombuffer(r5, np.uint8).reshape(-1, 22)[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1))
    d5 = np.where(d5 > 0, d5, np.float32(1.0))
    ref_codes = np.round(w5 / d5[:, None]).astype(np.int16).clip(-16, 15)
    assert t5.kind == 'q8_0' and np.array_equal(t5.codes.reshape(-1, 32).astype(np.int16) - 128, ref_codes)
    assert np.array_equal(t5.d.astype(np.float32), d5)
    neg = np.frombuffer(r5, np.uint8).reshape(-1, 22)[:, 0:2].copy().view(np.float16).reshape(-1) < 0
    assert np.any((np.round(w5 / d5[:, None]) == 16)[neg]), "the fixture must hold a q = 0 under a negative d"
    # clip=False: exact for every block -- equal to the ggml form as numbers (a d = 0 block gives -0.0 for negative
    # codes in the ggml form, +0.0 here)
    t5x = quant.from_gguf_q5_0(r5, (8, 64), clip=False)
    assert np.array_equal(t5x.dequant().reshape(-1), dec_q5_0(r5))
    differ = t5x.codes != t5.codes
    assert np.array_equal(differ.reshape(-1, 32), np.round(w5 / d5[:, None]) == 16)
    assert np.array_equal(f.tensor("blk.0.b.weight").view(np.uint32).reshape(-1), dec_q6_k(r6).view(np.uint32))
    assert np.array_equal(f.tensor("blk.0.c.weight").view(np.uint32).reshape(-1), bf.astype(np.uint32) << 16)
    f.close()
    cfg, ts = gguf.load_model(str(p))
    assert ts["blk.0.n.weight"].dtype == np.float32 and ts["blk.0.n.weight"].ndim == 1       # 1-D tensors stay float
    src = {"blk.0.b.weight": dec_q6_k(r6), "blk.0.c.weight": (bf.astype(np.uint32) << 16).view(np.float32),
           "blk.0.d.weight": f16.astype(np.float32), "blk.0.e.weight": f32}
    g = oracle.init()
    for name, x in src.items():
        t = ts[name]
        assert t.kind == 'q4_req'
        xb = x.reshape(-1, 32).astype(np.float64)
        want_scale = np.where(xb.max(1) > xb.min(1), (xb.max(1) - xb.min(1)) / 15.0, 1.0).astype(np.float32)
        assert np.array_equal(t.scale, want_scale) and np.array_equal(t.zp, xb.min(1).astype(np.float32))
        # through the op surface: floats scattered into a 4-bit map, read back dequantised
        g.map_create_typed(1, A.DTYPE_Q4, 1, t.size, 32)
        g.set_qparams(1, *t.qparams())
        g.scatter_contiguous(1, 0, t.data)
        h = g.map_gather_dev(1, g.upload_dev(np.arange(t.size, dtype=np.uint32))[0], t.size)[0]
        assert np.array_equal(g.download_dev(h, t.size), t.dequant().reshape(-1)), name
        # the extremes of every group are kept exactly; nothing moves by more than half a step (+ rounding)
        deq = t.dequant().reshape(-1, 32)
        assert np.array_equal(deq.min(1), xb.min(1).astype(np.float32))
        assert np.all(np.abs(deq - x.reshape(-1, 32)) <= 0.5 * want_scale[:, None] * (1 + 1e-5) + 1e-7)
