"""Pins for the oracle that do not come from the oracle: closed forms, invariants, brute force on
tiny inputs, and the reference loader's block decoders restated independently (CPU only)."""
import numpy as np
import pytest

import oracle
from oracle import blocks
from adam_amd import adamah as A
from adam_amd import quant


def up(g, a):
    return g.upload_dev(np.asarray(a, np.uint32))[0]


def f32map(g, mid, n, data=None):
    g.set_dtype(A.DTYPE_F32); g.map_create(mid, 1, n)
    if data is not None:
        g.scatter(mid, np.arange(len(data), dtype=np.uint32), np.asarray(data, np.float32))


def read(g, mid, lo, n):
    return g.gather(mid, np.arange(lo, lo + n, dtype=np.uint32)).view(np.float32).copy()


# ---------------------------------------------------------------- block formats / unpack
def test_q4_0_three_layouts_agree_bit_exactly():
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((8, 64)) * 0.02).astype(np.float32)
    d, codes = blocks.quantize_q4_0(w)
    direct = blocks.dequant_q4_0(d, codes)                                  # (code-8)*d
    via_gguf = blocks.decode_gguf_q4_0(blocks.gguf_q4_0_bytes(d, codes), w.size)   # loader's decoder
    g = oracle.init()
    g.map_create_typed(1, A.DTYPE_Q4, 1, w.size, 32)
    g.set_qparams(1, *blocks.q4_0_qparams(d))
    g.scatter_q4_packed_contiguous(1, 0, blocks.pack_linear_nibbles(codes))
    via_map = g.maps[1].deq(np.arange(w.size))                              # code*scale + zp
    assert np.array_equal(direct.view(np.uint32), via_gguf.view(np.uint32))
    assert np.array_equal(direct.view(np.uint32), via_map.view(np.uint32))
    # product-side packer makes the same bytes / scales
    qt = quant.quantize_q4_0(w)
    assert np.array_equal(qt.codes, blocks.pack_linear_nibbles(codes)) and np.array_equal(qt.d, d)
    assert np.array_equal(qt.dequant().reshape(-1).view(np.uint32), direct.view(np.uint32))
    d2, c2 = blocks.gguf_q4_0_to_codes(blocks.gguf_q4_0_bytes(d, codes), w.size)
    assert np.array_equal(d2, d) and np.array_equal(c2, codes)
    qt2 = quant.from_gguf_q4_0(blocks.gguf_q4_0_bytes(d, codes), w.shape)
    assert np.array_equal(qt2.codes, qt.codes)


def test_q8_0_layouts_agree_bit_exactly():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((4, 96)) * 0.02).astype(np.float32)
    d, q = blocks.quantize_q8_0(w)
    direct = blocks.dequant_q8_0(d, q)
    via_gguf = blocks.decode_gguf_q8_0(blocks.gguf_q8_0_bytes(d, q), w.size)
    g = oracle.init()
    g.map_create_typed(2, A.DTYPE_Q8, 1, w.size, 32)
    g.set_qparams(2, *blocks.q8_0_qparams(d))
    g.scatter_contiguous(2, 0, blocks.q8_to_u8(q))
    via_map = g.maps[2].deq(np.arange(w.size))
    assert np.array_equal(direct.view(np.uint32), via_gguf.view(np.uint32))
    assert np.array_equal(direct.view(np.uint32), via_map.view(np.uint32))
    qt = quant.quantize_q8_0(w)
    assert np.array_equal(qt.codes, blocks.q8_to_u8(q)) and np.array_equal(qt.d, d)
    assert np.array_equal(quant.from_gguf_q8_0(blocks.gguf_q8_0_bytes(d, q), w.shape).codes, qt.codes)


def test_affine_form_equals_offset_form_for_every_code_and_fp16_scale():
    # code*d + (-off*d) == (code-off)*d bit for bit whenever d is fp16-representable
    d = np.arange(1, 0x7C00, 7, dtype=np.uint16).view(np.float16).astype(np.float32)
    for off, ncode in ((8, 16), (128, 256)):
        c = np.arange(ncode, dtype=np.float32)[:, None]
        a = (c * d[None, :] + (np.float32(-off) * d)[None, :]).astype(np.float32)
        b = ((c - np.float32(off)) * d[None, :]).astype(np.float32)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_nibble_position_and_group_indexing_brute_force():
    # every nibble value at every position of a word, groups by absolute element index
    g = oracle.init()
    n = 16 * 8
    g.map_create_typed(1, A.DTYPE_Q4, 1, n, 8)
    scales = (np.arange(n // 8) + 1).astype(np.float32)
    zps = -(np.arange(n // 8)).astype(np.float32)
    g.set_qparams(1, scales, zps)
    words = np.zeros(n // 8, np.uint32)
    for v in range(16):
        for pos in range(8):
            words[v] |= np.uint32(((v + pos) % 16) << (4 * pos))
    g.scatter_q4_packed_contiguous(1, 0, words.view(np.uint8))
    got = g.maps[1].deq(np.arange(n))
    for i in range(n):
        w, pos = divmod(i, 8)
        assert got[i] == np.float32((w + pos) % 16) * scales[i // 8] + zps[i // 8]


def test_device_quantiser_roundtrip_and_clamp():
    g = oracle.init()
    g.map_create_typed(1, A.DTYPE_Q4, 1, 32, 32)
    g.set_qparams(1, np.array([0.5], np.float32), np.array([-1.0], np.float32))
    x = np.array([-9.0, -1.0, -0.5, 0.0, 6.5, 100.0] + [0.0] * 26, np.float32)
    g.scatter(1, np.arange(32, dtype=np.uint32), x)
    codes = g.maps[1].codes(np.arange(6))
    assert codes.tolist() == [0, 0, 1, 2, 15, 15]


# ---------------------------------------------------------------- GEMV
def _gemv_setup(g, W_codes_u8, scale, zp, x, N, K, dtype, group=32):
    g.map_create_typed(1, dtype, 1, N * K, group)
    g.set_qparams(1, scale, zp)
    if dtype == A.DTYPE_Q4:
        g.scatter_q4_packed_contiguous(1, 0, W_codes_u8)
    else:
        g.scatter_contiguous(1, 0, W_codes_u8)
    f32map(g, 0, K + N, x)
    return up(g, [0]), up(g, [0]), up(g, [K])


def test_gemv_integer_special_case_is_exact():
    rng = np.random.default_rng(3)
    N, K = 24, 64
    codes = rng.integers(0, 16, N * K).astype(np.uint8)
    x = rng.integers(-4, 5, K).astype(np.float32)
    g = oracle.init()
    a, b, c = _gemv_setup(g, blocks.pack_linear_nibbles(codes), np.ones(N * K // 32, np.float32),
                          np.zeros(N * K // 32, np.float32), x, N, K, A.DTYPE_Q4)
    g.map_matmul_t_xq4_dev(0, 1, a, b, c, 1, K, N)
    want = codes.reshape(N, K).astype(np.int64) @ x.astype(np.int64)
    assert np.array_equal(read(g, 0, K, N), want.astype(np.float32))


def test_gemv_matches_independent_float64_and_is_linear():
    rng = np.random.default_rng(4)
    N, K = 40, 96
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    qt = quant.quantize_q4_0(w)
    x1, x2 = rng.standard_normal(K).astype(np.float32), rng.standard_normal(K).astype(np.float32)
    ys = []
    for x in (x1, x2, x1 + x2):
        g = oracle.init()
        a, b, c = _gemv_setup(g, qt.codes, *qt.qparams(), x, N, K, A.DTYPE_Q4)
        g.map_matmul_t_xq4_dev(0, 1, a, b, c, 1, K, N)
        ys.append(read(g, 0, K, N))
        want = qt.dequant().astype(np.float64) @ x.astype(np.float64)
        assert np.linalg.norm(ys[-1] - want) / np.linalg.norm(want) < 1e-6
    assert np.allclose(ys[0] + ys[1], ys[2], rtol=0, atol=1e-5)
    # row permutation of W permutes y
    perm = rng.permutation(N)
    qp = quant.quantize_q4_0(w[perm])
    g = oracle.init()
    a, b, c = _gemv_setup(g, qp.codes, *qp.qparams(), x1, N, K, A.DTYPE_Q4)
    g.map_matmul_t_xq4_dev(0, 1, a, b, c, 1, K, N)
    assert np.array_equal(read(g, 0, K, N), ys[0][perm])


def test_matmul_M_gt_1_and_non_transposed_against_numpy():
    rng = np.random.default_rng(5)
    M, K, N = 3, 32, 8
    w = (rng.standard_normal((N, K))).astype(np.float32)
    qt = quant.quantize_q8_0(w)
    A_ = rng.standard_normal((M, K)).astype(np.float32)
    g = oracle.init()
    g.map_create_typed(2, A.DTYPE_Q8, 1, N * K, 32)
    g.set_qparams(2, *qt.qparams()); g.scatter_contiguous(2, 0, qt.codes)
    f32map(g, 0, M * K + M * N + 64, A_.reshape(-1))
    a, b, c = up(g, [0]), up(g, [0]), up(g, [M * K])
    g.map_matmul_t_xq8_dev(0, 2, a, b, c, M, K, N)
    assert np.allclose(read(g, 0, M * K, M * N).reshape(M, N), A_ @ qt.dequant().T, rtol=1e-5, atol=1e-5)
    # non-transposed: the same bytes read as B[K', N'] with K'=N, N'=K
    A2 = rng.standard_normal((M, N)).astype(np.float32)
    f32map(g, 0, M * N + M * K + 64, A2.reshape(-1))
    c2 = up(g, [M * N])
    g.map_matmul_xq8_dev(0, 2, a, b, c2, M, N, K)
    assert np.allclose(read(g, 0, M * N, M * K).reshape(M, K), A2 @ qt.dequant(), rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- norms / rope
def test_rmsnorm_closed_forms():
    g = oracle.init()
    dim, eps = 48, 1e-6
    w = np.linspace(0.5, 2.0, dim).astype(np.float32)
    f32map(g, 0, 4 * dim, np.concatenate([np.ones(dim), w]))
    s, wt, d = up(g, [0]), up(g, [dim]), up(g, [2 * dim])
    g.map_rmsnorm_dev(0, s, wt, d, 1, dim, eps)
    assert np.allclose(read(g, 0, 2 * dim, dim), w / np.sqrt(1 + eps), rtol=1e-6)
    rng = np.random.default_rng(6)
    x = rng.standard_normal(dim).astype(np.float32)
    outs = []
    for alpha in (1.0, 37.5):
        f32map(g, 0, 4 * dim, np.concatenate([x * alpha, w]))
        g.map_rmsnorm_dev(0, s, wt, d, 1, dim, 0.0)
        outs.append(read(g, 0, 2 * dim, dim))
    assert np.allclose(outs[0], outs[1], rtol=2e-6)          # scale invariance at eps = 0
    assert np.allclose(outs[0], x / np.sqrt(np.mean(x.astype(np.float64) ** 2)) * w, rtol=1e-5)
    r = up(g, [3 * dim])
    g.scatter(0, np.arange(3 * dim, 4 * dim, dtype=np.uint32), np.full(dim, 2.0, np.float32))
    g.map_rmsnorm_add_dev(0, s, wt, r, d, 1, dim, 0.0)
    assert np.allclose(read(g, 0, 2 * dim, dim), outs[1] + 2.0, rtol=2e-6)


def test_rope_identity_norm_composition_and_literal():
    g = oracle.init()
    H, D = 3, 16
    rng = np.random.default_rng(7)
    x = rng.standard_normal(H * D).astype(np.float32)
    f32map(g, 0, 4 * H * D, x)
    s, d, d2 = up(g, [0]), up(g, [H * D]), up(g, [2 * H * D])
    g.map_rope_dev(0, s, d, 1, H, D, 0, 10000.0)
    assert np.array_equal(read(g, 0, H * D, H * D), x)                      # pos 0 = identity
    g.map_rope_dev(0, s, d, 1, H, D, 5, 10000.0)
    y5 = read(g, 0, H * D, H * D).reshape(H, D)
    xr = x.reshape(H, D)
    assert np.allclose(y5[:, :8] ** 2 + y5[:, 8:] ** 2, xr[:, :8] ** 2 + xr[:, 8:] ** 2, rtol=1e-5)
    g.map_rope_dev(0, d, d2, 1, H, D, 7, 10000.0)                           # R(7) R(5) = R(12)
    g.map_rope_dev(0, s, d, 1, H, D, 12, 10000.0)
    assert np.allclose(read(g, 0, 2 * H * D, H * D), read(g, 0, H * D, H * D), atol=2e-6)
    # literal: dim 4, pos 1, base 10000 -> pair 0 turns by 1 rad, pair 1 by 0.01 rad
    f32map(g, 1, 8, [1.0, 1.0, 0.0, 0.0])
    g.map_rope_dev(1, up(g, [0]), up(g, [4]), 1, 1, 4, 1, 10000.0)
    assert np.allclose(read(g, 1, 4, 4), [np.cos(1.0), np.cos(0.01), np.sin(1.0), np.sin(0.01)], atol=1e-7)


def test_qk_norm_rope_equals_rmsnorm_then_rope_with_eps_1e6():
    g = oracle.init()
    Hq, Hk, D = 2, 1, 8
    rng = np.random.default_rng(8)
    q = rng.standard_normal(Hq * D).astype(np.float32); k = rng.standard_normal(Hk * D).astype(np.float32)
    wq = rng.uniform(0.5, 1.5, D).astype(np.float32); wk = rng.uniform(0.5, 1.5, D).astype(np.float32)
    f32map(g, 0, 128, np.concatenate([q, k, wq, wk]))
    qs = up(g, [0, D]); ks = up(g, [2 * D]); qw = up(g, [3 * D, 3 * D]); kw = up(g, [4 * D])
    g.map_qk_norm_rope_x_dev(0, 0, qs, qw, ks, kw, up(g, [64]), Hq, D, Hk, D, 9, 1e6)
    fused = read(g, 0, 64, (Hq + Hk) * D)
    tq, tk = up(g, [96, 96 + D]), up(g, [96 + 2 * D])
    g.map_rmsnorm_dev(0, qs, qw, tq, Hq, D, 1e-6)
    g.map_rmsnorm_dev(0, ks, kw, tk, Hk, D, 1e-6)
    g.map_rope_dev(0, up(g, [96]), up(g, [40]), 1, Hq + Hk, D, 9, 1e6)
    assert np.allclose(read(g, 0, 40, (Hq + Hk) * D), fused, atol=1e-6)


# ---------------------------------------------------------------- attention / activations
def test_attention_single_key_and_uniform_scores():
    g = oracle.init()
    H, D, T = 2, 8, 5
    rng = np.random.default_rng(9)
    V = rng.standard_normal((T, D)).astype(np.float32)
    f32map(g, 0, 256, np.concatenate([np.zeros(2 * T, np.float32), V.reshape(-1)]))
    sc = up(g, [0, T]); vv = up(g, [2 * T, 2 * T]); out = up(g, [128, 128 + D])
    g.map_attn_softmax_value_dev(0, sc, vv, out, H, 1, D, 0.3, 50.0)
    assert np.array_equal(read(g, 0, 128, D), V[0])                         # seq_len 1 -> V row exactly
    g.map_attn_softmax_value_dev(0, sc, vv, out, H, T, D, 0.3, 0.0)
    assert np.allclose(read(g, 0, 128, D), V.mean(axis=0), atol=1e-6)       # uniform scores -> mean of V
    assert np.array_equal(read(g, 0, 128, D), read(g, 0, 128 + D, D))       # equal q in one group -> equal out


def test_gated_activation_literals():
    g = oracle.init()
    f32map(g, 0, 16, [1.0, -2.0, 0.5, 3.0, 2.0, 2.0, 2.0, 0.5])
    a, b, d = up(g, [0, 1, 2, 3]), up(g, [4, 5, 6, 7]), up(g, [8, 9, 10, 11])
    g.map_op2_dev(0, A.OP_GEGLU, a, b, d, 4)
    gelu = lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))
    assert np.allclose(read(g, 0, 8, 4), [2 * gelu(1.0), 2 * gelu(-2.0), 2 * gelu(0.5), 0.5 * gelu(3.0)], atol=1e-6)
    assert abs(read(g, 0, 8, 1)[0] - 2 * 0.8411920) < 1e-6                  # tanh-GELU(1) = 0.841192
    g.map_op2_dev(0, A.OP_SWIGLU, a, b, d, 4)
    assert abs(read(g, 0, 8, 1)[0] - 2 * 0.7310586) < 1e-6                  # SiLU(1) = sigmoid(1)
    g.map_op1_dev(0, A.OP_TANH, a, d, 4)
    assert np.allclose(read(g, 0, 8, 4), np.tanh([1.0, -2.0, 0.5, 3.0]), atol=1e-7)
    g.map_broadcast_dev(0, A.OP_MUL, a, up(g, [4, 4, 4, 4]), d, 4)
    assert np.array_equal(read(g, 0, 8, 4), np.array([2.0, -4.0, 1.0, 6.0], np.float32))


def test_row_copy_rounds_to_fp16_inside_the_kv_range_only():
    g = oracle.init()
    vals = np.array([1.0001, 3.14159, -2.71828, 1e-3], np.float32)
    f32map(g, 0, 64, vals)
    g.kv_cache_fp16(0, 32, 16)
    g.map_row_copy_offset_dev(0, up(g, [0, 2]), up(g, [0]), 0, 1, 4)        # dst row 2 -> 8..11 (outside)
    g.map_row_copy_offset_dev(0, up(g, [0, 2]), up(g, [0]), 6, 1, 4)        # dst row 8 -> 32..35 (inside)
    assert np.array_equal(read(g, 0, 8, 4), vals)
    assert np.array_equal(read(g, 0, 32, 4), vals.astype(np.float16).astype(np.float32))


# ---------------------------------------------------------------- argmax tail
@pytest.mark.parametrize("dtype", ["q4", "q8"])
def test_matvec_argmax_equals_argmax_of_matvec(dtype):
    rng = np.random.default_rng(10)
    N, K, rpg = 70, 64, 16                                                 # N not a multiple of rpg
    w = rng.standard_normal((N, K)).astype(np.float32)
    w[33] = w[12]                                                          # exact tie between rows
    qt = quant.quantize_q4_0(w) if dtype == "q4" else quant.quantize_q8_0(w)
    x = rng.standard_normal(K).astype(np.float32)
    y = qt.dequant().astype(np.float64) @ x.astype(np.float64)
    boost = np.zeros(N); boost[[12, 33]] = 0.0
    g = oracle.init()
    mid, dt = (1, A.DTYPE_Q4) if dtype == "q4" else (2, A.DTYPE_Q8)
    g.map_create_typed(mid, dt, 1, N * K, 32)
    g.set_qparams(mid, *qt.qparams())
    if dtype == "q4":
        g.scatter_q4_packed_contiguous(mid, 0, qt.codes)
    else:
        g.scatter_contiguous(mid, 0, qt.codes)
    ng = (N + rpg - 1) // rpg
    f32map(g, 0, K + 2 * ng + 8, x)
    fn = g.map_matvec_argmax_t_xq4_dev if dtype == "q4" else g.map_matvec_argmax_t_xq8_dev
    fn(0, mid, up(g, [0]), up(g, [0]), up(g, np.arange(K, K + ng)), up(g, np.arange(K + ng, K + 2 * ng)),
       up(g, [K + 2 * ng]), K, N, rpg)
    tok = int(read(g, 0, K + 2 * ng, 1)[0])
    assert tok == int(np.argmax(y.astype(np.float32)))
    pidx = read(g, 0, K, ng).astype(int); pval = read(g, 0, K + ng, ng)
    for gi in range(ng):
        seg = y[gi * rpg:(gi + 1) * rpg].astype(np.float32)
        assert pidx[gi] == gi * rpg + int(np.argmax(seg)) and pval[gi] == seg.max()


def test_argmax_tie_nan_and_empty():
    g = oracle.init()
    f32map(g, 0, 16, [np.nan, 2.0, 7.0, 7.0, np.nan, -1.0])
    g.map_argmax_dev(0, up(g, np.arange(6)), up(g, [8]), 6)
    assert read(g, 0, 8, 1)[0] == 2.0
    f32map(g, 0, 16, [np.nan, np.nan])
    g.map_argmax_dev(0, up(g, np.arange(2)), up(g, [8]), 2)
    assert read(g, 0, 8, 1)[0] == 0.0                                       # all NaN -> first index


# ---------------------------------------------------------------- error behaviour
def test_error_codes():
    g = oracle.init()
    with pytest.raises(RuntimeError, match="code -3"):
        g.map_op2_dev(5, 0, 1, 1, 1, 1)                                     # unknown map
    f32map(g, 0, 8)
    with pytest.raises(RuntimeError, match="code -3"):
        g.map_op2_dev(0, 0, 99, 99, 99, 1)                                  # unknown handle
    g.map_create_typed(1, A.DTYPE_Q4, 1, 64, 32)
    with pytest.raises(RuntimeError, match="code -3"):
        g.set_qparams(1, np.ones(3, np.float32), np.zeros(3, np.float32))   # more groups than the map has
    with pytest.raises(RuntimeError, match="code -3"):
        g.scatter_q4_packed_contiguous(1, 1, np.zeros(2, np.uint8))         # odd start
    h, _ = g.upload_dev(np.zeros(4, np.uint32))
    assert g.upload_dev(np.zeros(5, np.uint32), handle=h)[0] == 0           # size change on re-upload


# ---- sampling tail: what the definitions fix, independent of the oracle's loops --------------------
def _sampling_map(g, vals, n=256):
    f32map(g, 2, n, np.zeros(n, np.float32))
    g.scatter(2, np.arange(len(vals), dtype=np.uint32), np.asarray(vals, np.float32))


def test_topk_equals_stable_sort_with_nan_lowest():
    g = oracle.init()
    rng = np.random.default_rng(3)
    v = rng.integers(-5, 6, 100).astype(np.float32)          # many ties
    v[[7, 50]] = np.nan
    _sampling_map(g, v)
    g.map_topk_dev(2, up(g, np.arange(100)), up(g, 128 + np.arange(64)), up(g, 192 + np.arange(64)), 100, 64)
    clean = np.where(np.isnan(v), np.float32(-3.402823466e+38), v)
    order = np.lexsort((np.arange(100), -clean.astype(np.float64)))[:64]   # value descending, then index ascending
    assert read(g, 2, 128, 64).astype(np.int64).tolist() == order.tolist()
    assert np.array_equal(read(g, 2, 192, 64), clean[order])
    # more rounds than candidates: the surplus stores index 0 and the lowest float
    _sampling_map(g, [1.0, 3.0])
    g.map_topk_dev(2, up(g, [0, 1]), up(g, [8, 9, 10]), up(g, [12, 13, 14]), 2, 3)
    assert read(g, 2, 8, 3).tolist() == [1.0, 0.0, 0.0]
    assert read(g, 2, 12, 3).tolist() == [3.0, 1.0, np.float32(-3.402823466e+38)]


def test_topp_closed_forms():
    g = oracle.init()
    logits = np.array([2.0, 1.0, 0.5, -1.0, -3.0], np.float32)
    sm = lambda t: np.exp((logits.astype(np.float64) - 2.0) / t) / np.exp((logits.astype(np.float64) - 2.0) / t).sum()
    for temp, top_p in [(1.0, 1.0), (0.7, 0.8), (2.0, 0.5), (1.0, 0.0)]:
        _sampling_map(g, logits)
        g.map_topp_dev(2, up(g, np.arange(5)), up(g, 16 + np.arange(5)), 5, temp, top_p)
        p = sm(temp)
        # map_topp.comp:77 leaves the prefix loop at once when top_p >= 0.999999: one candidate is kept
        keep = 1 if top_p >= 0.999999 else int(np.searchsorted(np.cumsum(p), top_p - 1e-9) + 1)
        want = np.zeros(5); want[:keep] = p[:keep] / p[:keep].sum()
        assert np.allclose(read(g, 2, 16, 5), want, atol=2e-6), (temp, top_p)
    # all candidates unusable -> zeros; a single usable one -> probability one on it
    _sampling_map(g, [np.nan, np.inf, -np.inf])
    g.map_topp_dev(2, up(g, [0, 1, 2]), up(g, [16, 17, 18]), 3, 1.0, 0.9)
    assert read(g, 2, 16, 3).tolist() == [0.0, 0.0, 0.0]
    _sampling_map(g, [np.nan, 4.0, np.nan])
    g.map_topp_dev(2, up(g, [0, 1, 2]), up(g, [16, 17, 18]), 3, 1.0, 0.5)
    assert read(g, 2, 16, 3).tolist() == [0.0, 1.0, 0.0]


def test_categorical_is_the_inverse_cdf_and_repeat_penalty_is_its_own_inverse():
    g = oracle.init()
    p = np.array([0.1, 0.0, 0.4, 0.5], np.float32); ids = np.array([7.0, 8.0, 9.0, 10.0], np.float32)
    edges = np.cumsum(p.astype(np.float64))
    for r in [0.0, 0.05, 0.0999, 0.1001, 0.49, 0.51, 0.999, 1.0, 7.0, -2.0, np.nan]:
        _sampling_map(g, np.concatenate([p, ids, [r]]))
        g.map_sample_categorical_dev(2, up(g, [4, 5, 6, 7]), up(g, [0, 1, 2, 3]), up(g, [8]), up(g, [9]), 4)
        rr = 0.0 if not np.isfinite(r) else min(max(r, 0.0), 0.99999994)
        want = ids[int(np.searchsorted(edges, rr * edges[-1], side="right"))]
        assert read(g, 2, 9, 1)[0] == want, r
    _sampling_map(g, np.concatenate([np.zeros(4), ids, [0.3]]))       # zero mass -> first candidate
    g.map_sample_categorical_dev(2, up(g, [4, 5, 6, 7]), up(g, [0, 1, 2, 3]), up(g, [8]), up(g, [9]), 4)
    assert read(g, 2, 9, 1)[0] == 7.0
    logits = np.array([2.0, -1.0, 0.0, 3.0, -4.0], np.float32)
    _sampling_map(g, logits)
    locs, toks = up(g, np.arange(5)), up(g, [3, 1, 4])
    g.map_repeat_penalty_dev(2, locs, toks, 3, 2.0)
    assert read(g, 2, 0, 5).tolist() == [2.0, -2.0, 0.0, 1.5, -8.0]
    g.map_repeat_penalty_dev(2, locs, toks, 3, 0.5)
    assert read(g, 2, 0, 5).tolist() == logits.tolist()


def test_resolve_idx_guards():
    g = oracle.init()
    vals = np.zeros(32, np.float32)
    vals[4:8] = [11.0, -5.0, np.nan, 44.0]; vals[8:13] = [3.0, 1.0, 2.0, -1.0, np.inf]
    _sampling_map(g, vals)
    g.map_resolve_idx_dev(2, up(g, [4]), up(g, [8, 9, 10, 11, 12]), up(g, 16 + np.arange(5)), 5)
    assert read(g, 2, 16, 5).tolist() == [44.0, 0.0, 0.0, 11.0, 11.0]


# ---------------------------------------------------------------- GEMV + partial top-k, rerank
def _load_q(g, mid, qt):
    dt = A.DTYPE_Q4 if qt.kind == "q4_0" else A.DTYPE_Q8
    g.map_create_typed(mid, dt, 1, qt.size, 32)
    g.set_qparams(mid, *qt.qparams())
    if qt.kind == "q4_0":
        g.scatter_q4_packed_contiguous(mid, 0, qt.codes)
    else:
        g.scatter_contiguous(mid, 0, qt.codes)


@pytest.mark.parametrize("dtype", ["q4", "q8"])
def test_matvec_topk_equals_insertion_into_a_sorted_list(dtype):
    """Independent statement of the list the shader builds: rows visited in order, each inserted before
    the first entry it beats (value greater, or equal with a smaller row), list cut at k."""
    rng = np.random.default_rng(12)
    N, K, k, rpg = 50, 64, 6, 16                               # last group has 2 rows < k
    w = rng.standard_normal((N, K)).astype(np.float32)
    w[21] = w[18]                                              # exact tie inside group 1
    qt = quant.quantize_q4_0(w) if dtype == "q4" else quant.quantize_q8_0(w)
    x = rng.standard_normal(K).astype(np.float32)
    y = (qt.dequant().astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    pen, rp = [18, 3, 3, 49, 77], np.float32(1.5)              # a duplicate and an id past N
    for r in set(pen):
        if r < N:
            y[r] = y[r] / rp if y[r] > 0 else y[r] * rp
    g = oracle.init()
    _load_q(g, 1, qt)
    ng = (N + rpg - 1) // rpg
    f32map(g, 0, K + 2 * ng * k + 8, x)
    fn = g.map_matvec_topk_t_xq4_ex_dev if dtype == "q4" else g.map_matvec_topk_t_xq8_ex_dev
    fn(0, 1, up(g, [0]), up(g, [0]), up(g, pen), up(g, K + np.arange(ng * k)), up(g, K + ng * k + np.arange(ng * k)),
       K, N, k, len(pen), float(rp), rpg)
    idx = read(g, 0, K, ng * k).reshape(ng, k); val = read(g, 0, K + ng * k, ng * k).reshape(ng, k)
    for gi in range(ng):
        lst = []
        for r in range(gi * rpg, min(N, (gi + 1) * rpg)):
            pos = len(lst)
            for i, (v, j) in enumerate(lst):
                if y[r] > v or (y[r] == v and r < j):
                    pos = i
                    break
            lst.insert(pos, (y[r], r))
            lst = lst[:k]
        for t in range(k):
            if t < len(lst):
                assert idx[gi, t] == lst[t][1] and val[gi, t] == lst[t][0]
            else:
                assert idx[gi, t] == 0 and val[gi, t] == np.float32(-3.402823466e+38)


def test_rerank_equals_row_dot_products():
    rng = np.random.default_rng(13)
    N, K = 40, 64
    qt = quant.quantize_q8_0(rng.standard_normal((N, K)).astype(np.float32))
    x = rng.standard_normal(K).astype(np.float32)
    y = qt.dequant().astype(np.float64) @ x.astype(np.float64)
    partial = np.array([7, 39, 0, 12, 12, 5], np.float32); sel = np.array([4, 1, 0, 5], np.float32)
    g = oracle.init()
    _load_q(g, 2, qt)
    f32map(g, 0, K + 64, np.concatenate([x, partial, sel]))
    g.map_matvec_rerank_t_xq8_dev(0, 2, up(g, [0]), up(g, [0]), up(g, [K]), up(g, K + 6 + np.arange(4)), up(g, [39, 5]),
                                  up(g, K + 20 + np.arange(4)), up(g, K + 30 + np.arange(4)), K, 4, 2, 2.0)
    toks = read(g, 0, K + 20, 4).astype(int).tolist(); vals = read(g, 0, K + 30, 4)
    assert toks == [12, 39, 7, 5]
    exp = [y[12], y[39] / 2 if y[39] > 0 else y[39] * 2, y[7], y[5] / 2 if y[5] > 0 else y[5] * 2]
    assert np.allclose(vals, np.array(exp, np.float32), rtol=1e-6)


def test_fused_projections_equal_their_separate_dot_products():
    rng = np.random.default_rng(14)
    K, rows = 64, (6, 2, 3)
    qt = quant.quantize_q4_0(rng.standard_normal((sum(rows), K)).astype(np.float32))
    x = rng.standard_normal(K).astype(np.float32)
    y = (qt.dequant().astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    g = oracle.init()
    _load_q(g, 1, qt)
    f32map(g, 0, K + 32, x)
    # results deliberately out of order: K first, then V, then Q
    g.map_fused_qkv_t_xq4_dev(0, 1, up(g, [0]), up(g, [0]), up(g, [6 * K]), up(g, [8 * K]), up(g, [K + 5]), up(g, [K]),
                              up(g, [K + 2]), K, *rows)
    assert np.array_equal(read(g, 0, K, 2), y[6:8]) and np.array_equal(read(g, 0, K + 2, 3), y[8:11])
    assert np.array_equal(read(g, 0, K + 5, 6), y[0:6])
    q8 = quant.quantize_q8_0(rng.standard_normal((8, K)).astype(np.float32))
    _load_q(g, 2, q8)
    g.map_fused_gateup_act_t_xq8_dev(0, 2, up(g, [0]), up(g, [0]), up(g, [4 * K]), up(g, [K + 16]), K, 4)
    z = q8.dequant().astype(np.float64) @ x.astype(np.float64)
    exp = z[:4] / (1 + np.exp(-z[:4])) * z[4:]
    assert np.allclose(read(g, 0, K + 16, 4), exp, rtol=1e-5)
    with pytest.raises(RuntimeError):
        g.map_fused_qkv_t_xq4_dev(0, 1, up(g, [0]), up(g, [0]), 424242, up(g, [0]), up(g, [K]), up(g, [K]), up(g, [K]), K, 1, 0, 0)


# ---------------------------------------------------------------- ops off the decode path: closed forms
def test_plain_matmuls_on_integer_matrices_with_distinct_shapes():
    """map_matmul_dev (B as [K, N]), map_matmul_t_x_dev (B as [N, K] in a second map) and map_matmul_x_dev (B as
    [K, N] in a second map) on small integer matrices with M, K, N all different and several ops: the products
    are exact in float32, and a transposed operand, a swapped dimension or a wrong base shows up as a mismatch."""
    rng = np.random.default_rng(21)
    M, K, N, n_ops = 3, 5, 7, 2
    Aop = rng.integers(-4, 5, (n_ops, M, K)).astype(np.float32)
    Bkn = rng.integers(-4, 5, (n_ops, K, N)).astype(np.float32)
    want = np.stack([Aop[o].astype(np.int64) @ Bkn[o].astype(np.int64) for o in range(n_ops)]).astype(np.float32)
    g = oracle.init()
    a_sz, b_sz, c_sz = M * K, K * N, M * N
    a0, b0, c0 = 0, n_ops * a_sz + 3, n_ops * (a_sz + b_sz) + 11
    f32map(g, 0, c0 + n_ops * c_sz + 4)
    g.scatter(0, np.arange(a0, a0 + n_ops * a_sz, dtype=np.uint32), Aop.reshape(-1))
    g.scatter(0, np.arange(b0, b0 + n_ops * b_sz, dtype=np.uint32), Bkn.reshape(-1))
    la, lb, lc = (up(g, base + np.arange(n_ops) * sz) for base, sz in ((a0, a_sz), (b0, b_sz), (c0, c_sz)))
    g.map_matmul_dev(0, la, lb, lc, M, K, N, n_ops)
    assert np.array_equal(read(g, 0, c0, n_ops * c_sz), want.reshape(-1))
    # weights in a second f32 map: [K, N] for map_matmul_x_dev, [N, K] for map_matmul_t_x_dev
    f32map(g, 3, 2 * n_ops * b_sz + 5)
    g.scatter(3, np.arange(2, 2 + n_ops * b_sz, dtype=np.uint32), Bkn.reshape(-1))
    g.scatter(3, np.arange(2 + n_ops * b_sz, 2 + 2 * n_ops * b_sz, dtype=np.uint32), Bkn.transpose(0, 2, 1).reshape(-1))
    for fn, base in ((g.map_matmul_x_dev, 2), (g.map_matmul_t_x_dev, 2 + n_ops * b_sz)):
        g.scatter(0, np.arange(c0, c0 + n_ops * c_sz, dtype=np.uint32), np.zeros(n_ops * c_sz, np.float32))
        fn(0, 3, la, up(g, base + np.arange(n_ops) * b_sz), lc, M, K, N, n_ops)
        assert np.array_equal(read(g, 0, c0, n_ops * c_sz), want.reshape(-1))


def test_fma_on_exact_values():
    g = oracle.init()
    a = np.array([1.5, -2.0, 0.25, 3.0], np.float32); b = np.array([4.0, 0.5, -8.0, 0.0], np.float32)
    c = np.array([0.5, 1.0, 1.0, -7.0], np.float32)
    f32map(g, 0, 20, np.concatenate([a, b, c]))
    g.map_fma_dev(0, up(g, np.arange(4)), up(g, 4 + np.arange(4)), up(g, 8 + np.arange(4)), up(g, [15, 14, 13, 12]), 4)
    assert read(g, 0, 12, 4).tolist() == [-7.0, -1.0, 0.0, 6.5]          # a*b + c, scattered in reverse


def test_row_softmax_closed_forms():
    """Equal entries -> 1/n; entries ln(1..n) -> k / (n(n+1)/2); a constant shift changes nothing; the row base is
    loc * row_size (not an absolute offset)."""
    g = oracle.init()
    n = 8
    rows = np.stack([np.full(n, 3.25), np.log(np.arange(1, n + 1)), np.log(np.arange(1, n + 1)) + 100.0]).astype(np.float32)
    f32map(g, 0, 8 * n, np.concatenate([np.zeros(n), rows.reshape(-1)]))          # rows 1, 2, 3 of size n
    g.map_softmax_dev(0, up(g, [1, 2, 3]), up(g, [5, 6, 7]), n, 3)
    out = read(g, 0, 5 * n, 3 * n).reshape(3, n)
    assert np.allclose(out[0], 1.0 / n, rtol=1e-6)
    tri = np.arange(1, n + 1) / (n * (n + 1) / 2)
    assert np.allclose(out[1], tri, rtol=1e-5) and np.allclose(out[2], tri, rtol=1e-4)
    assert np.allclose(out.sum(axis=1), 1.0, rtol=1e-6)


def test_layernorm_closed_forms():
    """A row a*k + b (k = 0..d-1) has mean b + a(d-1)/2 and variance a^2 (d^2-1)/12, so with gamma = 1, beta = 0
    the result is (k - (d-1)/2) / sqrt((d^2-1)/12) whatever a > 0 and b are; gamma and beta then scale and shift
    per element; source and destination bases are loc * dim, gamma / beta bases absolute."""
    g = oracle.init()
    d = 16
    k = np.arange(d)
    unit = (k - (d - 1) / 2) / np.sqrt((d * d - 1) / 12)
    rows = np.stack([3.0 * k + 7.0, 0.5 * k - 2.0]).astype(np.float32)
    gamma = np.linspace(0.5, 2.0, d).astype(np.float32); beta = np.linspace(-1.0, 1.0, d).astype(np.float32)
    f32map(g, 0, 8 * d, np.concatenate([rows.reshape(-1), np.ones(d), np.zeros(d), gamma, beta]))
    ones, zeros, gm, bt = 2 * d, 3 * d, 4 * d, 5 * d
    g.map_layernorm_dev(0, up(g, [0, 1]), up(g, [6, 7]), up(g, [ones, gm]), up(g, [zeros, bt]), d, 0.0, 2)
    out = read(g, 0, 6 * d, 2 * d).reshape(2, d)
    assert np.allclose(out[0], unit, atol=2e-6)
    assert np.allclose(out[1], unit * gamma + beta, atol=4e-6)
    # eps enters under the root: a constant row gives beta exactly, whatever eps > 0
    g.scatter(0, np.arange(0, d, dtype=np.uint32), np.full(d, 4.0, np.float32))
    g.map_layernorm_dev(0, up(g, [0]), up(g, [6]), up(g, [gm]), up(g, [bt]), d, 1e-5, 1)
    assert np.array_equal(read(g, 0, 6 * d, d), beta)


def test_reduce_over_packs():
    """Per loc, the pack's sum / max / min (op 0 / 1 / 2); source base is loc * pack_size, destination a
    single element offset."""
    g = oracle.init()
    g.set_dtype(A.DTYPE_F32); g.map_create(0, 4, 6)
    vals = np.array([[1, 2, 3, 4], [-5, 0.5, 7, -1], [2, 2, 2, 2]], np.float32)
    g.scatter(0, np.array([0, 1, 2], np.uint32), vals.reshape(-1))
    for op, want in ((0, [10.0, 1.5, 8.0]), (1, [4.0, 7.0, 2.0]), (2, [1.0, -5.0, 2.0])):
        g.map_reduce_dev(0, op, up(g, [0, 1, 2]), up(g, [20, 21, 23]), 3)
        got = g.gather(0, np.array([5], np.uint32)).view(np.float32)      # pack 5 = elements 20..23
        assert [got[0], got[1], got[3]] == want
