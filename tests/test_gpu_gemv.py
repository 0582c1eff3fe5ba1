"""HIP dequant-GEMV against the oracle through the C ABI (needs an MI355X).

Bars: nibble / byte / scale unpacking bit-exact; GEMV outputs within 1e-3 relative L2 of the
oracle (float32 accumulation on the device, float64 in the oracle)."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd import quant
from gpu_util import note, up, f32map, read, rel_l2, load_qtensor

pytestmark = pytest.mark.gpu
TOL = 1e-3


def both(hip):
    return (("hip", hip), ("oracle", oracle.init()))


def run_gemv(g, qt, x, offset=0, scale=None, zp=None, wmap=1):
    N, K = qt.shape
    load_qtensor(g, wmap, qt, offset=offset, scale=scale, zp=zp)
    f32map(g, 0, K + N + 8, x)
    fn = g.map_matmul_t_xq4_dev if qt.kind == 'q4_0' else g.map_matmul_t_xq8_dev
    g.batch_begin()
    fn(0, wmap, up(g, [0]), up(g, [offset]), up(g, [K]), 1, K, N)
    g.batch_end()
    return read(g, 0, K, N)


def test_unpack_bit_exact_block_and_affine(hip):
    rng = np.random.default_rng(11)
    for kind, quantize in (("q4", quant.quantize_q4_0), ("q8", quant.quantize_q8_0)):
        w = (rng.standard_normal((64, 96)) * 0.02).astype(np.float32)
        qt = quantize(w)
        note(f"unpack {kind} block layout")
        load_qtensor(hip, 1, qt)
        assert hip.map_layout(1) == 1
        got = hip.debug_dequant(1, 0, qt.size)
        want = qt.dequant().reshape(-1)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # the dequantising gather (embedding fetch path) gives the same bits
        locs = rng.permutation(qt.size)[:500].astype(np.uint32)
        gh, _, n, _ = hip.map_gather_dev(1, up(hip, locs), locs.size)
        assert np.array_equal(hip.download_dev(gh, n).view(np.uint32), want[locs].view(np.uint32))
        # arbitrary affine qparams (not Q4_0/Q8_0): generic layout, still bit-exact vs the oracle
        note(f"unpack {kind} affine layout")
        s = rng.uniform(0.001, 0.1, qt.size // 32).astype(np.float32)
        z = rng.uniform(-1, 1, qt.size // 32).astype(np.float32)
        o = oracle.init()
        for g in (hip, o):
            load_qtensor(g, 1, qt, scale=s, zp=z)
        assert hip.map_layout(1) == 0
        want = o.maps[1].deq(np.arange(qt.size))
        assert np.array_equal(hip.debug_dequant(1, 0, qt.size).view(np.uint32), want.view(np.uint32))
        # a sub-range that starts inside a block
        assert np.array_equal(hip.debug_dequant(1, 37, 100).view(np.uint32), want[37:137].view(np.uint32))


def test_layout_detection_rejects_near_misses(hip):
    qt = quant.quantize_q4_0(np.random.default_rng(0).standard_normal((4, 64)).astype(np.float32))
    s, z = qt.qparams()
    load_qtensor(hip, 1, qt)
    assert hip.map_layout(1) == 1
    z2 = z.copy(); z2[3] = np.nextafter(z2[3], np.float32(0))      # zp one ulp off -8*scale
    load_qtensor(hip, 1, qt, scale=s, zp=z2)
    assert hip.map_layout(1) == 0
    s2 = s.copy(); s2[5] = np.float32(s2[5] * (1 + 2.0 ** -20))    # scale not fp16-representable
    load_qtensor(hip, 1, qt, scale=s2, zp=(np.float32(-8) * s2))
    assert hip.map_layout(1) == 0


def test_gemv_config1_q4_0(hip):
    """BASELINE config 1: W 6912x1152 ~N(0,0.02) -> Q4_0 along K, x ~N(0,1), seed 0."""
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((6912, 1152)) * 0.02).astype(np.float32)
    x = rng.standard_normal(1152).astype(np.float32)
    qt = quant.quantize_q4_0(w)
    ys = {}
    for name, g in both(hip):
        note(f"gemv config1 on {name}")
        ys[name] = run_gemv(g, qt, x)
    assert rel_l2(ys["hip"], ys["oracle"]) < TOL
    assert rel_l2(ys["hip"], ys["oracle"]) < 2e-5      # what fp32 accumulation should give


@pytest.mark.parametrize("N,K", [(6144, 4096), (4096, 4096), (14336, 4096), (28672, 4096), (4096, 14336)])
def test_gemv_llama_shapes_q4_0(hip, N, K):
    rng = np.random.default_rng(N + K)
    w = (rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02))
    x = rng.standard_normal(K).astype(np.float32)
    qt = quant.quantize_q4_0(w)
    del w
    note(f"gemv q4_0 {N}x{K} hip")
    y = run_gemv(hip, qt, x)
    note(f"gemv q4_0 {N}x{K} oracle")
    want = run_gemv(oracle.init(), qt, x)
    assert rel_l2(y, want) < TOL


@pytest.mark.parametrize("N,K", [(8192, 4096), (1000, 1152)])
def test_gemv_q8_0(hip, N, K):
    rng = np.random.default_rng(N)
    qt = quant.quantize_q8_0((rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)))
    x = rng.standard_normal(K).astype(np.float32)
    note(f"gemv q8_0 {N}x{K}")
    assert rel_l2(run_gemv(hip, qt, x, wmap=2), run_gemv(oracle.init(), qt, x, wmap=2)) < TOL


@pytest.mark.parametrize("kind", ["q4", "q8"])
def test_gemv_affine_qparams_and_offsets(hip, kind):
    """Generic (non Q4_0/Q8_0) qparams at a non-zero, block-aligned base; and an unaligned base that
    must take the element-wise path."""
    rng = np.random.default_rng(21)
    N, K = 300, 256
    qt = (quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0)(
        rng.standard_normal((N, K)).astype(np.float32))
    s = rng.uniform(0.001, 0.1, N * K // 32).astype(np.float32)
    z = rng.uniform(-1, 1, N * K // 32).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    note(f"affine {kind} aligned offset")
    a = run_gemv(hip, qt, x, offset=64 * 32, scale=s, zp=z)
    b = run_gemv(oracle.init(), qt, x, offset=64 * 32, scale=s, zp=z)
    assert rel_l2(a, b) < TOL
    # unaligned row starts: K = 40 (not a multiple of 32) over the same bytes
    note(f"affine {kind} K=40 unaligned rows")
    o = oracle.init()
    outs = []
    for g in (hip, o):
        load_qtensor(g, 1, qt, scale=s, zp=z)
        f32map(g, 0, 512, x[:40])
        fn = g.map_matmul_t_xq4_dev if kind == "q4" else g.map_matmul_t_xq8_dev
        fn(0, 1, up(g, [0]), up(g, [6]), up(g, [64]), 1, 40, 50)
        outs.append(read(g, 0, 64, 50))
    assert rel_l2(outs[0], outs[1]) < TOL


def test_matmul_batched_rows_ops_and_non_transposed(hip):
    rng = np.random.default_rng(22)
    M, K, N, n_ops = 5, 64, 48, 3
    qt = quant.quantize_q4_0(rng.standard_normal((n_ops * N, K)).astype(np.float32))
    acts = rng.standard_normal(n_ops * M * K).astype(np.float32)
    res = []
    for name, g in both(hip):
        note(f"matmul M>1 n_ops>1 on {name}")
        load_qtensor(g, 1, qt)
        f32map(g, 0, n_ops * M * K + 2 * n_ops * M * N + 8, acts)
        la = up(g, [i * M * K for i in range(n_ops)])
        lb = up(g, [i * N * K for i in range(n_ops)])
        c0 = n_ops * M * K
        lc = up(g, [c0 + i * M * N for i in range(n_ops)])
        g.map_matmul_t_xq4_dev(0, 1, la, lb, lc, M, K, N, n_ops)
        t = read(g, 0, c0, n_ops * M * N)
        lc2 = up(g, [c0 + n_ops * M * N])
        g.map_matmul_xq4_dev(0, 1, up(g, [0]), up(g, [0]), lc2, M, K, N, 1)   # B read as [K, N]
        res.append((t, read(g, 0, c0 + n_ops * M * N, M * N)))
    assert rel_l2(res[0][0], res[1][0]) < TOL and rel_l2(res[0][1], res[1][1]) < TOL


# row lengths on either side of the kernel's choice of step (48 or 64 blocks): one short step (1152, 1536), several
# short steps with the last one part empty (3072 -> 2 x 48, 2080 -> 65 blocks in 2 x 48, 4000 -> 125 blocks in
# 3 x 48 where 2 x 64 would do: long steps), long steps with a ragged last one (6912), exact long steps (2048)
@pytest.mark.parametrize("N,K", [(1, 32), (17, 64), (33, 4096), (16, 15872), (1153, 1152), (130, 1536), (66, 3072),
                                 (259, 4000), (1152, 6912), (40, 2080), (77, 2048)])
def test_gemv_edge_shapes(hip, N, K):
    rng = np.random.default_rng(N * 7 + K)
    qt = quant.quantize_q4_0(rng.standard_normal((N, K)).astype(np.float32))
    x = rng.standard_normal(K).astype(np.float32)
    note(f"gemv edge {N}x{K}")
    assert rel_l2(run_gemv(hip, qt, x), run_gemv(oracle.init(), qt, x)) < TOL


def test_gemv_error_codes(hip):
    qt = quant.quantize_q4_0(np.ones((4, 32), np.float32))
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, 64, np.ones(32))
    a, b, c = up(hip, [0]), up(hip, [0]), up(hip, [32])
    assert hip._lib.map_matmul_t_xq4_dev(0, 9, a, b, c, 1, 32, 4, 1) == -3        # inactive map
    assert hip._lib.map_matmul_t_xq4_dev(0, 1, a, 60000, c, 1, 32, 4, 1) == -3    # unknown handle
    assert hip._lib.map_matmul_t_xq8_dev(0, 1, a, b, c, 1, 32, 4, 1) == -3        # Q4 map to the Q8 entry
    assert hip._lib.map_matmul_t_xq4_dev(0, 1, a, b, c, 1, 32, 5, 1) == -3        # weights run past the map
    assert hip._lib.map_matmul_t_xq4_dev(0, 1, a, b, c, 1, 32, 0, 1) == 0         # N == 0 is a no-op
    assert hip._lib.map_set_qparams(1, None, None, 1) == -3
    assert hip.scatter_q4_packed_contiguous(1, 1, np.zeros(2, np.uint8), 4) == (1 << 64) - 3   # odd start: -3
    h, _ = hip.upload_dev(np.zeros(4, np.uint32))
    assert hip.upload_dev(np.zeros(5, np.uint32), handle=h)[0] == 0               # size change -> 0


# ---- guard for the cross-lane moves of the Q4 GEMV -----------------------------------------------------
def _integer_weights(N, K, seed):
    """Q4_0 blocks with scale 1: the weights are the integers q - 8."""
    q = np.random.default_rng(seed).integers(0, 16, (N, K), dtype=np.uint8)
    codes = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8).reshape(-1)
    return quant.QTensor('q4_0', (N, K), np.ones(N * K // 32, np.float16), codes), q.astype(np.float64) - 8.0


@pytest.mark.parametrize("K,N", [(4096, 515), (1152, 1024), (6912, 1152)])
@pytest.mark.parametrize("pro", ["none", "rmsnorm", "norm2", "combine"])
def test_unit_scale_integer_weights_give_exact_sums(hip, pro, K, N):
    """Guard for the cross-lane moves of the matrix-instruction GEMV: the kernel hands blocks, scales, block maxima
    and integer sums from lane to lane (ds_bpermute, DPP), and every such move is kept an instruction of its own
    because, folded by the compiler into its consumer, the kernel once returned wrong sums without any other sign.
    With weights q - 8 at scale 1 and activations that are small integers (or integers over a power of two) every
    product and every partial sum is exact in int32 and in float32, whichever order the lanes add them in: the
    result must EQUAL the integer dot products, for every staging variant of the kernel -- plain, RMSNorm folded in,
    both norms of a layer boundary folded in, merge of the attention slices folded in (operands chosen so that the
    norms' factors are 1/2 and 1/4 and the softmax is uniform over 1024 rows)."""
    rng = np.random.default_rng(K + N)
    if pro == "combine":
        K = 1024                                       # 4 heads x 256 over one KV head: the merge in the GEMV's staging
    qt, W = _integer_weights(N, K, K * 3 + N)
    load_qtensor(hip, 1, qt)
    assert hip.map_layout(1) == 1
    note(f"gemv exact integer sums pro={pro} {N}x{K}")
    if pro == "combine":
        ctx, Hq, d = 1024, 4, 256
        V = rng.integers(-1, 2, (ctx, d)).astype(np.float32)
        Kc = rng.standard_normal((ctx, d)).astype(np.float32)
        q_pos, out_pos, y_pos = Hq * ctx, Hq * ctx + Hq * d, Hq * ctx + 2 * Hq * d
        kv = (y_pos + N + d - 1) // d * d
        f32map(hip, 0, kv + 2 * ctx * d, None)
        hip.kv_cache_fp16(0, kv, 2 * ctx * d)
        hip.scatter_contiguous(0, q_pos, np.zeros(Hq * d, np.float32))        # q = 0: every score is 0
        hip.scatter_contiguous(0, kv, Kc.reshape(-1)); hip.scatter_contiguous(0, kv + ctx * d, V.reshape(-1))
        s_rows, o_rows = up(hip, np.arange(Hq) * ctx), up(hip, out_pos + np.arange(Hq) * d)
        hip.batch_begin()
        hip.map_matmul_t_dev(0, up(hip, q_pos + np.arange(Hq) * d), up(hip, [kv] * Hq), s_rows, 1, d, ctx, Hq)
        hip.map_attn_softmax_value_dev(0, s_rows, up(hip, [kv + ctx * d] * Hq), o_rows, Hq, ctx, d, float(1 / 16), 0.0)
        hip.fusion_flush()
        hip.map_matmul_t_xq4_dev(0, 1, up(hip, [out_pos]), up(hip, [0]), up(hip, [y_pos]), 1, K, N)
        hip.batch_end()
        x = np.tile(V.astype(np.float64).sum(0) / ctx, Hq)
        assert np.array_equal(read(hip, 0, out_pos, K), x.astype(np.float32))
        assert hip.get_last_barrier_count() == 2                              # attention, GEMV with the merge
        y = read(hip, 0, y_pos, N)
    else:
        src = rng.choice([-2.0, 2.0], K).astype(np.float32)
        w1 = np.full(K, 2.0, np.float32)
        w2 = rng.choice([1.0, 2.0, 4.0], K).astype(np.float32)
        o = {"src": 0, "w1": K, "w2": 2 * K, "res": 3 * K, "x": 4 * K, "y": 5 * K}
        f32map(hip, 0, 5 * K + N + 8, np.concatenate([src, w1, w2, src]))      # residual = source
        h = lambda n: up(hip, [o[n]])
        hip.batch_begin()
        if pro == "none":
            x = rng.integers(-4, 5, K).astype(np.float32)
            hip.scatter_contiguous(0, o["x"], x)
        elif pro == "rmsnorm":                                                 # mean(src^2) = 4, eps 0: factor 1/2
            hip.map_rmsnorm_dev(0, h("src"), h("w2"), h("x"), 1, K, 0.0)
            x = src * 0.5 * w2
        else:                                   # t = src/2 * 2 + src = +-4; mean(t^2) = 16, eps 0: factor 1/4
            hip.map_rmsnorm_add_dev(0, h("src"), h("w1"), h("res"), h("res"), 1, K, 0.0)
            hip.map_rmsnorm_dev(0, h("res"), h("w2"), h("x"), 1, K, 0.0)
            x = 2.0 * src * 0.25 * w2
        hip.map_matmul_t_xq4_dev(0, 1, h("x"), up(hip, [0]), h("y"), 1, K, N)
        hip.batch_end()
        if K <= 4096:                           # (longer rows do not fit the staging's registers: the norms run apart)
            assert hip.get_last_barrier_count() == 1                          # the norms rode in the GEMV's staging
        assert np.array_equal(read(hip, 0, o["x"], K), x.astype(np.float32))
        if pro == "norm2":
            assert np.array_equal(read(hip, 0, o["res"], K), 2.0 * src)
        y = read(hip, 0, o["y"], N)
    want = W @ x.astype(np.float64)
    assert np.all(np.abs(want) < 2 ** 24 / 1024)
    assert np.array_equal(y, want.astype(np.float32))


@pytest.mark.parametrize("N,K", [(3, 4096), (5, 512), (1021, 4096), (4100, 4096), (7170, 2048), (16389, 4096), (28676, 512),
                                 (65537, 512), (100003, 512)])
def test_every_row_belongs_to_exactly_one_wave(hip, N, K):
    """The launcher deals the 4-row bundles out to the waves as floor(g * bundles / waves), which the kernel evaluates
    with a multiplication and a shift prepared on the host instead of a division: row counts on either side of
    multiples of 4, of the wave count and of the workgroup count, with and without a K split.  Integer weights at
    scale 1 and small integer activations make every row's result exact, so a row that no wave took (its place still
    holds the marker) or that was summed from another row's blocks fails equality."""
    qt, W = _integer_weights(N, K, N + K)
    x = np.random.default_rng(N).integers(-3, 4, K).astype(np.float32)
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, K + N + 8, np.concatenate([x, np.full(N + 8, -12345.0, np.float32)]))
    note(f"gemv row shares {N}x{K}")
    hip.batch_begin()
    hip.map_matmul_t_xq4_dev(0, 1, up(hip, [0]), up(hip, [0]), up(hip, [K]), 1, K, N)
    hip.batch_end()
    got = read(hip, 0, K, N + 8)
    assert np.array_equal(got[:N], (W @ x.astype(np.float64)).astype(np.float32))
    assert np.all(got[N:] == -12345.0)                    # and nothing past the last row
