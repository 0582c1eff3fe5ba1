"""Batched (M > 1) quantised matmul on the matrix cores against the oracle (needs an MI355X).

BASELINE config 5 shapes: M = 512 (prefill chunk) and M = 16 (batched decode) over Llama-3-8B-shape
Q4_0 matrices.  Bars, relative L2 per output row against the float64 product of the dequantised matrix:
Q4_0 weights 3e-5 (both operands enter the matrix cores as exact two-term fp16 sums, float32 accumulation --
a forward pass chains ~200 of these, so the single product has to sit far inside the path's 1e-3);
Q8_0 weights (the LM head of a lockstep batch, the last product of a pass) and the element-wise kernels 1e-3."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from adam_amd import quant
from gpu_util import note, up, f32map, put, read, rel_l2, load_qtensor

pytestmark = pytest.mark.gpu
TOL = 1e-3
TOL_Q4 = 3e-5


def run(g, qt, x, n_ops=1, scale=None, zp=None):
    """x: [n_ops, M, K]; the same weight matrix for every op.  Returns [n_ops, M, N]."""
    N, K = qt.shape
    n_ops, M, _ = x.shape
    load_qtensor(g, 1, qt, scale=scale, zp=zp)
    f32map(g, 0, n_ops * M * (K + N) + 8, x.reshape(-1))
    a = up(g, [i * M * K for i in range(n_ops)])
    c = up(g, [n_ops * M * K + i * M * N for i in range(n_ops)])
    g.batch_begin()
    g.map_matmul_t_xq4_dev(0, 1, a, up(g, [0] * n_ops), c, M, K, N, n_ops)
    g.batch_end()
    return read(g, 0, n_ops * M * K, n_ops * M * N).reshape(n_ops, M, N)


@pytest.mark.parametrize("M,N,K", [(16, 4096, 4096), (512, 4096, 4096), (16, 4096, 14336), (512, 1000, 1152),
                                   (2, 64, 128), (40, 130, 256), (100, 6144, 4096), (16, 28672, 4096), (9, 24600, 1152)])
def test_batched_q4_matmul_matches_oracle(hip, M, N, K):
    rng = np.random.default_rng(M + N + K)
    qt = quant.quantize_q4_0((rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)))
    x = rng.standard_normal((1, M, K), dtype=np.float32)
    note(f"gemm q4 M={M} N={N} K={K} hip")
    y = run(hip, qt, x)[0]
    note(f"gemm q4 M={M} N={N} K={K} reference product")
    want = (x[0].astype(np.float64) @ qt.dequant().astype(np.float64).T)
    for m in range(M):
        assert rel_l2(y[m], want[m]) < TOL_Q4, m
    if M * N * K <= 40 * 130 * 256:      # the oracle's own M > 1 path on the small case
        assert rel_l2(y, run(oracle.init(), qt, x)[0]) < TOL
    if M <= 16 and N >= 24576:           # wide matrices take the kernel whose waves share the activation tile
        import os
        os.environ["ADAMAH_GEMM_ROWS16"] = "0"
        try:
            y0 = run(hip, qt, x)[0]
        finally:
            del os.environ["ADAMAH_GEMM_ROWS16"]
        assert not np.array_equal(y, y0) and rel_l2(y, y0) < 1e-5      # another kernel, the same product


def test_batched_matmul_row_scaling_and_ops(hip):
    """Rows of very different magnitude (1e-6 ... 1e5), a zero row, and two ops in one call: every
    row keeps its own power-of-two scale, so each stays within tolerance."""
    rng = np.random.default_rng(7)
    N, K, M = 256, 512, 20
    qt = quant.quantize_q4_0((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    x = rng.standard_normal((2, M, K)).astype(np.float32)
    x[0, 3] *= 1e5; x[0, 4] *= 1e-6; x[1, 7] = 0.0; x[1, 9] *= 3e4
    note("gemm q4 row scaling")
    y = run(hip, qt, x, n_ops=2)
    w = qt.dequant().astype(np.float64)
    for op in range(2):
        want = x[op].astype(np.float64) @ w.T
        for m in range(M):
            if np.any(want[m]):
                assert rel_l2(y[op, m], want[m]) < TOL_Q4, (op, m)
            else:
                assert not np.any(y[op, m])


def test_batched_matmul_other_layouts_take_generic_path(hip):
    """Affine qparams (not Q4_0) and K not a multiple of 128 run the element-wise kernel; same answers."""
    rng = np.random.default_rng(9)
    for (N, K, affine) in ((96, 256, True), (50, 96, False)):
        qt = quant.quantize_q4_0(rng.standard_normal((N, K)).astype(np.float32))
        s = rng.uniform(0.001, 0.1, N * K // 32).astype(np.float32) if affine else None
        z = rng.uniform(-1, 1, N * K // 32).astype(np.float32) if affine else None
        x = rng.standard_normal((1, 5, K)).astype(np.float32)
        note(f"gemm generic N={N} K={K} affine={affine}")
        assert rel_l2(run(hip, qt, x, scale=s, zp=z), run(oracle.init(), qt, x, scale=s, zp=z)) < TOL


@pytest.mark.parametrize("M,N,K", [(16, 3000, 4096), (2, 64, 128), (23, 130, 256), (32, 1000, 1152)])
def test_batched_q8_matmul_matches_oracle(hip, M, N, K):
    """Up to 32 rows over Q8_0 blocks take the matrix cores as well (the LM head of a lockstep batch)."""
    rng = np.random.default_rng(M + N + K)
    qt = quant.quantize_q8_0((rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)))
    x = rng.standard_normal((M, K), dtype=np.float32)
    x[M - 1] *= 1e4
    outs = []
    for g in (hip, oracle.init()) if M * N * K <= 23 * 130 * 256 else (hip,):
        note(f"gemm q8 M={M} N={N} K={K}")
        load_qtensor(g, 2, qt)
        f32map(g, 0, M * (K + N) + 8, x.reshape(-1))
        g.batch_begin()
        g.map_matmul_t_xq8_dev(0, 2, up(g, [0]), up(g, [0]), up(g, [M * K]), M, K, N, 1)
        g.batch_end()
        outs.append(read(g, 0, M * K, M * N).reshape(M, N))
    want = x.astype(np.float64) @ qt.dequant().astype(np.float64).T
    for m in range(M):
        assert rel_l2(outs[0][m], want[m]) < TOL, m
    if len(outs) > 1:
        assert rel_l2(outs[0], outs[1]) < TOL


def test_consecutive_matmuls_over_the_same_rows_share_conversion_and_launch(hip):
    """Q, K and V projections of a chunk read the same rows: the second and third matmul skip the fp16
    conversion launch.  A write to the rows in between (kernel or upload) brings it back, and so does a
    result that lands on them."""
    rng = np.random.default_rng(11)
    M, K, N = 16, 256, 64
    qt = quant.quantize_q4_0(rng.standard_normal((3 * N, K), dtype=np.float32) * np.float32(0.05))
    x = rng.standard_normal((M, K), dtype=np.float32)
    w = qt.dequant().astype(np.float64)
    note("gemm conversion reuse")
    load_qtensor(hip, 1, qt)
    f32map(hip, 0, M * K + 3 * M * N + 64, x.reshape(-1))
    a, cs = up(hip, [0]), [up(hip, [M * K + i * M * N]) for i in range(3)]
    bs = [up(hip, [i * N * K]) for i in range(3)]
    for order, launches in (((2, 1, 0), 4), ((0, 1, 2), 2)):
        # matrices not in storage order: one conversion, three matmuls; in storage order (W_k right after
        # W_q, W_v right after W_k): one conversion and ONE matmul over the stacked rows
        put(hip, 0, M * K, np.zeros(3 * M * N, np.float32))
        hip.batch_begin()
        for i in order:
            hip.map_matmul_t_xq4_dev(0, 1, a, bs[i], cs[i], M, K, N, 1)
        hip.batch_end()
        assert hip.get_last_barrier_count() == launches
        y = read(hip, 0, M * K, 3 * M * N).reshape(3, M, N)
        for i in range(3):
            assert rel_l2(y[i], x.astype(np.float64) @ w[i * N:(i + 1) * N].T) < TOL
        if launches == 4:
            apart = y.copy()
        else:
            assert np.array_equal(y.view(np.uint32), apart.view(np.uint32))   # merged == one by one, bit for bit
    # rows rewritten between two matmuls: converted again, and the new values are the ones used
    x2 = rng.standard_normal((M, K), dtype=np.float32)
    hip.batch_begin()
    hip.map_matmul_t_xq4_dev(0, 1, a, bs[0], cs[0], M, K, N, 1)
    hip.scatter_contiguous(0, 0, x2.reshape(-1))
    hip.map_matmul_t_xq4_dev(0, 1, a, bs[1], cs[1], M, K, N, 1)
    hip.batch_end()
    y = read(hip, 0, M * K, 2 * M * N).reshape(2, M, N)
    assert rel_l2(y[0], x.astype(np.float64) @ w[:N].T) < TOL
    assert rel_l2(y[1], x2.astype(np.float64) @ w[N:2 * N].T) < TOL
    # a result stored over the rows themselves (M * N == M * K here): nothing is reused afterwards
    qs = quant.quantize_q4_0(rng.standard_normal((K, K), dtype=np.float32) * np.float32(0.05))
    load_qtensor(hip, 3, qs)
    hip.batch_begin()
    hip.map_matmul_t_xq4_dev(0, 3, a, up(hip, [0]), a, M, K, K, 1)
    hip.map_matmul_t_xq4_dev(0, 1, a, bs[2], cs[2], M, K, N, 1)
    hip.batch_end()
    assert hip.get_last_barrier_count() == 4
    x3 = (x2.astype(np.float64) @ qs.dequant().astype(np.float64).T)
    assert rel_l2(read(hip, 0, M * K + 2 * M * N, M * N).reshape(M, N), x3 @ w[2 * N:].T) < 3 * TOL


@pytest.mark.parametrize("dim,rows,add", [(4096, 16, False), (1152, 5, True), (8192, 3, False), (256, 40, True)])
def test_rmsnorm_rows_feed_the_matmul_without_a_conversion_launch(hip, dim, rows, add):
    """RMSNorm over the rows of a matrix followed by a batched matmul over those rows: the norm kernel also
    writes the matmul's fp16 operand form, so the pair costs two launches, and every output word equals
    the three-launch form's (ADAMAH_RMSNORM_EMIT=0).  Dims that are not a multiple of 128 take the
    element-wise matmul and still match the oracle."""
    import os
    rng = np.random.default_rng(dim + rows)
    N = 96
    qt = quant.quantize_q4_0(rng.standard_normal((N, dim), dtype=np.float32) * np.float32(0.05))
    x = rng.standard_normal((rows, dim), dtype=np.float32) * np.float32(3.0)
    res = rng.standard_normal((rows, dim), dtype=np.float32)
    wn = rng.uniform(0.5, 1.5, dim).astype(np.float32)

    def go(g):
        load_qtensor(g, 1, qt)
        w0 = 3 * rows * dim + rows * N
        f32map(g, 0, w0 + dim + 8, np.concatenate([x.reshape(-1), res.reshape(-1)]))
        put(g, 0, w0, wn)
        src, rs = up(g, np.arange(rows) * dim), up(g, rows * dim + np.arange(rows) * dim)
        dst, wl = up(g, 2 * rows * dim + np.arange(rows) * dim), up(g, [w0] * rows)
        a, b, c = up(g, [2 * rows * dim]), up(g, [0]), up(g, [3 * rows * dim])   # (an upload in between would void the note)
        g.batch_begin()
        if add:
            g.map_rmsnorm_add_dev(0, src, wl, rs, dst, rows, dim, 1e-5)
        else:
            g.map_rmsnorm_dev(0, src, wl, dst, rows, dim, 1e-5)
        g.map_matmul_t_xq4_dev(0, 1, a, b, c, rows, dim, N, 1)
        g.batch_end()
        n = g.get_last_barrier_count() if g is hip else None
        return read(g, 0, 2 * rows * dim, rows * dim + rows * N), n

    note(f"rmsnorm rows + matmul dim={dim} rows={rows} add={add}")
    fused, n_fused = go(hip)
    os.environ["ADAMAH_RMSNORM_EMIT"] = "0"
    try:
        apart, n_apart = go(hip)
    finally:
        del os.environ["ADAMAH_RMSNORM_EMIT"]
    assert np.array_equal(fused.view(np.uint32), apart.view(np.uint32))
    if dim % 128 == 0:
        assert (n_fused, n_apart) == (2, 3)
    want, _ = go(oracle.init())
    assert rel_l2(fused[:rows * dim], want[:rows * dim]) < 1e-5
    assert rel_l2(fused[rows * dim:], want[rows * dim:]) < TOL


@pytest.mark.parametrize("kind,M,K,Ns", [("q4", 16, 4096, (4096, 1024, 1024)), ("q4", 5, 256, (40, 24)), ("q8", 16, 512, (100, 60, 33, 7)),
                                         ("q4", 32, 1152, (1024, 256, 256)), ("q4", 100, 256, (200, 72, 72)),
                                         ("q4", 512, 4096, (4096, 1024, 1024))])
def test_stacked_matmuls_place_every_result_where_its_op_asked(hip, monkeypatch, kind, M, K, Ns):
    """Matmuls over the same rows with weight matrices back to back but results at unrelated places and of
    different widths (not multiples of 16 either): one launch, each [M, N_i] result at its own base, equal
    bit for bit to the ops run one by one (ADAMAH_GEMM_MERGE=0).  (With the split over K off: how many shares of K
    a launch is cut into goes by its width, so the stacked launch and the single ones add in different orders;
    test_narrow_matrix_under_many_rows_split_over_k covers that path.)"""
    import os
    monkeypatch.setenv("ADAMAH_GEMM_SPLITK", "0")
    rng = np.random.default_rng(sum(Ns) + M)
    Nt = sum(Ns)
    w = rng.standard_normal((Nt, K), dtype=np.float32) * np.float32(0.05)
    qt = (quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0)(w)
    x = rng.standard_normal((M, K), dtype=np.float32)
    fn_name = "map_matmul_t_xq4_dev" if kind == "q4" else "map_matmul_t_xq8_dev"
    mid = 1 if kind == "q4" else 2
    gap = 24
    c0, offs = [], M * K + 8
    for n_i in reversed(Ns):                       # results in reverse order, with gaps between them
        c0.insert(0, offs); offs += M * n_i + gap
    total = offs

    def go(g):
        load_qtensor(g, mid, qt)
        f32map(g, 0, total, x.reshape(-1))
        a = up(g, [0])
        bs, cs, b = [], [], 0
        for n_i, c in zip(Ns, c0):
            bs.append(up(g, [b])); cs.append(up(g, [c])); b += n_i * K
        g.batch_begin()
        for n_i, bh, ch in zip(Ns, bs, cs):
            getattr(g, fn_name)(0, mid, a, bh, ch, M, K, n_i, 1)
        g.batch_end()
        return read(g, 0, 0, total), (g.get_last_barrier_count() if g is hip else None)

    note(f"stacked matmuls {kind} M={M} K={K} Ns={Ns}")
    merged, n_merged = go(hip)
    os.environ["ADAMAH_GEMM_MERGE"] = "0"
    try:
        apart, n_apart = go(hip)
    finally:
        del os.environ["ADAMAH_GEMM_MERGE"]
    assert (n_merged, n_apart) == (2, 1 + len(Ns))
    assert np.array_equal(merged.view(np.uint32), apart.view(np.uint32))
    wd = qt.dequant().astype(np.float64)
    r0 = 0
    for n_i, c in zip(Ns, c0):
        want = x.astype(np.float64) @ wd[r0:r0 + n_i].T
        assert rel_l2(merged[c:c + M * n_i].reshape(M, n_i), want) < TOL
        r0 += n_i
    assert not merged[M * K:M * K + 8].any()       # nothing outside the results was written


@pytest.mark.parametrize("M,K,N,in_place", [(16, 4096, 4096, True), (7, 256, 50, False), (32, 1152, 72, True),
                                            (512, 4096, 4096, True), (400, 4096, 4100, False)])
def test_residual_add_stored_by_the_matmul(hip, M, K, N, in_place):
    """hidden += X W^T issued as matmul then add: the matmul's store also writes residual + result (two launches
    with the conversion instead of three); the projection itself still lands in its own rows.  All words equal
    the unfused sequence's (ADAMAH_GEMM_EPI=0).  With many rows the add rides in the launch that adds the shares
    of a matmul run over shares of K (three launches instead of four)."""
    import os
    rng = np.random.default_rng(M + N)
    qt = quant.quantize_q4_0(rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05))
    x = rng.standard_normal((M, K), dtype=np.float32)
    hid = rng.standard_normal((M, N), dtype=np.float32)
    y0, h0 = M * K, M * K + M * N
    d0 = h0 if in_place else h0 + M * N
    total = h0 + 2 * M * N

    def go(g):
        load_qtensor(g, 1, qt)
        f32map(g, 0, total, np.concatenate([x.reshape(-1), np.zeros(M * N, np.float32), hid.reshape(-1)]))
        a, b, c = up(g, [0]), up(g, [0]), up(g, [y0])
        hy, hh, hd = up(g, y0 + np.arange(M * N)), up(g, h0 + np.arange(M * N)), up(g, d0 + np.arange(M * N))
        g.batch_begin()
        g.map_matmul_t_xq4_dev(0, 1, a, b, c, M, K, N, 1)
        g.map_op2_dev(0, A.OP_ADD, hh, hy, hd, M * N)
        g.batch_end()
        return read(g, 0, 0, total), (g.get_last_barrier_count() if g is hip else None)

    note(f"matmul + residual add M={M} K={K} N={N} in_place={in_place}")
    fused, n_fused = go(hip)
    os.environ["ADAMAH_GEMM_EPI"] = "0"
    try:
        apart, n_apart = go(hip)
    finally:
        del os.environ["ADAMAH_GEMM_EPI"]
    assert (n_fused, n_apart) == ((2, 3) if M <= 32 else (3, 4))
    assert np.array_equal(fused.view(np.uint32), apart.view(np.uint32))
    if M <= 32:
        want, _ = go(oracle.init())
        assert rel_l2(fused[y0:], want[y0:]) < TOL
    else:                                  # (the oracle's op surface takes minutes over this many rows)
        y = x.astype(np.float64) @ qt.dequant().astype(np.float64).T
        assert rel_l2(fused[y0:h0].reshape(M, N), y) < TOL
        assert rel_l2(fused[d0:d0 + M * N].reshape(M, N), y + hid) < TOL


@pytest.mark.parametrize("op,M,K,N,in_place", [("swiglu", 16, 14336, 96, False), ("geglu", 5, 6912, 64, False), ("swiglu", 40, 256, 50, False),
                                               ("geglu", 16, 1024, 96, True)])
def test_gated_activation_feeds_the_matmul_without_a_conversion_launch(hip, op, M, K, N, in_place):
    """act = GLU(gate, up) over M rows followed by the batched matmul over act: the activation's launch also writes
    the matmul's fp16 operand form (two launches instead of three), and every word equals the separate ops'
    (ADAMAH_GLU_EMIT=0).  An activation stored over its own gate rows is left as it was."""
    import os
    rng = np.random.default_rng(M + K)
    qt = quant.quantize_q4_0(rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.05))
    gate = rng.standard_normal((M, K), dtype=np.float32) * np.float32(2.0)
    upv = rng.standard_normal((M, K), dtype=np.float32)
    a0 = 0 if in_place else 2 * M * K
    y0 = 3 * M * K
    code = A.OP_SWIGLU if op == "swiglu" else A.OP_GEGLU

    def go(g):
        load_qtensor(g, 1, qt)
        f32map(g, 0, y0 + M * N + 8, np.concatenate([gate.reshape(-1), upv.reshape(-1)]))
        hg, hu, ha = up(g, np.arange(M * K)), up(g, M * K + np.arange(M * K)), up(g, a0 + np.arange(M * K))
        a, b, c = up(g, [a0]), up(g, [0]), up(g, [y0])
        g.batch_begin()
        g.map_op2_dev(0, code, hg, hu, ha, M * K)
        g.map_matmul_t_xq4_dev(0, 1, a, b, c, M, K, N, 1)
        g.batch_end()
        return read(g, 0, 0, y0 + M * N), (g.get_last_barrier_count() if g is hip else None)

    note(f"{op} + matmul M={M} K={K} N={N} in_place={in_place}")
    fused, n_fused = go(hip)
    os.environ["ADAMAH_GLU_EMIT"] = "0"
    try:
        apart, n_apart = go(hip)
    finally:
        del os.environ["ADAMAH_GLU_EMIT"]
    assert np.array_equal(fused.view(np.uint32), apart.view(np.uint32))
    if K % 128 == 0:
        assert (n_fused, n_apart) == ((3, 3) if in_place else (2, 3))
    want, _ = go(oracle.init())
    assert rel_l2(fused[a0:a0 + M * K], want[a0:a0 + M * K]) < 1e-5
    assert rel_l2(fused[y0:], want[y0:]) < TOL


@pytest.mark.parametrize("kind,op,M,K,F", [("q4", "swiglu", 16, 4096, 14336), ("q4", "geglu", 5, 256, 48), ("q8", "swiglu", 32, 512, 80),
                                           ("q4", "swiglu", 16, 256, 40), ("q4", "geglu", 40, 256, 48)])
def test_gated_activation_stored_by_the_stacked_gate_up_matmul(hip, kind, op, M, K, F):
    """gate = X Wg^T, up = X Wu^T (matrices back to back), act = GLU(gate, up), then a matmul over act, as a
    batched decode step issues them: for M <= 32 and F a multiple of 16 the stacked launch stores act as well
    (conversion + stacked matmul + conversion + matmul = 4 launches), every word equal to the separate ops'
    (ADAMAH_GEMM_EPI=0, ADAMAH_GLU_EMIT=0: 5); otherwise the activation's own launch leaves the fp16 form (4)."""
    import os
    rng = np.random.default_rng(M + K + F)
    qfn = quant.quantize_q4_0 if kind == "q4" else quant.quantize_q8_0
    qt = qfn(rng.standard_normal((2 * F, K), dtype=np.float32) * np.float32(0.05))
    N2 = 24
    fn_name = "map_matmul_t_xq4_dev" if kind == "q4" else "map_matmul_t_xq8_dev"
    mid = 1 if kind == "q4" else 2
    x = rng.standard_normal((M, K), dtype=np.float32)
    g0, u0, a0 = M * K, M * K + M * F, M * K + 2 * M * F
    y0 = a0 + M * F
    total = y0 + M * N2 + 8
    wd = rng.standard_normal((N2, F), dtype=np.float32) * np.float32(0.05)
    down_ok = F % 128 == 0

    def go(g):
        load_qtensor(g, mid, qt)
        if down_ok:
            load_qtensor(g, 3, quant.quantize_q4_0(wd))
        f32map(g, 0, total, x.reshape(-1))
        a, b0, b1 = up(g, [0]), up(g, [0]), up(g, [F * K])
        cg, cu, ca, cy = up(g, [g0]), up(g, [u0]), up(g, [a0]), up(g, [y0])
        hg, hu, ha = up(g, g0 + np.arange(M * F)), up(g, u0 + np.arange(M * F)), up(g, a0 + np.arange(M * F))
        g.batch_begin()
        getattr(g, fn_name)(0, mid, a, b0, cg, M, K, F, 1)
        getattr(g, fn_name)(0, mid, a, b1, cu, M, K, F, 1)
        g.map_op2_dev(0, A.OP_SWIGLU if op == "swiglu" else A.OP_GEGLU, hg, hu, ha, M * F)
        if down_ok:
            g.map_matmul_t_xq4_dev(0, 3, ca, up(g, [0]), cy, M, F, N2, 1)
        g.batch_end()
        return read(g, 0, 0, total), (g.get_last_barrier_count() if g is hip else None)

    note(f"gate/up + {op} {kind} M={M} K={K} F={F}")
    fused, n_fused = go(hip)
    os.environ["ADAMAH_GEMM_EPI"] = "0"
    os.environ["ADAMAH_GLU_EMIT"] = "0"
    try:
        apart, n_apart = go(hip)
    finally:
        del os.environ["ADAMAH_GEMM_EPI"], os.environ["ADAMAH_GLU_EMIT"]
    assert np.array_equal(fused.view(np.uint32), apart.view(np.uint32))
    if down_ok:
        assert (n_fused, n_apart) == (4, 5)
    else:
        assert (n_fused, n_apart) == ((2, 3) if M <= 32 and F % 16 == 0 else (3, 3))
    want, _ = go(oracle.init())
    assert rel_l2(fused[g0:a0], want[g0:a0]) < TOL
    assert rel_l2(fused[a0:y0], want[a0:y0]) < TOL
    if down_ok:
        assert rel_l2(fused[y0:y0 + M * N2], want[y0:y0 + M * N2]) < TOL
    assert not fused[y0 + M * N2:].any()


@pytest.mark.parametrize("M,N,K,Ns", [(512, 4096, 4096, None), (487, 4096, 14336, None), (512, 6144, 4096, (4096, 1024, 1024)),
                                      (400, 4100, 4096, None)])
def test_narrow_matrix_under_many_rows_split_over_k(hip, monkeypatch, M, N, K, Ns):
    """Matrices too narrow for the widest tile to fill the chip are run as shares of K whose raw sums a second launch
    adds: same product as the unsplit launch (and the reference's) for whole and ragged tiles, a last share shorter
    than the others, and stacked matrices with results in three places."""
    rng = np.random.default_rng(M + N + K)
    qt = quant.quantize_q4_0((rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)))
    x = rng.standard_normal((M, K), dtype=np.float32)
    want = x.astype(np.float64) @ qt.dequant().astype(np.float64).T

    def once():
        load_qtensor(hip, 1, qt)
        f32map(hip, 0, M * K + M * N + 64, x.reshape(-1))
        hip.batch_begin()
        if Ns is None:
            hip.map_matmul_t_xq4_dev(0, 1, up(hip, [0]), up(hip, [0]), up(hip, [M * K]), M, K, N, 1)
        else:                            # storage order: one launch over the stacked rows
            r = 0
            for n in Ns:
                hip.map_matmul_t_xq4_dev(0, 1, up(hip, [0]), up(hip, [r * K]), up(hip, [M * K + M * r]), M, K, n, 1)
                r += n
        hip.batch_end()
        return read(hip, 0, M * K, M * N), hip.get_last_barrier_count()

    note(f"gemm q4 split-K M={M} N={N} K={K}")
    y1, l1 = once()
    monkeypatch.setenv("ADAMAH_GEMM_SPLITK", "0")
    y0, l0 = once()
    if Ns is None:
        got1, got0 = y1.reshape(M, N), y0.reshape(M, N)
    else:
        got1, got0 = np.empty((M, N), np.float32), np.empty((M, N), np.float32)
        r = 0
        for n in Ns:
            got1[:, r:r + n] = y1[M * r:M * (r + n)].reshape(M, n)
            got0[:, r:r + n] = y0[M * r:M * (r + n)].reshape(M, n)
            r += n
    for m in range(0, M, 7):
        assert rel_l2(got1[m], want[m]) < TOL_Q4 and rel_l2(got0[m], want[m]) < TOL_Q4, m
    assert rel_l2(got1, got0) < 1e-5
    assert l1 == l0 + 1, (l1, l0)        # the launch that adds the shares
