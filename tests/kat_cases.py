"""Known-answer cases of the reference, runnable on any implementation of the op surface.

Every case transcribes the inputs and literal expected outputs of one scenario in the
reference's tests/test_decode_primitives.py (line ranges cited per case) or
tests/test_q4_roundtrip.py.  The reference drives them through its UUCIS convenience
wrapper; here the same maps, handles and ops are issued directly on the binding's methods.
`g` is the backend object (HIP binding or NumPy oracle), `A` a namespace with OP_* / DTYPE_*.
"""
import numpy as np


def _f32map(g, A, map_id, n):
    g.set_dtype(A.DTYPE_F32)
    g.map_create(map_id, 1, n)


def _h(g, arr):
    h, _ = g.upload_dev(np.asarray(arr, dtype=np.uint32))
    assert h != 0
    return h


def _read(g, map_id, locs):
    return g.gather(map_id, np.asarray(locs, dtype=np.uint32)).view(np.float32)


def kat_argmax(g, A):
    """test_decode_primitives.py:17-29: tie -> lower index."""
    _f32map(g, A, 8, 12)
    logits = np.array([-3.0, 5.5, 2.0, 5.5, 4.0, -1.0], np.float32)
    g.scatter(8, np.arange(6, dtype=np.uint32), logits)
    g.map_argmax_dev(8, _h(g, np.arange(6)), _h(g, [10]), 6)
    assert int(_read(g, 8, [10])[0]) == 1


def kat_softmax_abs(g, A):
    """:98-119."""
    _f32map(g, A, 3, 16)
    vals = np.zeros(16, np.float32)
    vals[0:3] = [1.0, 2.0, 3.0]; vals[8:11] = [0.0, 0.0, 1.0]
    g.scatter(3, np.arange(16, dtype=np.uint32), vals)
    row_h = _h(g, [0, 8])
    g.batch_begin(); g.map_softmax_abs_dev(3, row_h, row_h, 3, 2); g.batch_end()
    out = _read(g, 3, [0, 1, 2, 8, 9, 10])
    exp = np.array([0.09003057, 0.24472848, 0.66524094, 0.21194157, 0.21194157, 0.57611686], np.float32)
    assert np.allclose(out, exp, atol=1e-5), out


def kat_attn_softmax_abs(g, A):
    """:122-149: scale 0.5, cap 1.0; expected = softmax(tanh(0.5 s))."""
    _f32map(g, A, 6, 16)
    vals = np.zeros(16, np.float32)
    vals[0:3] = [1.0, 2.0, 3.0]; vals[8:11] = [0.0, 0.0, 1.0]
    g.scatter(6, np.arange(16, dtype=np.uint32), vals)
    row_h = _h(g, [0, 8])
    g.batch_begin(); g.map_attn_softmax_abs_dev(6, row_h, row_h, 3, 2, 0.5, 1.0); g.batch_end()
    out = _read(g, 6, [0, 1, 2, 8, 9, 10])

    def ref(row):
        s = np.tanh(row * 0.5)
        e = np.exp(s - s.max())
        return e / e.sum()
    exp = np.concatenate([ref(np.array([1.0, 2.0, 3.0])), ref(np.array([0.0, 0.0, 1.0]))])
    # literal values of that formula, independent of any code under test
    lit = np.array([0.25597878, 0.34535455, 0.39866667, 0.27875098, 0.27875098, 0.44249803])
    assert np.allclose(exp, lit, atol=1e-6)
    assert np.allclose(out, lit, atol=1e-5), out


def kat_q8_gather_scatter(g, A):
    """:152-171: raw [124,132,128,130], scale .5, zp -64 -> [-2, 2, 0, 1]."""
    g.map_create_typed(13, A.DTYPE_Q8, 1, 4, 4)
    g.set_qparams(13, np.array([0.5], np.float32), np.array([-64.0], np.float32))
    g.scatter(13, np.arange(4, dtype=np.uint32), np.array([124, 132, 128, 130], np.uint8))
    _f32map(g, A, 14, 4)
    src = _h(g, np.arange(4)); dst = _h(g, np.arange(4))
    gh, ticket, n, _ = g.map_gather_dev(13, src, 4)
    assert gh != 0 and n == 4
    g.map_scatter_dev(14, dst, 4, gh)
    assert np.allclose(_read(g, 14, np.arange(4)), [-2.0, 2.0, 0.0, 1.0], atol=1e-6)


def kat_row_gather_xq8(g, A):
    """:174-189: row 1 of a 2x4 Q8 matrix -> [6, -4, 0, 2]."""
    g.map_create_typed(4, A.DTYPE_Q8, 1, 8, 4)
    g.set_qparams(4, np.array([0.5, 0.5], np.float32), np.array([-64.0, -64.0], np.float32))
    g.scatter(4, np.arange(8, dtype=np.uint32), np.array([124, 132, 128, 130, 140, 120, 128, 132], np.uint8))
    _f32map(g, A, 5, 4)
    g.batch_begin(); g.map_row_gather_xq8_dev(5, 4, 0, 0, 1, 4, 1.0); g.batch_end()
    assert np.allclose(_read(g, 5, np.arange(4)), [6.0, -4.0, 0.0, 2.0], atol=1e-6)


def kat_matvec_t_xq8(g, A):
    """:192-214: x=[1,2,-1,.5] times two Q8 rows -> [1.5, -7.0]."""
    g.map_create_typed(7, A.DTYPE_Q8, 1, 8, 4)
    g.set_qparams(7, np.array([0.5, 0.5], np.float32), np.array([-64.0, -64.0], np.float32))
    g.scatter(7, np.arange(8, dtype=np.uint32), np.array([128, 130, 132, 134, 120, 124, 128, 132], np.uint8))
    _f32map(g, A, 8, 8)
    g.scatter(8, np.arange(4, dtype=np.uint32), np.array([1.0, 2.0, -1.0, 0.5], np.float32))
    vec_h = _h(g, np.arange(4)); out_h = _h(g, [4, 5]); base_h = _h(g, [0])
    g.batch_begin(); g.map_matmul_t_xq8_dev(8, 7, vec_h, base_h, out_h, 1, 4, 2); g.batch_end()
    assert np.allclose(_read(g, 8, [4, 5]), [1.5, -7.0], atol=1e-5)


def kat_matvec_t_xq4(g, A):
    """:355-381: identity rows quantised on the device with scale 1/15, zp 0 -> all ~1 (atol .05)."""
    K, N = 8, 4
    g.map_create_typed(14, A.DTYPE_Q4, 1, K * N, 32)
    g.set_qparams(14, np.array([1.0 / 15.0], np.float32), np.array([0.0], np.float32))
    g.scatter(14, np.arange(K * N, dtype=np.uint32), np.eye(N, K, dtype=np.float32).flatten())
    _f32map(g, A, 15, K + N + 4)
    g.scatter(15, np.arange(K, dtype=np.uint32), np.ones(K, np.float32))
    a_h, b_h, c_h = _h(g, [0]), _h(g, [0]), _h(g, [K])
    g.batch_begin(); g.map_matmul_t_xq4_dev(15, 14, a_h, b_h, c_h, 1, K, N); g.batch_end()
    assert np.allclose(_read(g, 15, np.arange(K, K + N)), np.ones(N), atol=0.05)


def kat_q4_matmul_identity(g, A):
    """test_q4_roundtrip.py:97-141: C = A . B^T with Q4 B = identity rows (min/max qparams per
    group of 32), RMSE < 0.01 against the float result."""
    M, K, N = 4, 32, 8
    rng = np.random.default_rng(0)
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = np.eye(N, K, dtype=np.float32)
    g.map_create_typed(14, A.DTYPE_Q4, 1, K * N, 32)
    flat = b.flatten()
    sc = np.empty(N, np.float32); zp = np.empty(N, np.float32)
    for gi in range(N):
        ch = flat[gi * 32:(gi + 1) * 32]
        sc[gi] = (ch.max() - ch.min()) / 15.0 if ch.max() > ch.min() else 1.0
        zp[gi] = ch.min()
    g.set_qparams(14, sc, zp)
    g.scatter(14, np.arange(K * N, dtype=np.uint32), flat)
    _f32map(g, A, 15, M * K + M * N)
    g.scatter(15, np.arange(M * K, dtype=np.uint32), a.flatten())
    a_h, b_h, c_h = _h(g, [0]), _h(g, [0]), _h(g, [M * K])
    g.batch_begin(); g.map_matmul_t_xq4_dev(15, 14, a_h, b_h, c_h, M, K, N); g.batch_end()
    out = _read(g, 15, np.arange(M * K, M * K + M * N)).reshape(M, N)
    assert float(np.sqrt(np.mean((out - a @ b.T) ** 2))) < 0.01


def kat_batch_gather_scatter(g, A):
    """:384-398."""
    _f32map(g, A, 0, 8); _f32map(g, A, 1, 8)
    src = _h(g, np.arange(4)); dst = _h(g, np.arange(4))
    g.scatter(0, np.arange(4, dtype=np.uint32), np.array([9.0, -2.0, 7.0, 1.5], np.float32))
    g.batch_begin()
    gh, _, _, _ = g.map_gather_dev(0, src, 4)
    g.map_scatter_dev(1, dst, 4, gh)
    g.batch_end()
    assert np.allclose(_read(g, 1, np.arange(4)), [9.0, -2.0, 7.0, 1.5], atol=1e-6)


def kat_row_copy_offset(g, A):
    """:401-420: spec [0,3,1,5], offset 2, row 4 -> rows land at 20..23 and 28..31."""
    _f32map(g, A, 2, 40)
    data = np.zeros(40, np.float32)
    data[:8] = [1.0, 2.0, 3.0, 4.0, 10.0, 20.0, 30.0, 40.0]
    g.scatter(2, np.arange(40, dtype=np.uint32), data)
    spec_h = _h(g, [0, 3, 1, 5]); base_h = _h(g, [0])
    g.batch_begin(); g.map_row_copy_offset_dev(2, spec_h, base_h, 2, 2, 4); g.batch_end()
    vals = _read(g, 2, list(range(20, 24)) + list(range(28, 32)))
    assert np.allclose(vals, [1.0, 2.0, 3.0, 4.0, 10.0, 20.0, 30.0, 40.0], atol=1e-6)
    untouched = _read(g, 2, list(range(8, 20)) + list(range(24, 28)) + list(range(32, 40)))
    assert np.all(untouched == 0.0)


def kat_fusion_row_copy_then_matmul(g, A):
    """:423-446: row copy then matmul_t inside one batch with fusion on -> [10, 100]."""
    g.fusion_enable(True)
    _f32map(g, A, 11, 32)
    data = np.zeros(32, np.float32)
    data[:8] = [1.0, 2.0, 3.0, 4.0, 10.0, 20.0, 30.0, 40.0]
    data[8:12] = 1.0
    g.scatter(11, np.arange(32, dtype=np.uint32), data)
    spec_h = _h(g, [0, 0, 1, 1]); sb_h = _h(g, [0])
    a_h, b_h, c_h = _h(g, [8]), _h(g, [20]), _h(g, [12])
    g.batch_begin()
    g.map_row_copy_offset_dev(11, spec_h, sb_h, 5, 2, 4)
    g.map_matmul_t_dev(11, a_h, b_h, c_h, 1, 4, 2)
    g.batch_end()
    assert np.allclose(_read(g, 11, [12, 13]), [10.0, 100.0], atol=1e-6)
    g.fusion_enable(False)


def kat_scalar_state(g, A):
    """:449-478 through op2 codes: copy (a+0), increment, EQ, GE, OR."""
    _f32map(g, A, 9, 9)
    state = np.array([3.0, 0.0, 1.0, 4.0, 0.0, 0.0, 0.0, 0.0, 0.0], np.float32)
    g.scatter(9, np.arange(9, dtype=np.uint32), state)
    L = {i: _h(g, [i]) for i in range(9)}
    g.map_op2_dev(9, A.OP_ADD, L[0], L[8], L[1], 1)      # next = current + 0
    g.map_op2_dev(9, A.OP_ADD, L[1], L[2], L[1], 1)      # next += one
    g.map_op2_dev(9, A.OP_EQ, L[1], L[3], L[7], 1)
    g.map_op2_dev(9, A.OP_GE, L[1], L[3], L[4], 1)
    g.map_op2_dev(9, A.OP_OR, L[4], L[5], L[6], 1)
    out = _read(g, 9, np.arange(8))
    assert int(out[1]) == 4 and int(out[4]) == 1 and int(out[6]) == 1 and int(out[7]) == 1


def kat_fusion_batch_order(g, A):
    """:481-504: ADD then argmax in one batch -> 2; NEG in the next -> [-1,-2,-3]."""
    g.fusion_enable(True)
    _f32map(g, A, 12, 12)
    src, dbl, win, neg = _h(g, [0, 1, 2]), _h(g, [4, 5, 6]), _h(g, [8]), _h(g, [9, 10, 11])
    g.scatter(12, np.arange(12, dtype=np.uint32), np.array([1.0, 2.0, 3.0] + [0.0] * 9, np.float32))
    g.batch_begin()
    g.map_op2_dev(12, A.OP_ADD, src, src, dbl, 3)
    g.map_argmax_dev(12, dbl, win, 3)
    g.batch_end()
    assert int(_read(g, 12, [8])[0]) == 2
    g.batch_begin(); g.map_op1_dev(12, A.OP_NEG, src, neg, 3); g.batch_end()
    assert np.allclose(_read(g, 12, [9, 10, 11]), [-1.0, -2.0, -3.0], atol=1e-6)
    g.fusion_enable(False)


def kat_decode_plan_runtime_args(g, A):
    """:507-573: a plan with DECODE_RUNTIME_POS / _SEQ_LEN sentinels equals the direct ops."""
    if not getattr(g, '_has_decode_plan', False):
        return
    seed = np.zeros(24, np.float32)
    seed[0:6] = [1.0, 2.0, 3.0, 10.0, 20.0, 30.0]
    for mid in (6, 7):
        _f32map(g, A, mid, 24)
        g.scatter(mid, np.arange(24, dtype=np.uint32), seed)
    src_h, dst_h = _h(g, [0, 1, 2]), _h(g, [12, 13, 14])
    spec_h, base_h = _h(g, [1, 0]), _h(g, [0])
    g.batch_begin()
    g.map_op2_dev(6, A.OP_ADD, src_h, src_h, dst_h, 3)
    g.map_row_copy_offset_dev(6, spec_h, base_h, 8, 1, 3)
    g.batch_end()
    ops = [A.DecodePlanOp(kind=A.DECODE_OP_OP2, map_id=7, op_code=A.OP_ADD, h0=src_h, h1=src_h, h2=dst_h,
                          u0=A.DECODE_RUNTIME_SEQ_LEN),
           A.DecodePlanOp(kind=A.DECODE_OP_ROW_COPY_OFFSET, map_id=7, h0=spec_h, h1=base_h,
                          u0=A.DECODE_RUNTIME_POS, u1=1, u2=3)]
    try:
        g.register_decode_plan(1, ops)
        g.decode_step(1, pos=8, seq_len=3)
    finally:
        g.clear_decode_plan(1)
    # the copy's destination row (0 + pos 8) * 3 = 24 lies past the 24-element map in the reference's
    # own scenario, so elements 8..10 stay 0 on both maps; the doubled values land at 12..14
    for probe, lit in (([8, 9, 10], [0.0, 0.0, 0.0]), ([12, 13, 14], [2.0, 4.0, 6.0])):
        d, p = _read(g, 6, probe), _read(g, 7, probe)
        assert np.allclose(d, p, atol=1e-6) and np.allclose(p, lit, atol=1e-6)

def kat_topk(g, A):
    """test_decode_primitives.py:32-45: top 3 of six logits, the tie at 5.5 resolved to the lower index."""
    _f32map(g, A, 10, 20)
    logits = np.array([-3.0, 5.5, 2.0, 5.5, 4.0, -1.0], np.float32)
    g.scatter(10, np.arange(6, dtype=np.uint32), logits)
    g.map_topk_dev(10, _h(g, np.arange(6)), _h(g, [8, 9, 10]), _h(g, [12, 13, 14]), 6, 3)
    assert _read(g, 10, [8, 9, 10]).astype(np.int32).tolist() == [1, 3, 4]
    assert np.allclose(_read(g, 10, [12, 13, 14]), [5.5, 5.5, 4.0], atol=1e-6)


def kat_topp(g, A):
    """:48-60: temperature 1, top_p 0.9 over [5, 4, 1, -1] keeps two candidates."""
    _f32map(g, A, 11, 16)
    g.scatter(11, np.arange(4, dtype=np.uint32), np.array([5.0, 4.0, 1.0, -1.0], np.float32))
    g.map_topp_dev(11, _h(g, [0, 1, 2, 3]), _h(g, [8, 9, 10, 11]), 4, 1.0, 0.9)
    assert np.allclose(_read(g, 11, [8, 9, 10, 11]), [0.7310586, 0.26894143, 0.0, 0.0], atol=1e-5)


def kat_resolve_idx_and_categorical(g, A):
    """:63-95: positions [2, 0] of the id list at 4.. resolve to [33, 11]; r = 0.6 over p = [0.25, 0.75]
    picks the second candidate."""
    _f32map(g, A, 12, 32)   # the reference's wrapper calls this array 16
    vals = np.zeros(32, np.float32)
    vals[4:8] = [11.0, 22.0, 33.0, 44.0]; vals[8:10] = [2.0, 0.0]; vals[16:18] = [0.25, 0.75]; vals[20] = 0.6
    g.scatter(12, np.arange(32, dtype=np.uint32), vals)
    resolved, dst = _h(g, [12, 13]), _h(g, [21])
    g.batch_begin()
    g.map_resolve_idx_dev(12, _h(g, [4]), _h(g, [8, 9]), resolved, 2)
    g.map_sample_categorical_dev(12, resolved, _h(g, [16, 17]), _h(g, [20]), dst, 2)
    g.batch_end()
    assert _read(g, 12, [12, 13]).astype(np.int32).tolist() == [33, 11]
    assert int(_read(g, 12, [21])[0]) == 11


def _diag_q8(g, A, map_id):
    """Q8 rows [1,0,0,0], [0,2,0,0], [0,0,3,0], [0,0,0,4]: codes 128 + value, scale 1, zero point -128."""
    g.map_create_typed(map_id, A.DTYPE_Q8, 1, 16, 4)
    g.set_qparams(map_id, np.ones(4, np.float32), np.full(4, -128.0, np.float32))
    raw = np.full(16, 128, np.uint8)
    raw[[0, 5, 10, 15]] = [129, 130, 131, 132]
    g.scatter(map_id, np.arange(16, dtype=np.uint32), raw)


def kat_matvec_topk_t_xq8(g, A):
    """:217-257: logits [1, 2, 3, 4] of a ones vector, repeat penalty 2 on row 3 (4 -> 2), k = 2:
    [2, 1] with values [3, 2] (the tie at 2.0 goes to the lower row)."""
    _diag_q8(g, A, 7)
    _f32map(g, A, 8, 16)
    g.scatter(8, np.arange(4, dtype=np.uint32), np.ones(4, np.float32))
    idx_h, val_h = _h(g, [4, 5]), _h(g, [8, 9])
    g.batch_begin()
    g.map_matvec_topk_t_xq8_dev(8, 7, _h(g, [0, 1, 2, 3]), _h(g, [0]), _h(g, [3]), idx_h, val_h, 4, 4, 2, 1, 2.0)
    g.batch_end()
    assert _read(g, 8, [4, 5]).astype(np.int32).tolist() == [2, 1]
    assert np.allclose(_read(g, 8, [8, 9]), [3.0, 2.0], atol=1e-5)


def kat_matvec_topk_t_xq4(g, A):
    """:260-301: the same through Q4 weights quantised on the device (scale 4/15): first index 2, second
    1 or 3, values [3, 2] within 0.15."""
    g.map_create_typed(13, A.DTYPE_Q4, 1, 16, 32)
    g.set_qparams(13, np.array([4.0 / 15.0], np.float32), np.array([0.0], np.float32))
    g.scatter(13, np.arange(16, dtype=np.uint32), np.diag([1.0, 2.0, 3.0, 4.0]).astype(np.float32).reshape(-1))
    _f32map(g, A, 14, 16)
    g.scatter(14, np.arange(4, dtype=np.uint32), np.ones(4, np.float32))
    idx_h, val_h = _h(g, [4, 5]), _h(g, [8, 9])
    g.batch_begin()
    g.map_matvec_topk_t_xq4_dev(14, 13, _h(g, [0, 1, 2, 3]), _h(g, [0]), _h(g, [3]), idx_h, val_h, 4, 4, 2, 1, 2.0)
    g.batch_end()
    idx = _read(g, 14, [4, 5]).astype(np.int32)
    assert idx[0] == 2 and idx[1] in (1, 3)
    assert np.allclose(_read(g, 14, [8, 9]), [3.0, 2.0], atol=0.15)


def kat_matvec_rerank_t_xq8(g, A):
    """:304-352: partial id list [0, 1, 2, 3] at 8.., shortlist positions [3, 1]; exact logits 4 and 2, the
    penalty 2 on token 3 -> ids [3, 1], values [2, 2]."""
    _diag_q8(g, A, 13)
    _f32map(g, A, 14, 32)
    vals = np.zeros(32, np.float32)
    vals[0:4] = 1.0; vals[8:12] = [0.0, 1.0, 2.0, 3.0]; vals[12:14] = [3.0, 1.0]
    g.scatter(14, np.arange(32, dtype=np.uint32), vals)
    idx_h, val_h = _h(g, [16, 17]), _h(g, [20, 21])
    g.batch_begin()
    g.map_matvec_rerank_t_xq8_dev(14, 13, _h(g, [0, 1, 2, 3]), _h(g, [0]), _h(g, [8]), _h(g, [12, 13]), _h(g, [3]),
                                  idx_h, val_h, 4, 2, 1, 2.0)
    g.batch_end()
    assert _read(g, 14, [16, 17]).astype(np.int32).tolist() == [3, 1]
    assert np.allclose(_read(g, 14, [20, 21]), [2.0, 2.0], atol=1e-5)


ALL = [kat_argmax, kat_topk, kat_topp, kat_resolve_idx_and_categorical, kat_softmax_abs, kat_attn_softmax_abs, kat_q8_gather_scatter, kat_row_gather_xq8,
       kat_matvec_t_xq8, kat_matvec_t_xq4, kat_q4_matmul_identity, kat_batch_gather_scatter,
       kat_row_copy_offset, kat_fusion_row_copy_then_matmul, kat_scalar_state, kat_fusion_batch_order,
       kat_decode_plan_runtime_args, kat_matvec_topk_t_xq8, kat_matvec_topk_t_xq4, kat_matvec_rerank_t_xq8]
