"""Sampling tail (top-k, top-p, index resolution, categorical draw, repetition penalty): HIP vs oracle.

Bit-exact for indices and copied values; probabilities within 1e-6 (one expf per candidate)."""
import numpy as np
import pytest

import oracle
from adam_amd import adamah as A
from gpu_util import note, up, f32map, read

pytestmark = pytest.mark.gpu


def pair(hip):
    return [hip, oracle.init()]


# 4096 < n <= 40960 takes the selection kernel (one launch), everything else the rounds: sizes on both sides of both
# limits, the sampled LM head's 1024 lists of 40, a list with more ties than k at the k-th value
@pytest.mark.parametrize("n,k,seed", [(6, 3, 0), (100, 64, 1), (262144, 8, 2), (1000, 40, 3), (5, 9, 4), (257, 1, 5),
                                      (4096, 40, 6), (4097, 40, 7), (40960, 40, 8), (40961, 40, 9), (12345, 64, 10),
                                      (30000, 1, 11), (8000, 33, 12)])
def test_topk(hip, n, k, seed):
    rng = np.random.default_rng(seed)
    v = (rng.integers(-50, 50, n) / 4).astype(np.float32)         # ties on purpose
    if n > 8:
        v[rng.integers(0, n, 3)] = np.nan
    if seed == 12:
        v[:] = np.float32(1.5)                                     # every candidate ties: the lowest indices win
        v[7000] = np.float32(2.0)
    outs = []
    for g in pair(hip):
        note(f"topk n={n} k={k}")
        f32map(g, 0, n + 256, np.concatenate([v, np.full(256, 9.0, np.float32)]))
        g.map_topk_dev(0, up(g, np.arange(n)), up(g, n + np.arange(k)), up(g, n + 128 + np.arange(k)), n, k)
        outs.append((read(g, 0, n, k), read(g, 0, n + 128, k)))
    assert np.array_equal(outs[0][0], outs[1][0])
    assert np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32))


@pytest.mark.parametrize("n,temp,top_p,seed", [(4, 1.0, 0.9, 0), (64, 0.7, 0.95, 1), (40, 1.5, 0.3, 2), (8, 1e-9, 0.5, 3),
                                               (16, 1.0, 1.0, 4), (10, 1.0, 0.0, 5)])
def test_topp(hip, n, temp, top_p, seed):
    rng = np.random.default_rng(seed)
    v = np.sort(rng.standard_normal(n).astype(np.float32) * 3)[::-1].copy()
    if n >= 16:
        v[5] = np.nan; v[9] = np.inf
    outs = []
    for g in pair(hip):
        note(f"topp n={n} T={temp} p={top_p}")
        f32map(g, 0, 256, np.concatenate([v, np.zeros(256 - n, np.float32)]))
        g.map_topp_dev(0, up(g, np.arange(n)), up(g, 128 + np.arange(n)), n, temp, top_p)
        outs.append(read(g, 0, 128, n))
    assert np.allclose(outs[0], outs[1], atol=1e-6)
    assert np.array_equal(outs[0] == 0, outs[1] == 0)              # same candidates kept


def test_resolve_categorical_penalty_chain(hip):
    """The sampling sequence of a decode step: top-k, top-p, draw, resolve -- and the repetition penalty."""
    rng = np.random.default_rng(11)
    V, k = 5000, 40
    logits = rng.standard_normal(V).astype(np.float32) * 4
    recent = rng.integers(0, V, 64)
    for r in (0.0, 0.37, 0.93, 0.99999994):
        outs = []
        for g in pair(hip):
            note(f"sampling chain r={r}")
            f32map(g, 0, V + 512, np.concatenate([logits, np.zeros(512, np.float32)]))
            g.scatter(0, np.array([V + 300], np.uint32), np.array([r], np.float32))
            all_locs = up(g, np.arange(V))
            idx, val, prob = up(g, V + np.arange(k)), up(g, V + 64 + np.arange(k)), up(g, V + 128 + np.arange(k))
            g.batch_begin()
            g.map_repeat_penalty_dev(0, all_locs, up(g, recent), 64, 1.3)
            g.map_topk_dev(0, all_locs, idx, val, V, k)
            g.map_topp_dev(0, val, prob, k, 0.8, 0.9)
            g.map_sample_categorical_dev(0, idx, prob, up(g, [V + 300]), up(g, [V + 301]), k)
            g.map_resolve_idx_dev(0, up(g, [V]), up(g, [V + 302]), up(g, [V + 303]), 1)
            g.batch_end()
            outs.append((read(g, 0, 0, V), read(g, 0, V, k), read(g, 0, V + 128, k), read(g, 0, V + 301, 1), read(g, 0, V + 303, 1)))
        assert np.array_equal(outs[0][0].view(np.uint32), outs[1][0].view(np.uint32))   # penalised logits
        assert np.array_equal(outs[0][1], outs[1][1])                                   # candidate ids
        assert np.allclose(outs[0][2], outs[1][2], atol=1e-6)
        assert outs[0][3][0] == outs[1][3][0] and outs[0][4][0] == outs[1][4][0]


def test_limits_and_errors(hip):
    note("sampling limits")
    f32map(hip, 0, 256, np.zeros(256, np.float32))
    h = up(hip, np.arange(128))
    with pytest.raises(RuntimeError, match="code -3"):
        hip.map_topk_dev(0, h, h, h, 128, 65)
    with pytest.raises(RuntimeError, match="code -3"):
        hip.map_topp_dev(0, h, h, 65, 1.0, 0.9)
    with pytest.raises(RuntimeError, match="code -3"):
        hip.map_sample_categorical_dev(0, h, h, h, h, 65)
    with pytest.raises(RuntimeError, match="code -3"):
        hip.map_repeat_penalty_dev(0, h, h, 65, 1.1)
    with pytest.raises(RuntimeError, match="code -3"):
        hip.map_topk_dev(0, up(hip, [1, 2]), h, h, 3, 1)          # handle shorter than n
    hip.map_topk_dev(0, h, h, h, 0, 4)                            # empty: accepted, nothing done
    hip.map_topp_dev(0, h, h, 0, 1.0, 0.9)
