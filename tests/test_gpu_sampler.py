"""GPU parity of the sampler kernel (through the C ABI) against the CPU oracle.

The deterministic parts are compared exactly: the greedy token stream under the penalty recurrence, and the
kept set after top-k / top-p filtering (every drawn token must be in the oracle's kept set).  The stochastic
draw is counter-based (seed, row, step), so it is checked for reproducibility and for its distribution:
empirical frequencies over many (row, step) counters against the oracle's filtered, renormalised
probabilities.  The reference's draw uses a wall-clock seed and cannot be reproduced at all, so the
distribution is the only parity there is for it.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _draw(hip, logits, B, steps, seed, penalties=None, **kw):
    V = logits.shape[-1]
    rows = np.ascontiguousarray(np.broadcast_to(logits, (B, V)), dtype=np.float32)
    d_logits = hip.DeviceArray.from_numpy(rows)
    d_probs = hip.DeviceArray((B, V), np.float32)
    d_out = hip.DeviceArray((B,), np.int32)
    out = np.zeros((steps, B), np.int32)
    for s in range(steps):
        hip.sample(B, V, d_logits, penalties, d_probs, d_out, seed=seed, step=s, **kw)
        hip.device_sync()
        out[s] = d_out.numpy()
    return out


def test_greedy_with_penalties_matches_oracle_stream(gpu, orc):
    hip = gpu
    rng = np.random.default_rng(0)
    V = 65536
    logits = (rng.standard_normal(V) * 3).astype(np.float32)
    logits[[5, 70, 4099]] = logits.max() + 1.0   # exact three-way tie at the top: lowest index wins
    pen_host = np.zeros(V, np.float32)
    d_pen = hip.DeviceArray.zeros((1, V), np.float32)
    got = _draw(hip, logits, 1, 24, seed=1, penalties=d_pen, presence=2.0, frequency=0.5, decay=0.9,
                temperature=0.7, top_k=0, top_p=0.0)[:, 0]
    want = [orc.sample_greedy_penalty(logits, pen_host, 2.0, 0.5, 0.9, 0.7) for _ in range(24)]
    assert got.tolist() == want
    assert got[0] == 5 and len(set(want)) > 3     # the penalties do move the choice around
    err = float(np.max(np.abs(d_pen.numpy()[0] - pen_host)))
    assert err <= 1e-6


@pytest.mark.parametrize("top_k,top_p,temperature", [(20, 0.3, 1.0), (5, 1.0, 1.0), (0, 0.9, 1.5), (50, 0.95, 0.5),
                                                      (1, 1.0, 1.0), (0, 1.0, 2.0)])
def test_draws_stay_in_kept_set_and_follow_filtered_distribution(gpu, orc, top_k, top_p, temperature):
    hip = gpu
    rng = np.random.default_rng(3)
    V = 4096
    logits = (rng.standard_normal(V) * 2.5).astype(np.float32)
    logits[[100, 200, 300]] = logits.max() - 0.5    # ties inside the kept set
    kept, probs = orc.sample_filter(logits, None, temperature, top_k, top_p)
    assert kept >= 1
    B, steps = 64, 128
    draws = _draw(hip, logits, B, steps, seed=77, temperature=temperature, top_k=top_k, top_p=top_p).ravel()
    in_set = bool(np.all(probs[draws] > 0))
    assert in_set
    if top_k == 1:
        assert set(draws.tolist()) == {int(np.argmax(logits))}
        return
    # frequencies: compare on the entries that carry real mass (expected count >= 20), 5 sigma each
    want = probs.astype(np.float64) / probs.sum(dtype=np.float64)
    n = draws.size
    freq = np.bincount(draws, minlength=V) / n
    heavy = np.nonzero(want * n >= 20)[0]
    assert heavy.size >= 1
    sigma = np.sqrt(want[heavy] * (1 - want[heavy]) / n)
    worst = float(np.max(np.abs(freq[heavy] - want[heavy]) / sigma))
    assert worst <= 5.0
    # total variation distance over everything
    tv = 0.5 * float(np.abs(freq - want).sum())
    assert tv <= 0.5 * np.sqrt(max(kept, 1) / n) + 0.02


def test_rows_longer_than_the_register_path_follow_the_filtered_distribution(gpu, orc):
    """Rows of more than 65536 entries keep their slices in the probs scratch instead of registers: same kept set,
    same distribution; greedy picks the lowest index among tied maxima."""
    hip = gpu
    rng = np.random.default_rng(13)
    V = 131072
    logits = (rng.standard_normal(V) * 2.5).astype(np.float32)
    logits[[7, 70000, 131071]] = logits.max() + 0.25      # a tie that straddles the 65536 boundary
    kept, probs = orc.sample_filter(logits, None, 0.8, 12, 0.9)
    draws = _draw(hip, logits, 64, 64, seed=5, temperature=0.8, top_k=12, top_p=0.9).ravel()
    in_set = bool(np.all(probs[draws] > 0))
    assert in_set
    want = probs.astype(np.float64) / probs.sum(dtype=np.float64)
    freq = np.bincount(draws, minlength=V) / draws.size
    heavy = np.nonzero(want * draws.size >= 20)[0]
    assert heavy.size >= 3
    sigma = np.sqrt(want[heavy] * (1 - want[heavy]) / draws.size)
    worst = float(np.max(np.abs(freq[heavy] - want[heavy]) / sigma))
    assert worst <= 5.0
    greedy = _draw(hip, logits, 2, 2, seed=1, top_k=1).ravel()
    assert set(greedy.tolist()) == {7}


def test_draw_is_a_function_of_seed_row_and_step(gpu):
    hip = gpu
    rng = np.random.default_rng(5)
    logits = rng.standard_normal(2048).astype(np.float32)
    a = _draw(hip, logits, 8, 16, seed=11, top_k=0, top_p=1.0)
    b = _draw(hip, logits, 8, 16, seed=11, top_k=0, top_p=1.0)
    c = _draw(hip, logits, 8, 16, seed=12, top_k=0, top_p=1.0)
    assert np.array_equal(a, b)
    assert not np.array_equal(a, c)
    rows_differ = len({tuple(a[:, r]) for r in range(8)}) > 1
    steps_differ = len({tuple(a[s]) for s in range(16)}) > 1
    assert rows_differ and steps_differ


def test_argmax_picks_lowest_index_among_ties(gpu):
    hip = gpu
    rng = np.random.default_rng(9)
    B, V = 5, 65536
    logits = rng.standard_normal((B, V)).astype(np.float32)
    logits[0, [70000 % V, 123, 60000]] = 9.0
    logits[1, V - 1] = 9.0
    logits[2, 0] = 9.0
    logits[3] = -np.inf
    logits[3, 4097] = -1e30
    out = hip.DeviceArray((B,), np.int32)
    hip.argmax(B, V, hip.DeviceArray.from_numpy(logits), out)
    hip.device_sync()
    assert out.numpy().tolist() == np.argmax(logits, axis=1).tolist()


def test_sampler_argument_errors(gpu):
    hip = gpu
    d = hip.DeviceArray((1, 8), np.float32)
    o = hip.DeviceArray((1,), np.int32)
    with pytest.raises(hip.RwkvHipError, match="multiple of 4"):
        hip.sample(1, 6, d, None, d, o)
    with pytest.raises(hip.RwkvHipError, match="Temperature outside range"):
        hip.sample(1, 8, d, None, d, o, temperature=0.0)
    with pytest.raises(hip.RwkvHipError, match="B must be positive"):
        hip.sample(0, 8, d, None, d, o)
