"""The oracle's temperature / top-p sampler over packed top-k lists, pinned by the scenario the reference's own
hardware test checks its kernel with (go/engine/hip/hip_hardware_test.go:582-640: 64 candidates 60 - rank/2 in a
262144-token vocabulary, softcap 30, top-k 40 / 64, top-p 1 / 0.95, five draws, against the host sampler over the
soft-capped logits), by closed forms (weights 3:1, a nucleus cut on known weights, temperature as a rescaling of
the scores) and by numpy's softmax as the distribution the draws must follow."""
import numpy as np
import pytest

from oracle import orc


def _pack(scores, tokens=None):
    tokens = range(len(scores)) if tokens is None else tokens
    return np.array([orc.pack_greedy_best(float(s), int(t)) for s, t in zip(scores, tokens)], dtype=np.uint64)


def _tok(packed):
    return orc.unpack_greedy_best(packed)[0] if packed else None


def test_reference_hardware_scenario_matches_host_sampler():
    V = 262144
    logits = np.full(V, -100, np.float32)
    for rank in range(64):
        logits[200000 + rank * 17] = 60 - rank / 2
    packed = _pack(logits)
    host = orc.softcap_logits(logits, 30)
    seen = set()
    for k in (40, 64):
        top = np.sort(packed)[::-1][:k]
        for top_p in (1.0, 0.95):
            for draw in (0, 0.1, 0.5, 0.9, 0.999999):
                got = _tok(orc.packed_topk_sample(top, 1.0, top_p, 30.0, draw))
                want, _ = orc.host_sample(host, 1.0, k, top_p, draw)
                assert got == want, (k, top_p, draw)
                seen.add(got)
    assert len(seen) > 8                      # the draws really spread over the candidates


def test_closed_forms():
    two = _pack([np.log(3.0), 0.0], [7, 9])                       # weights 3 : 1
    assert [_tok(orc.packed_topk_sample(two, 1.0, 1.0, 0.0, d)) for d in (0.0, 0.5, 0.7499, 0.7501, 0.99, 1.0, 5.0, -1.0)] == \
        [7, 7, 7, 9, 9, 9, 9, 7]
    # temperature divides the scores: 2 ln 3 at temperature 2 is the same distribution
    hot = _pack([2 * np.log(3.0), 0.0], [7, 9])
    assert [_tok(orc.packed_topk_sample(hot, 2.0, 1.0, 0.0, d)) for d in (0.74, 0.76)] == [7, 9]
    # a zero of temperature or of top-p alone stands for 1; both zero: greedy
    assert _tok(orc.packed_topk_sample(two, 0.0, 1.0, 0.0, 0.76)) == 9
    assert _tok(orc.packed_topk_sample(two, 1.0, 0.0, 0.0, 0.76)) == 9
    assert _tok(orc.packed_topk_sample(two, 0.0, 0.0, 0.0, 0.99)) == 7
    # nucleus: weights 0.5, 0.3, 0.2 -> top-p 0.7 keeps two (0.8 >= 0.7), draws are over the kept 0.8
    three = _pack(np.log([0.5, 0.3, 0.2]), [4, 5, 6])
    assert [_tok(orc.packed_topk_sample(three, 1.0, 0.7, 0.0, d)) for d in (0.0, 0.62, 0.63, 0.999)] == [4, 4, 5, 5]
    assert _tok(orc.packed_topk_sample(three, 1.0, 1.0, 0.0, 0.999)) == 6
    assert _tok(orc.packed_topk_sample(three, 1.0, 0.5, 0.0, 0.999)) == 4          # 0.5 >= 0.5: one candidate
    # softcap: scores tanh(s/c)*c; with c = 1 the scores 10 and 0.5 become ~1 and 0.4621 -> weights 1 : e^(0.4621-1)
    capped = _pack([10.0, 0.5], [1, 2])
    p_first = 1.0 / (1.0 + np.exp(np.tanh(0.5) - np.tanh(10.0)))
    assert _tok(orc.packed_topk_sample(capped, 1.0, 1.0, 1.0, p_first - 1e-6)) == 1
    assert _tok(orc.packed_topk_sample(capped, 1.0, 1.0, 1.0, p_first + 1e-6)) == 2
    # holes are skipped, an empty list gives nothing
    holes = np.array([0, two[0], 0, two[1], 0], dtype=np.uint64)
    assert [_tok(orc.packed_topk_sample(holes, 1.0, 1.0, 0.0, d)) for d in (0.74, 0.76)] == [7, 9]
    assert orc.packed_topk_sample(np.zeros(4, np.uint64), 1.0, 1.0, 0.0, 0.3) == 0
    assert _tok(orc.packed_topk_sample(holes, 0.0, 0.0, 0.0, 0.9)) == 7


def test_draws_follow_the_softmax():
    rng = np.random.default_rng(5)
    scores = np.sort(rng.normal(0, 2, 40).astype(np.float32))[::-1]
    top = _pack(scores, rng.permutation(1000)[:40])
    for temperature in (0.7, 1.0, 1.8):
        z = scores.astype(np.float64) / temperature
        prob = np.exp(z - z.max())
        prob /= prob.sum()
        draws = (np.arange(20000) + 0.5) / 20000
        picks = np.array([orc.packed_topk_sample(top, temperature, 1.0, 0.0, d) for d in draws], dtype=np.uint64)
        freq = np.array([(picks == p).mean() for p in top])
        assert np.abs(freq - prob).max() < 1e-4


def test_argument_rules():
    top = _pack([1.0, 0.0])
    for args in ((-1.0, 1.0, 0.0, 0.5), (np.inf, 1.0, 0.0, 0.5), (1.0, 1.5, 0.0, 0.5), (1.0, -0.1, 0.0, 0.5),
                 (1.0, 1.0, -1.0, 0.5), (1.0, 1.0, 0.0, np.nan), (np.nan, 1.0, 0.0, 0.5)):
        with pytest.raises(orc.OracleError) as e:
            orc.packed_topk_sample(top, *args)
        assert e.value.code == orc.ORC_ERR_SIZE
    with pytest.raises(orc.OracleError):
        orc.packed_topk_sample(np.zeros(129, np.uint64), 1.0, 1.0, 0.0, 0.5)
    with pytest.raises(orc.OracleError):
        orc.host_sample(np.zeros(4, np.float32), 1.0, 9, 1.0, 0.5)
    with pytest.raises(orc.OracleError):
        orc.host_sample(np.full(4, np.nan, np.float32), 1.0, 2, 1.0, 0.5)
    assert orc.host_sample(np.array([0.5, 2.0, 2.0], np.float32), 0.0, 0, 0.0, 0.9)[0] == 1      # greedy: first maximum
