"""TokenSampler (Noeda/rllama src/token_sampler.rs:83-174): the oracle's restatement against a closed form written
independently in float64, then the library's host implementation against the oracle.  CPU only (host arithmetic)."""
import numpy as np
import pytest

import oracle
import rllama_amd


def closed_form(logits, temperature, top_p, top_k, penalty, existing):
    """What the reference computes, derived by hand from :99-159 in float64: token 0's logit becomes exactly 0 (the penalty
    and the 'maximum' only ever touch token 0), every other logit is divided by the temperature, softmax, then the cuts."""
    l = np.asarray(logits, np.float64).copy()
    if temperature > 0:
        l = l / temperature
    l[0] = 0.0
    p = np.exp(l)
    p = p / p.sum()
    order = sorted(range(len(p)), key=lambda i: (-p[i], i))[:top_k]
    acc, keep = 0.0, []
    for i in order:
        keep.append(i)
        acc += p[i]
        if acc >= top_p:
            break
    return np.array(keep), p[keep], float(p[keep].sum())


CASES = [
    dict(temperature=1.0, top_p=1.0, top_k=5, penalty=1.0, existing=[]),
    dict(temperature=0.2, top_p=1.0, top_k=1, penalty=0.8, existing=[3, 0, 0, 7]),        # TokenSampler::new() defaults
    dict(temperature=0.7, top_p=0.9, top_k=40, penalty=1.3, existing=[0, 5, 5, 9]),
    dict(temperature=2.5, top_p=0.5, top_k=1000, penalty=0.5, existing=[1, 2, 3]),
    dict(temperature=0.0, top_p=0.95, top_k=10, penalty=1.0, existing=[]),                # temperature 0: logits used as they are
    dict(temperature=1.0, top_p=2.0, top_k=10**9, penalty=1.0, existing=[]),              # no cut at all
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("vocab", [2, 17, 1000, 32000])
def test_oracle_candidates_match_closed_form(case, vocab):
    rng = np.random.default_rng(vocab)
    logits = (rng.standard_normal(vocab) * 3).astype(np.float32)
    ids, probs, total = oracle.sample_candidates(logits, case["temperature"], case["top_p"], case["top_k"], case["penalty"], case["existing"])
    wi, wp, wt = closed_form(logits, case["temperature"], case["top_p"], case["top_k"], case["penalty"], case["existing"])
    # fp32 against float64: the same ids except where two probabilities differ by less than fp32 noise, or the top-p sum lands within noise of the threshold
    assert abs(len(ids) - len(wi)) <= 1
    m = min(len(ids), len(wi))
    same = ids[:m] == wi[:m]
    rtol = 2e-5 if vocab < 1000 else 1e-4  # the reference's sequential fp32 sum over the vocabulary drifts by about sqrt(vocab) ulp
    assert np.all(same | (np.abs(probs[:m] - wp[:m]) <= rtol * wp[:m]))
    assert np.allclose(probs[:m], wp[:m], rtol=rtol, atol=1e-12)
    if len(ids) == len(wi):
        assert abs(total - wt) <= rtol * max(wt, 1e-30)
    assert np.all(np.diff(probs) <= 0)


def test_oracle_token0_quirks():
    """Only token 0 is shifted and penalised (token_sampler.rs:105, :113, :121 loop over the rows of a 1 x vocab tensor)."""
    logits = np.array([5.0, 1.0, 2.0, -1.0], np.float32)
    ids, probs, _ = oracle.sample_candidates(logits, 1.0, 1.0, 4, 1.0, [])
    e = np.exp(np.array([0.0, 1.0, 2.0, -1.0]))
    assert list(ids) == [2, 1, 0, 3] and np.allclose(probs, (e / e.sum())[[2, 1, 0, 3]], rtol=1e-6)
    # a penalty on other tokens changes nothing; on token 0 it changes nothing either, because the shift removes it again
    for existing in ([1, 1, 2], [0, 0, 0]):
        i2, p2, _ = oracle.sample_candidates(logits, 1.0, 1.0, 4, 0.25, existing)
        assert list(i2) == [2, 1, 0, 3] and np.array_equal(p2, probs)
    # no maximum is subtracted from the others: large logits overflow exp() and the probabilities turn into NaN, sorted last
    ids, probs, _ = oracle.sample_candidates(np.array([0.0, 100.0, 1.0], np.float32), 1.0, 1.0, 3, 1.0, [])
    assert np.isnan(probs[-1]) and set(ids) == {0, 1, 2}
    # top_k == 1 agrees with the greedy entry point
    for seed in range(5):
        lg = (np.random.default_rng(seed).standard_normal(500) * 4).astype(np.float32)
        ids, probs, total = oracle.sample_candidates(lg, 0.2, 1.0, 1, 0.8, [4, 0])
        tok, p, _ = oracle.sample_greedy(lg, 0.2)
        assert ids[0] == tok and probs[0] == np.float32(p) and total == float(probs[0])


def test_oracle_pick_walks_the_cumulative_sum():
    ids, probs = np.array([7, 3, 9], np.int32), np.array([0.5, 0.25, 0.125], np.float32)
    total = 0.875
    assert oracle.sample_pick(ids, probs, total, 0.0) == (7, pytest.approx(0.5 / total))
    assert oracle.sample_pick(ids, probs, total, 0.5 / total)[0] == 7          # acc >= p picks on equality
    assert oracle.sample_pick(ids, probs, total, 0.58)[0] == 3
    assert oracle.sample_pick(ids, probs, total, 1.0)[0] == 9
    assert oracle.sample_pick(ids[:0], probs[:0], 0.0, 0.3) == (0, 0.0)        # nothing left: the fall-through (0, 0.0)
    # drawing many times reproduces the distribution
    rng = np.random.default_rng(1)
    picks = [oracle.sample_pick(ids, probs, total, float(u))[0] for u in rng.random(20000)]
    freq = np.array([picks.count(t) for t in ids]) / len(picks)
    assert np.allclose(freq, probs / total, atol=0.012)


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("vocab", [2, 17, 1000, 32000])
def test_library_sampler_equals_oracle(case, vocab):
    rng = np.random.default_rng(100 + vocab)
    logits = (rng.standard_normal(vocab) * 3).astype(np.float32)
    if vocab > 20:
        logits[5] = logits[11] = logits[2]  # exact ties: both order them by id
    ts = rllama_amd.TokenSampler().temperature(case["temperature"]).top_p(case["top_p"]).top_k(case["top_k"]).repetition_penalty(case["penalty"])
    ids, probs, total = ts.candidates(logits, case["existing"])
    oi, op, ot = oracle.sample_candidates(logits, case["temperature"], case["top_p"], case["top_k"], case["penalty"], case["existing"])
    assert np.array_equal(ids, oi) and np.array_equal(probs, op) and total == ot
    for u in (0.0, 0.3, 0.77, 1.0):
        class _U:
            def random(self, dtype=None):
                return np.float32(u)
        tok, p = ts.sample(logits, case["existing"], _U())
        assert (tok, p) == oracle.sample_pick(oi, op, ot, u)


def test_library_sampler_settings_and_errors():
    ts = rllama_amd.TokenSampler()
    assert (ts.get_temperature(), ts.get_top_p(), ts.get_top_k(), ts.get_repetition_penalty()) == (pytest.approx(0.2), 1.0, 1, pytest.approx(0.8))
    t2 = ts.top_k(50).temperature(1.5)
    assert (t2.get_top_k(), t2.get_temperature(), ts.get_top_k()) == (50, 1.5, 1)  # builder style: the original is unchanged
    nan_case = np.array([0.0, 100.0, 1.0], np.float32)
    ids, probs, _ = ts.top_k(3).temperature(1.0).repetition_penalty(1.0).candidates(nan_case)
    oi, op, _ = oracle.sample_candidates(nan_case, 1.0, 1.0, 3, 1.0, [])
    assert np.array_equal(ids, oi) and np.array_equal(np.isnan(probs), np.isnan(op))
    with pytest.raises(rllama_amd.RllamaHipError):
        class _Bad:
            def random(self, dtype=None):
                return np.float32(1.5)
        ts.sample(np.zeros(4, np.float32), [], _Bad())
