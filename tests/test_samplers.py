"""Host samplers (TopkSampler / TopPSampler of the reference's
models/samplers.cpp:37-101) against their closed form: the candidate set and
its probabilities are fixed by the logits alone; the draw is checked for
reproducibility under a seed and for its frequencies."""
import numpy as np
import pytest

from vkllama_amd import model as M


def ranked(logits):
    """ids by descending logit, ties toward the lower id"""
    return np.lexsort((np.arange(logits.size), -logits.astype(np.float64)))


def softmax32(x):
    e = np.exp((x - x[0]).astype(np.float32)).astype(np.float32)
    return e / np.float32(e.sum(dtype=np.float32))


@pytest.fixture
def logits():
    rng = np.random.default_rng(5)
    return (rng.standard_normal(32000) * 3).astype(np.float32)


def test_top1_is_argmax_lowest_index_wins(logits):
    s = M.Sampler("topk", 1, seed=1)
    assert s.sample(logits) == int(np.argmax(logits))
    tied = logits.copy()
    tied[[17, 4000, 31999]] = tied.max() + 1
    assert s.sample(tied) == 17
    ids, probs = s.candidates()
    assert ids.tolist() == [17] and probs.tolist() == [1.0]


@pytest.mark.parametrize("k", [2, 40, 1000])
def test_topk_candidates_and_probabilities(logits, k):
    s = M.Sampler("topk", k, seed=3)
    tok = s.sample(logits)
    ids, probs = s.candidates()
    order = ranked(logits)[:k]
    assert np.array_equal(ids, order)
    assert np.allclose(probs, softmax32(logits[order]), rtol=1e-5, atol=1e-9)
    assert abs(float(probs.sum()) - 1) < 1e-4
    assert tok in ids


def test_topk_larger_than_vocabulary_is_clamped():
    x = np.array([0.5, 2.0, -1.0], np.float32)
    s = M.Sampler("topk", 40, seed=0)
    assert s.sample(x) in (0, 1, 2)
    ids, probs = s.candidates()
    assert ids.tolist() == [1, 0, 2]
    assert np.allclose(probs, softmax32(x[[1, 0, 2]]), rtol=1e-6)


@pytest.mark.parametrize("p", [0.0, 0.3, 0.9, 1.0])
def test_topp_candidates_and_probabilities(logits, p):
    s = M.Sampler("topp", p, seed=11)
    tok = s.sample(logits)
    ids, probs = s.candidates()
    order = ranked(logits)
    full = softmax32(logits[order])
    # tokens are added while the mass so far is below p (samplers.cpp:84-89);
    # fp32 sums taken in another order may move a mass that lies within 1e-4
    # of p across it, so both neighbours of such a boundary are accepted
    mass_before = np.concatenate(([0.0], np.cumsum(full.astype(np.float64))[:-1]))
    n_lo = max(int(np.sum(mass_before < p - 1e-4)), 1)
    n_hi = max(int(np.sum(mass_before < p + 1e-4)), 1)
    n = ids.size
    assert n_lo <= n <= n_hi and np.array_equal(ids, order[:n])
    assert np.allclose(probs, softmax32(logits[order[:n]]), rtol=1e-4, atol=1e-9)  # fp32 sum over up to 32000 terms
    assert tok in ids


def test_seed_reproduces_the_sequence(logits):
    a, b, c = M.Sampler("topk", 50, seed=42), M.Sampler("topk", 50, seed=42), M.Sampler("topk", 50, seed=43)
    sa = [a.sample(logits) for _ in range(64)]
    sb = [b.sample(logits) for _ in range(64)]
    sc = [c.sample(logits) for _ in range(64)]
    assert sa == sb and sa != sc
    u = M.Sampler("topk", 50)                    # random-device seed: still a valid draw
    assert u.sample(logits) in a.candidates()[0]


def test_draw_frequencies_follow_the_probabilities():
    x = np.log(np.array([0.5, 0.25, 0.125, 0.0625, 0.0625], np.float32))
    s = M.Sampler("topk", 5, seed=2024)
    n = 40000
    counts = np.bincount([s.sample(x) for _ in range(n)], minlength=5)
    p = np.exp(x.astype(np.float64))
    sigma = np.sqrt(n * p * (1 - p))
    assert np.all(np.abs(counts - n * p) < 5 * sigma)


def test_bad_parameters_are_rejected():
    with pytest.raises(ValueError):
        M.Sampler("topk", 0)
    s = M.Sampler("topp", 0.5, seed=1)
    assert s.sample(np.zeros(0, np.float32)) == -1
