"""Sampling on the device (vkl_sample_f32) against the closed form of the
host samplers: candidate set and probabilities follow from the logits, the
draw from the documented counter-based uniform number."""
import ctypes as C

import numpy as np
import pytest

from vkllama_amd import capi

pytestmark = pytest.mark.gpu
M64 = (1 << 64) - 1


@pytest.fixture(scope="module")
def dev():
    return capi.Device(0)


def uniform01(seed, counter):
    z = (seed + 0x9E3779B97F4A7C15 * (counter + 1)) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    z ^= z >> 31
    return np.float32(z >> 40) * np.float32(1.0 / 16777216.0)


def ranked(logits):
    return np.lexsort((np.arange(logits.size), -logits.astype(np.float64)))


def softmax_seq(x):
    e = np.exp((x - x[0]).astype(np.float32)).astype(np.float32)
    return e / np.cumsum(e, dtype=np.float32)[-1]


def run(dev, logits, k, p, seed, counter, counter_dev=None):
    L = capi.lib()
    dl = dev.upload(logits)
    tok, ids, probs, n = dev.alloc(4), dev.alloc(4096), dev.alloc(4096), dev.alloc(4)
    cd = dev.upload(np.array([counter_dev], np.uint32)) if counter_dev is not None else None
    capi.check(L.vkl_sample_f32(dl.ptr, logits.size, k, C.c_float(p), seed, counter, cd.ptr if cd else None,
                                tok.ptr, ids.ptr, probs.ptr, n.ptr, dev.stream), "vkl_sample_f32")
    nn = int(n.read(np.uint32, (1,))[0])
    return int(tok.read(np.uint32, (1,))[0]), ids.read(np.uint32, (1024,))[:nn], probs.read(np.float32, (1024,))[:nn]


@pytest.fixture
def logits():
    rng = np.random.default_rng(9)
    return (rng.standard_normal(32000) * 3).astype(np.float32)


def test_top1_is_the_lowest_index_argmax(dev, logits):
    x = logits.copy()
    x[[77, 9000, 31999]] = x.max() + 2
    tok, ids, probs = run(dev, x, 1, -1.0, 5, 0)
    assert tok == 77 and ids.tolist() == [77] and probs.tolist() == [1.0]
    x[:] = -1.5                                   # all equal: id 0
    assert run(dev, x, 1, -1.0, 5, 0)[0] == 0


@pytest.mark.parametrize("k", [2, 40, 64, 1000, 5000])
@pytest.mark.parametrize("V", [32000, 1000, 37])
def test_topk_candidates_probabilities_and_draw(dev, logits, k, V):
    x = logits[:V].copy()
    x[5] = x[11] = x[3]                            # ties inside the vocabulary
    for counter in (0, 1, 12345):
        tok, ids, probs = run(dev, x, k, -1.0, 42, counter)
        keep = min(k, 1024, V)
        order = ranked(x)[:keep]
        assert np.array_equal(ids, order)
        want = softmax_seq(x[order])
        assert np.allclose(probs, want, rtol=2e-5, atol=1e-12)
        cum = np.cumsum(probs, dtype=np.float32)
        hit = np.nonzero(cum > uniform01(42, counter))[0]
        assert tok == ids[hit[0] if hit.size else keep - 1]


@pytest.mark.parametrize("p", [0.0, 0.3, 0.9, 1.0])
def test_topp_candidates(dev, logits, p):
    tok, ids, probs = run(dev, logits, 0, p, 7, 3)
    order = ranked(logits)
    full = softmax_seq(logits[order]).astype(np.float64)
    mass_before = np.concatenate(([0.0], np.cumsum(full)[:-1]))
    n_lo = min(max(int(np.sum(mass_before < p - 1e-4)), 1), 1024)
    n_hi = min(max(int(np.sum(mass_before < p + 1e-4)), 1), 1024)
    assert n_lo <= ids.size <= n_hi
    assert np.array_equal(ids, order[:ids.size])
    assert np.allclose(probs, softmax_seq(logits[order[:ids.size]]), rtol=1e-4, atol=1e-12)
    assert tok in ids


def test_device_counter_advances_the_generator(dev, logits):
    a = run(dev, logits, 50, -1.0, 99, 10, counter_dev=5)[0]
    b = run(dev, logits, 50, -1.0, 99, 15)[0]
    assert a == b
    toks = {run(dev, logits, 50, -1.0, 99, c)[0] for c in range(40)}
    assert len(toks) > 5                           # different counters, different draws


def test_draw_frequencies(dev):
    x = np.log(np.array([0.5, 0.25, 0.125, 0.0625, 0.0625], np.float32))
    L = capi.lib()
    n = 6000
    dl, toks = dev.upload(x), dev.alloc(4 * n)
    for i in range(n):
        capi.check(L.vkl_sample_f32(dl.ptr, 5, 5, C.c_float(-1.0), 2024, i, None, toks.ptr.value + 4 * i, None, None, None,
                                    dev.stream), "vkl_sample_f32")
    counts = np.bincount(toks.read(np.uint32, (n,)), minlength=5)
    pr = np.exp(x.astype(np.float64))
    assert np.all(np.abs(counts - n * pr) < 5 * np.sqrt(n * pr * (1 - pr)))


def test_arguments_are_checked(dev, logits):
    L = capi.lib()
    dl, tok = dev.upload(logits), dev.alloc(4)
    assert L.vkl_sample_f32(dl.ptr, 32000, 0, C.c_float(-1.0), 1, 0, None, tok.ptr, None, None, None, dev.stream) != 0
    assert L.vkl_sample_f32(dl.ptr, 32000, 0, C.c_float(1.5), 1, 0, None, tok.ptr, None, None, None, dev.stream) != 0
    assert L.vkl_sample_f32(None, 32000, 4, C.c_float(-1.0), 1, 0, None, tok.ptr, None, None, None, dev.stream) != 0
