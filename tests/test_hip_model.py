"""The llama2 token loop on the GPU (C++ drop-in classes through the C ABI of
include/vkl_model.h) against the CPU oracle on the same seeded weights.

Bars: greedy token ids identical to the oracle's; fp32 logits (fp16 values
widened) within 1e-2 of the oracle relative to the largest logit; KV-cache
contents within one fp16 ulp in layer 0 and 1e-2 deeper down.
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from vkllama_amd import capi, model as M

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

SMALL = dict(dim=256, n_layers=3, n_heads=4, ffn=704, vocab=1024, maxlen=64, eps=1e-5, wtype=8)
SMALL128 = dict(dim=256, n_layers=2, n_heads=2, ffn=352, vocab=640, maxlen=48, eps=1e-5, wtype=8)
# the tiny-llama benchmark configuration
TINY = dict(dim=512, n_layers=8, n_heads=8, ffn=1376, vocab=32000, maxlen=512, eps=1e-5, wtype=8)


def logit_err(got, want):
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-6))


def set_path(m, fused):
    """0: operator chain for single tokens too; 1: fused decode step, one launch
    per phase; 2: fused decode step, one launch per layer (the default)."""
    m.set_option("fused_decode", int(fused > 0))
    if fused:
        m.set_option("decode_mode", fused - 1)


@pytest.fixture(scope="module")
def small():
    w = M.synth_weights(SMALL, seed=11)
    return SMALL, w


@pytest.mark.parametrize("fused", [0, 1, 2])
def test_prefill_then_decode_logits_and_caches(small, fused):
    cfg, w = small
    prompt = np.array([5, 17, 99, 3, 64, 8, 1000], np.uint32)
    m = M.Llama2(cfg, w)
    set_path(m, fused)
    om = O.OracleModel(cfg, w)
    got = m.forward(prompt, 0)
    want = om.forward(prompt, 0)
    assert logit_err(got, want) < 1e-2
    pos = len(prompt)
    for tok in (7, 300, 12):
        got = m.forward([tok], pos)
        want = om.forward([tok], pos)
        assert logit_err(got, want) < 1e-2, (fused, pos)
        pos += 1
    for layer in range(cfg["n_layers"]):
        for value in (0, 1):
            g = m.read_kv_cache(layer, value)[:, :pos].astype(np.float32)
            o = (om.vcache(layer) if value else om.kcache(layer))[:, :pos].astype(np.float32)
            assert np.abs(g - o).max() <= 1e-2 * max(np.abs(o).max(), 1e-3), (layer, value)
            # untouched cache rows stay zero
            assert not m.read_kv_cache(layer, value)[:, pos:].any()
    m.close()


def test_decode_from_position_zero_to_the_last_position():
    """One-token steps from an empty cache (context length 1) up to the last
    position the cache holds, with a cache length that is not a multiple of 4."""
    cfg = dict(SMALL, maxlen=26)
    w = M.synth_weights(cfg, seed=3)
    m = M.Llama2(cfg, w)
    m.set_option("fused_decode", 1)
    om = O.OracleModel(cfg, w)
    tok = 5
    for pos in range(cfg["maxlen"]):
        got = m.forward([tok], pos)
        want = om.forward([tok], pos)
        assert logit_err(got, want) < 1e-2, pos
        assert int(np.argmax(got)) == int(np.argmax(want)), pos
        tok = int(np.argmax(want))
    m.close()


def test_fused_decode_equals_operator_chain(small):
    cfg, w = small
    prompt = np.array([9, 8, 7, 6], np.uint32)
    a, b = M.Llama2(cfg, w), M.Llama2(cfg, w)
    a.set_option("fused_decode", 1)
    b.set_option("fused_decode", 0)
    la, lb = a.forward(prompt, 0), b.forward(prompt, 0)
    assert np.array_equal(la, lb)                          # same prefill path
    pos = len(prompt)
    for tok in (1, 2, 3, 4, 5):
        la, lb = a.forward([tok], pos), b.forward([tok], pos)
        assert logit_err(la, lb) < 5e-3
        assert int(np.argmax(la)) == int(np.argmax(lb))
        pos += 1
    a.close(), b.close()


@pytest.mark.parametrize("cfg,seed", [(SMALL, 11), (SMALL128, 5)])
@pytest.mark.parametrize("fused", [0, 1, 2])
def test_greedy_ids_identical_to_oracle_small(cfg, seed, fused):
    w = M.synth_weights(cfg, seed=seed)
    prompt = np.array([5, 17, 99, 3], np.uint32)
    m = M.Llama2(cfg, w)
    set_path(m, fused)
    ids, _, _ = m.generate_greedy(prompt, 24)
    want, _ = O.OracleModel(cfg, w).generate_greedy(prompt, 24)
    assert list(ids) == list(want)
    m.close()


@pytest.mark.parametrize("wtype", [8, 1])
def test_wide_rows_decode_and_prompt(wtype):
    """Row widths of the 13B shape (dim 5120, ffn 13824: activation rows of two
    and four 4096-value chunks, weight rows of more than one item, 40 heads) on
    a one-layer model: prompt pass and one-token steps against the oracle."""
    cfg = dict(dim=5120, n_layers=1, n_heads=40, ffn=13824, vocab=512, maxlen=48, eps=1e-5, wtype=wtype)
    w = M.synth_weights(cfg, seed=7)
    m = M.Llama2(cfg, w)
    om = O.OracleModel(cfg, w)
    prompt = np.array([5, 17, 99, 3, 64, 8, 300, 2, 11], np.uint32)
    assert logit_err(m.forward(prompt, 0), om.forward(prompt, 0)) < 1e-2
    pos, tok = len(prompt), 7
    for _ in range(4):
        got, want = m.forward([tok], pos), om.forward([tok], pos)
        assert logit_err(got, want) < 1e-2, pos
        assert int(np.argmax(got)) == int(np.argmax(want)), pos
        tok, pos = int(np.argmax(want)), pos + 1
    ids, _, _ = m.generate_greedy(prompt, 8)
    want_ids, _ = om.generate_greedy(prompt, 8)
    assert list(ids) == list(want_ids)
    m.close()


def test_full_width_properties():
    """The 7B widths (dim 4096, ffn 11008, 32 heads, vocabulary 32000) on two
    layers, through properties that need no oracle: the decode step and the
    prompt pass agree on the same position, generation is repeatable bit for
    bit, and the replayed graph gives the ids of the step-by-step launches."""
    cfg = dict(dim=4096, n_layers=2, n_heads=32, ffn=11008, vocab=32000, maxlen=96, eps=1e-5, wtype=8)
    w = M.synth_weights(cfg, seed=99)
    m = M.Llama2(cfg, w)
    # (the reference rotates the last block's query of a prompt pass at the
    # pass's first position; with that reproduced the two would differ)
    m.set_option("lastblock_rope_quirk", 0)
    rng = np.random.default_rng(99)
    prompt = rng.integers(3, cfg["vocab"], 40).astype(np.uint32)
    whole = m.forward(prompt, 0)                 # prompt pass, last row
    m.forward(prompt[:-1], 0)
    step = m.forward(prompt[-1:], len(prompt) - 1)  # the same position as a decode step
    assert logit_err(step, whole) < 1e-2
    assert int(np.argmax(step)) == int(np.argmax(whole))
    runs = []
    for graph in (1, 1, 0):
        m.set_option("decode_graph", graph)
        ids, _, _ = m.generate_greedy(prompt, 32)
        runs.append(list(ids))
    assert runs[0] == runs[1] == runs[2]
    m.close()


def test_tiny_llama_config2_greedy_128_tokens():
    """Tiny-llama benchmark configuration: prompt of 16 ids in [3, 32000), greedy 128 tokens;
    the first 32 must equal the oracle's (here: all of them are compared and
    the fixture pins the oracle's own sequence)."""
    w = M.synth_weights(TINY, seed=1234)
    rng = np.random.default_rng(1234)
    prompt = rng.integers(3, 32000, 16).astype(np.uint32)
    m = M.Llama2(TINY, w)
    ids, t_pre, t_dec = m.generate_greedy(prompt, 128)
    want, _ = O.OracleModel(TINY, w).generate_greedy(prompt, 128)
    assert list(ids[:32]) == list(want[:32])
    n_same = int(np.argmax(np.concatenate([ids != want, [True]])))
    print("config 2: %d of 128 greedy ids identical; prefill %.1f ms, decode %.1f ms (%.0f tok/s)"
          % (n_same, t_pre, t_dec, 127e3 / t_dec))
    with open(os.path.join(GOLDEN, "tiny_llama_c2_greedy.json")) as f:
        gold = json.load(f)
    assert list(prompt) == gold["prompt"]
    assert list(want[:32]) == gold["oracle_ids"][:32]
    assert list(ids[:32]) == gold["oracle_ids"][:32]
    m.close()


def test_lastblock_rope_quirk_switch(small):
    cfg, w = small
    prompt = np.array([5, 17, 99, 3, 64, 8], np.uint32)
    for quirk in (1, 0):
        m = M.Llama2(cfg, w)
        m.set_option("lastblock_rope_quirk", quirk)
        got = m.forward(prompt, 0)
        want = O.OracleModel(cfg, w, lastblock_rope_quirk=bool(quirk)).forward(prompt, 0)
        assert logit_err(got, want) < 1e-2
        m.close()


@pytest.mark.parametrize("fused", [0, 1, 2])
def test_fp16_weights_model(fused):
    """FP16 matrices: operator chain, and the fused decode step on its fp16
    weight path."""
    cfg = dict(SMALL, wtype=1, n_layers=2)
    w = M.synth_weights(cfg, seed=3)
    prompt = np.array([5, 17, 99], np.uint32)
    m = M.Llama2(cfg, w)
    set_path(m, fused)
    om = O.OracleModel(cfg, w)
    assert logit_err(m.forward(prompt, 0), om.forward(prompt, 0)) < 1e-2
    assert logit_err(m.forward([4], 3), om.forward([4], 3)) < 1e-2
    ids, _, _ = m.generate_greedy(prompt, 24)
    want, _ = O.OracleModel(cfg, w).generate_greedy(prompt, 24)
    assert list(ids) == list(want)
    m.close()


def test_decode_flag_areas_are_pooled(dev):
    """vkl_decode_flags_acquire / release: the flags that workgroups poll inside
    a launch live in device memory that no cache holds, which must never be
    freed; the library hands areas out of a pool, zeroed, and takes them back.
    A model holds one while it lives."""
    import ctypes as C
    from vkllama_amd import capi
    raw = C.CDLL(capi.HIP_LIB_PATH)
    raw.vkl_decode_flags_acquire.argtypes = [C.POINTER(C.c_void_p)]
    raw.vkl_decode_flags_acquire.restype = C.c_int
    raw.vkl_decode_flags_release.argtypes = [C.c_void_p]
    raw.vkl_decode_flags_release.restype = None
    a, b = C.c_void_p(), C.c_void_p()
    assert raw.vkl_decode_flags_acquire(C.byref(a)) == 0 and a.value
    assert raw.vkl_decode_flags_acquire(C.byref(b)) == 0 and b.value and b.value != a.value
    raw.vkl_decode_flags_release(a)
    cfg = dict(SMALL, n_layers=1)
    m = M.Llama2(cfg, M.synth_weights(cfg, seed=2))      # takes the area just handed back
    c = C.c_void_p()
    assert raw.vkl_decode_flags_acquire(C.byref(c)) == 0 and c.value not in (a.value, b.value)
    m.close()
    d = C.c_void_p()
    assert raw.vkl_decode_flags_acquire(C.byref(d)) == 0 and d.value == a.value   # the model's, back in the pool
    for q in (b, c, d):
        raw.vkl_decode_flags_release(q)
    raw.vkl_decode_flags_release(None)                    # a no-op
    assert raw.vkl_decode_flags_acquire(None) != 0


def test_operator_attention_option(small):
    """Option "operator_attention": the attention of a prompt pass as the
    reference's three operators (scores, masked softmax with probabilities
    rounded to fp16 one by one, P V; multiheadattention_v2.cpp:272-317)
    instead of the one-launch attention with its running maximum.  RoPE and
    cache rows do not depend on the form (bit-identical caches), both forms
    meet the oracle's logits, and the greedy ids are the oracle's either way."""
    cfg, w = small
    prompt = np.random.default_rng(3).integers(3, cfg["vocab"], 37).astype(np.uint32)
    om = O.OracleModel(cfg, w)
    want = om.forward(prompt, 0)
    a, b = M.Llama2(cfg, w), M.Llama2(cfg, w)
    b.set_option("operator_attention", 1)
    la, lb = a.forward(prompt, 0), b.forward(prompt, 0)
    assert logit_err(la, want) < 1e-2 and logit_err(lb, want) < 1e-2
    assert not np.array_equal(la, lb)                       # two forms, two roundings
    assert np.array_equal(a.read_kv_cache(0, 0), b.read_kv_cache(0, 0))
    assert np.array_equal(a.read_kv_cache(0, 1), b.read_kv_cache(0, 1))
    ids, _ = om.generate_greedy(prompt, 8)
    assert list(b.generate_greedy(prompt, 8)[0]) == list(ids)
    b.set_option("operator_attention", 0)
    assert np.array_equal(b.forward(prompt, 0), la)
    a.close(), b.close(), om.close()


def test_errors(small):
    cfg, w = small
    m = M.Llama2(cfg, w)
    with pytest.raises(capi.VklError, match=r"\(11\)"):      # OutOfRange
        m.forward([1, 2, 3], cfg["maxlen"] - 1)
    with pytest.raises(capi.VklError, match=r"\(11\)"):
        m.forward([1], cfg["maxlen"])
    with pytest.raises(capi.VklError, match=r"\(3\)"):       # InvalidArgument
        m.forward(np.zeros(0, np.uint32), 0)
    # ids past the vocabulary read row 0 (UNK), like the reference's embedding shader
    a = m.forward([cfg["vocab"] + 5], 0)
    m2 = M.Llama2(cfg, w)
    b = m2.forward([0], 0)
    assert np.array_equal(a, b)
    m.close(), m2.close()
    # a matrix with fewer bytes than its shape needs is rejected at load (OutOfRange)
    short = dict(w)
    short["blk.0.ffn_up.weight"] = w["blk.0.ffn_up.weight"][:-1]
    with pytest.raises(capi.VklError, match=r"\(11\)"):
        M.Llama2(cfg, short)


def test_blocks_of_different_type_never_reach_the_fused_step():
    """The fused decode kernels index every block with ONE dtype and ONE set of
    shapes.  A model whose second block holds FP16 matrices while the first
    holds Q8_0 (models/llama2.h:348-431 would load such a file) must be served
    by the operator chain: the decode plan reports no phases (it is not
    usable), and a decode step still equals the last row of a prompt pass."""
    cfg = dict(SMALL, n_layers=2)
    w = M.synth_weights(cfg, seed=17)
    w16 = M.synth_weights(dict(cfg, wtype=1), seed=17)
    mixed = dict(w)
    for name in w:
        if name.startswith("blk.1.") and not name.endswith("_norm.weight"):
            mixed[name] = w16[name]
    m = M.Llama2(cfg, mixed)
    assert m.phase_bytes("upgate", 8) == 0
    uniform = M.Llama2(cfg, w)
    assert uniform.phase_bytes("upgate", 8) > 0
    uniform.close()
    prompt = np.array([5, 17, 99, 3, 64], np.uint32)
    m.set_option("lastblock_rope_quirk", 0)
    m.forward(prompt[:4], 0)
    step = m.forward(prompt[4:], 4)
    full = m.forward(prompt, 0)
    assert np.isfinite(step).all()
    assert logit_err(step, full) < 1e-2
    m.close()


@pytest.mark.parametrize("cfg,seed", [(SMALL, 11), (SMALL128, 5), (TINY, 1234)])
def test_layer_launch_decode_matches_oracle(cfg, seed):
    """decode_mode 1: one launch per layer; the workgroups stay for the five
    phases, hand the activations over through memory and wait for one another.
    Ids identical to the oracle's, and logits bit-identical to the
    launch-per-phase step (both keep the same order of every sum)."""
    w = M.synth_weights(cfg, seed=seed)
    prompt = np.array([5, 17, 99, 3], np.uint32)
    m = M.Llama2(cfg, w)
    m.set_option("decode_mode", 1)
    m0 = M.Llama2(cfg, w)
    om = O.OracleModel(cfg, w)
    assert logit_err(m.forward(prompt, 0), om.forward(prompt, 0)) < 1e-2
    m0.forward(prompt, 0)
    got = m.forward([7], 4)
    assert logit_err(got, om.forward([7], 4)) < 1e-2
    assert np.array_equal(got, m0.forward([7], 4))
    want, _ = O.OracleModel(cfg, w).generate_greedy(prompt, 32)
    for graph in (1, 0):
        m.set_option("decode_graph", graph)
        ids, _, t_dec = m.generate_greedy(prompt, 32)
        assert list(ids) == list(want), graph
    assert m.decode_recoveries() == 0
    m.close(), m0.close()


@pytest.mark.parametrize("cfg", [dict(dim=4096, n_layers=2, n_heads=32, ffn=11008, vocab=1024, maxlen=256, eps=1e-5,
                                      wtype=8),
                                 dict(dim=5120, n_layers=1, n_heads=40, ffn=13824, vocab=640, maxlen=128, eps=1e-5,
                                      wtype=8),
                                 dict(dim=4096, n_layers=2, n_heads=32, ffn=11008, vocab=1024, maxlen=256, eps=1e-5,
                                      wtype=1),
                                 dict(dim=512, n_layers=3, n_heads=8, ffn=1376, vocab=2048, maxlen=128, eps=1e-5,
                                      wtype=1)])
def test_layer_launch_equals_phase_launches(cfg):
    """One launch per layer against one launch per phase at the row widths of
    the 7B and 13B shapes and with fp16 weights: greedy ids and the logits of a
    further step bit for bit, replayed from a graph and launched step by step
    (the launch-per-phase form is what the other tests hold against the
    oracle)."""
    w = M.synth_weights(cfg, seed=3)
    prompt = np.random.default_rng(3).integers(3, cfg["vocab"], 7).astype(np.uint32)
    m = M.Llama2(cfg, w)
    runs = {}
    for mode in (0, 1):
        m.set_option("decode_mode", mode)
        for graph in (1, 0):
            m.set_option("decode_graph", graph)
            ids, _, _ = m.generate_greedy(prompt, 40)
            logits = m.forward([int(ids[-1])], 7 + 39)
            runs[(mode, graph)] = (list(ids), logits.copy())
    assert m.decode_recoveries() == 0
    m.close()
    ref_ids, ref_logits = runs[(0, 0)]
    for key, (ids, logits) in runs.items():
        assert ids == ref_ids, key
        assert np.array_equal(logits.view(np.uint32), ref_logits.view(np.uint32)), key


def test_layer_launch_long_context_equals_phase_launches():
    """Above the split length mode 1 runs K/Q/V, the split attention and then
    Wo + up/gate + down in one launch; ids and logits bit for bit those of the
    launch-per-phase form, across the switch at the split length."""
    cfg = dict(dim=256, n_layers=2, n_heads=4, ffn=352, vocab=640, maxlen=160, eps=1e-5, wtype=8)
    w = M.synth_weights(cfg, seed=21)
    prompt = np.random.default_rng(21).integers(3, cfg["vocab"], 90).astype(np.uint32)
    m = M.Llama2(cfg, w)
    m.set_option("attn_split_min", 100)
    runs = {}
    for mode in (0, 1):
        m.set_option("decode_mode", mode)
        for graph in (1, 0):
            m.set_option("decode_graph", graph)
            ids, _, _ = m.generate_greedy(prompt, 30)
            logits = m.forward([int(ids[-1])], 90 + 29)
            runs[(mode, graph)] = (list(ids), logits.copy())
    assert m.decode_recoveries() == 0
    m.close()
    ref_ids, ref_logits = runs[(0, 0)]
    for key, (ids, logits) in runs.items():
        assert ids == ref_ids, key
        assert np.array_equal(logits.view(np.uint32), ref_logits.view(np.uint32)), key


@pytest.mark.parametrize("heads", [4, 2])
def test_long_context_decode_uses_split_attention(heads):
    """From 1024 positions on the decode step splits each head's context over
    several workgroups of one launch (the last to finish adds the parts); logits, greedy ids
    and the cache rows written on the way must still match the oracle."""
    cfg = dict(dim=256, n_layers=2, n_heads=heads, ffn=352, vocab=640, maxlen=1280, eps=1e-5, wtype=8)
    w = M.synth_weights(cfg, seed=21)
    rng = np.random.default_rng(21)
    prompt = rng.integers(3, cfg["vocab"], 1100).astype(np.uint32)
    m = M.Llama2(cfg, w)
    om = O.OracleModel(cfg, w)
    assert logit_err(m.forward(prompt, 0), om.forward(prompt, 0)) < 1e-2
    pos = len(prompt)
    for tok in (7, 300, 12, 5):
        got, want = m.forward([tok], pos), om.forward([tok], pos)
        assert logit_err(got, want) < 1e-2, pos
        assert int(np.argmax(got)) == int(np.argmax(want))
        pos += 1
    for layer in range(cfg["n_layers"]):
        for value in (0, 1):
            g = m.read_kv_cache(layer, value)[:, 1100:pos].astype(np.float32)
            o = (om.vcache(layer) if value else om.kcache(layer))[:, 1100:pos].astype(np.float32)
            assert np.abs(g - o).max() <= 1e-2 * max(np.abs(o).max(), 1e-3), (layer, value)
    m.close()


@pytest.mark.parametrize("n_prompt,n_gen", [(4, 40), (1016, 24), (1100, 24)])
def test_graph_replayed_loop_equals_stepwise_and_oracle(n_prompt, n_gen):
    """generate_greedy replays one captured step per token (token index and
    position advance in device memory); the ids must equal those of the
    step-by-step launches and the oracle's, also across the switch of the
    attention phase to its split form at 1024 positions, and on a second use
    of the cached graphs."""
    cfg = dict(dim=256, n_layers=2, n_heads=4, ffn=352, vocab=640, maxlen=1280, eps=1e-5, wtype=8)
    w = M.synth_weights(cfg, seed=33)
    rng = np.random.default_rng(33)
    prompt = rng.integers(3, cfg["vocab"], n_prompt).astype(np.uint32)
    want, _ = O.OracleModel(cfg, w).generate_greedy(prompt, n_gen)
    m = M.Llama2(cfg, w)
    for graph in (1, 0, 1):
        m.set_option("decode_graph", graph)
        ids, _, _ = m.generate_greedy(prompt, n_gen)
        assert list(ids) == list(want), graph
        # eager work between replays: a plain forward pass
        m.forward(prompt[:3], 0)
    m.close()


@pytest.mark.parametrize("cfg", [TINY, dict(dim=5120, n_layers=2, n_heads=40, ffn=1376, vocab=1024, maxlen=256, eps=1e-5,
                                              wtype=8),
                                 dict(dim=4096, n_layers=2, n_heads=32, ffn=1376, vocab=1024, maxlen=256, eps=1e-5,
                                      wtype=1)])
def test_attention_and_wo_in_one_launch_equals_two_launches(cfg):
    """Below the split length the decode step runs the attention phase and the
    Wo projection in one launch (option "fuse_attn_wo", on by default): the
    projection's workgroups wait inside the launch for the heads.  Ids and
    logits must equal those of the two separate launches bit for bit, replayed
    from a graph and launched step by step (the two-launch form is what the
    other tests of this file hold against the oracle)."""
    w = M.synth_weights(cfg, seed=5)
    prompt = np.random.default_rng(5).integers(3, cfg["vocab"], 9).astype(np.uint32)
    m = M.Llama2(cfg, w)
    runs = {}
    for fuse in (1, 0):
        m.set_option("fuse_attn_wo", fuse)
        for graph in (1, 0):
            m.set_option("decode_graph", graph)
            ids, _, _ = m.generate_greedy(prompt, 48)
            logits = m.forward([int(ids[-1])], 9 + 47)
            runs[(fuse, graph)] = (list(ids), logits.copy())
    m.set_option("fuse_attn_wo", 1)
    m.close()
    ref_ids, ref_logits = runs[(0, 0)]
    for key, (ids, logits) in runs.items():
        assert ids == ref_ids, key
        assert np.array_equal(logits.view(np.uint32), ref_logits.view(np.uint32)), key


@pytest.mark.parametrize("mode", [0, 1])
def test_wait_inside_a_launch_is_bounded_and_recovered(mode):
    """Workgroups that wait for others inside a launch (the Wo projection for
    the attention heads, in the attention + Wo launch of mode 0 and in the
    one-launch layer of mode 1) poll a bounded number of times.  With the heads
    kept silent from the host (option "wait_test": the flags stay unset, 4
    polls) every such wait gives up: all launches still end, the workgroups
    concerned store nothing, the status word reports it, and the model repeats
    the work on the launches that wait for nothing.  The ids are those of an
    undisturbed run, and the repeat is counted."""
    cfg = TINY
    w = M.synth_weights(cfg, seed=9)
    prompt = np.random.default_rng(9).integers(3, cfg["vocab"], 6).astype(np.uint32)
    m = M.Llama2(cfg, w)
    m.set_option("decode_mode", mode)
    want, _, _ = m.generate_greedy(prompt, 24)
    want_logits = m.forward([int(want[0])], 6)
    assert m.decode_recoveries() == 0
    n = 0
    try:
        for graph in (0, 1):
            m.set_option("decode_mode", mode), m.set_option("fuse_attn_wo", 1)
            m.set_option("wait_test", 4)
            m.set_option("decode_graph", graph)
            ids, _, _ = m.generate_greedy(prompt, 24)
            n += 1
            assert m.decode_recoveries() == n
            assert list(ids) == list(want)
        m.set_option("decode_mode", mode), m.set_option("fuse_attn_wo", 1)
        got = m.forward([int(want[0])], 6)
        assert m.decode_recoveries() == n + 1
        assert np.array_equal(got, want_logits)
    finally:
        m.set_option("wait_test", 0)
    m.set_option("decode_mode", mode), m.set_option("fuse_attn_wo", 1)
    for graph in (1, 0):
        m.set_option("decode_graph", graph)
        ids, _, _ = m.generate_greedy(prompt, 24)
        assert list(ids) == list(want)
    assert m.decode_recoveries() == n + 1
    m.close()


@pytest.mark.parametrize("fused", [0, 1, 2])
def test_sampled_generation_on_the_device(small, fused):
    """generate_sampled: k = 1 is the greedy sequence; a seed reproduces a top-k
    sequence; every drawn token is one of the k most likely tokens of the
    oracle's logits for the sequence so far (the candidate rule of
    models/samplers.cpp:37-64), and top-p stays inside its candidate set."""
    cfg, w = small
    prompt = np.array([5, 17, 99, 3], np.uint32)
    m = M.Llama2(cfg, w)
    set_path(m, fused)
    greedy, _, _ = m.generate_greedy(prompt, 12)
    top1, _, _ = m.generate_sampled(prompt, 12, topk=1, seed=3)
    assert list(top1) == list(greedy)
    a, _, _ = m.generate_sampled(prompt, 16, topk=8, seed=7)
    b, _, _ = m.generate_sampled(prompt, 16, topk=8, seed=7)
    c, _, _ = m.generate_sampled(prompt, 16, topk=8, seed=8)
    assert list(a) == list(b) and list(a) != list(c) and list(a) != list(greedy[:1]) * 16
    # the loop replayed from a captured graph (the draw is the last launch of
    # every step, k / p / seed in device memory) and launched step by step
    # with the sampler called from the host draw the same tokens
    m.set_option("decode_graph", 0)
    for kw in (dict(topk=8, seed=7), dict(topk=3, seed=11), dict(topp=0.6, seed=5)):
        m.set_option("decode_graph", 1)
        replayed, _, _ = m.generate_sampled(prompt, 16, **kw)
        m.set_option("decode_graph", 0)
        stepwise, _, _ = m.generate_sampled(prompt, 16, **kw)
        assert list(replayed) == list(stepwise), kw
    m.set_option("decode_graph", 1)
    assert list(m.generate_sampled(prompt, 16, topk=8, seed=7)[0]) == list(a)
    om = O.OracleModel(cfg, w)
    logits = om.forward(prompt, 0)
    pos = len(prompt)
    for t in a:
        order = np.lexsort((np.arange(logits.size), -logits.astype(np.float64)))
        # a logit within fp16 rounding of the k-th may swap places with it
        assert int(t) in order[:8] or logits[t] >= logits[order[7]] - 2e-2 * abs(logits[order[7]])
        logits = om.forward([int(t)], pos)
        pos += 1
    om.close()
    d, _, _ = m.generate_sampled(prompt, 8, topp=0.0, seed=1)     # p = 0 keeps the top token only
    assert list(d) == list(greedy[:8])
    with pytest.raises(RuntimeError):
        m.generate_sampled(prompt, 4, topk=0)
    m.close()
