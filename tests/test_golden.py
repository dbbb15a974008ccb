"""Committed fixtures under tests/golden/ (written by tests/golden/make_golden.py
from the CPU oracle on seeded inputs; the reference ships no golden vectors for
this path) checked from both sides:

* CPU: the oracle still reproduces them bit for bit (guards against drift of
  the oracle itself);
* GPU: the HIP kernels, through the C ABI, meet the parity bars on them
  (bit-exact for quantisation / embedding / RoPE, 1e-2 relative for fp16
  outputs of dot-product kernels).
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from util import rel_err, ulp_diff_f16
from vkllama_amd import capi

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
K = 256


@pytest.fixture(scope="module")
def g():
    with np.load(os.path.join(GOLDEN, "ops_golden.npz"), allow_pickle=False) as d:
        return {k: d[k] for k in d.files}


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


# ------------------------------------------------------------------ CPU -----
def test_oracle_reproduces_op_fixtures(g):
    assert np.array_equal(bits(O.matmul_q8_0(g["q8_x"], g["q8_w"], K)), bits(g["q8_y"]))
    k, q, v = O.kqv_q8_0(g["q8_x"], g["q8_w"], g["q8_w2"], g["q8_w3"], K)
    assert np.array_equal(bits(k), bits(g["kqv_k"]))
    assert np.array_equal(bits(q), bits(g["kqv_q"]))
    assert np.array_equal(bits(v), bits(g["kqv_v"]))
    assert np.array_equal(bits(O.ffn_upgate_q8_0(g["q8_x"], g["q8_w"], g["q8_w2"], K)), bits(g["upgate"]))
    assert np.array_equal(bits(O.rmsnorm(g["q8_x"], g["norm_w"], 1e-5)), bits(g["norm_y"]))
    fc, fs = O.rope_tables(64, 64)
    assert np.array_equal(bits(O.rope(g["rope_x"], fc, fs, 17)), bits(g["rope_y"]))
    assert np.array_equal(bits(O.softmax(g["softmax_x"], True, 17)), bits(g["softmax_y"]))
    assert np.array_equal(bits(O.matmul_f16_tb(g["tb_a"], g["tb_b"], scale=0.125)), bits(g["tb_y"]))
    assert np.array_equal(bits(O.matmul_f16_nn(g["nn_a"], g["tb_b"])), bits(g["nn_y"]))
    assert np.array_equal(O.quantize_q8_0(g["quant_x"], 2), g["quant_y"])
    assert np.array_equal(bits(O.embedding_q8_0(g["q8_w"], K, g["embed_toks"], 0)), bits(g["embed_y"]))


def test_lane_order_fixture_shows_the_references_own_freedom():
    """tests/golden/llama2_7b_q8_0_c3_lane_orders.json (written by
    make_golden.py --llama2-7b-lane-orders): the committed 7B-shape sequence
    fed to the oracle in five legal orders of the reference's subgroupAdd.

    What it pins: (1) legal orders move the logits of this workload by as much
    as the GPU's order of sums does (0.03 and more, 0.7 % of the largest
    logit); (2) they flip the arg-max of a step whose order-0 margin is two
    fp16 steps, so the ids of this random-init workload are not a property of
    the reference but of one of its implementations; (3) every such flip obeys
    the near-tie rule the GPU tests use (margin <= 2 x the largest deviation);
    (4) the step at which the GPU's own sequence leaves the committed one
    (generated token 7, index 6) is the narrowest near-tie of the 32: one fp16
    step, an eighth of the deviation between legal orders at that step."""
    with open(os.path.join(GOLDEN, "llama2_7b_q8_0_c3_lane_orders.json")) as f:
        d = json.load(f)
    with open(os.path.join(GOLDEN, "llama2_7b_q8_0_c3_greedy.json")) as f:
        gold = json.load(f)
    assert d["fed_ids"] == gold["oracle_ids"] and d["argmax"]["0"] == gold["oracle_ids"]
    margin = np.array(d["margin_order0"])
    orders = sorted(k for k in d["argmax"] if k != "0")
    assert len(orders) >= 4
    flips = 0
    for o in orders:
        dev = np.array(d["max_abs_dev_from_order0"][o])
        assert dev.max() >= 0.03 and dev.max() / min(d["max_logit"]) < 1e-2      # (1), and inside the 1e-2 bar
        for i in range(32):
            if d["argmax"][o][i] != d["argmax"]["0"][i]:
                flips += 1
                assert margin[i] <= 2.0 * dev[i]                                   # (3)
                assert margin[i] >= 0.0078                                         # (2): two fp16 steps at 4..8
    assert flips >= 1                                                              # (2)
    assert int(np.argmin(margin)) == 6 and margin[6] <= 0.0040                     # (4)
    assert min(d["max_abs_dev_from_order0"][o][6] for o in orders) >= 6 * margin[6]


def test_op_fixtures_against_float64(g):
    """The fixtures themselves are sane: the stored outputs agree with a float64
    evaluation of the textbook formulas to fp16 accuracy."""
    deq = O.dequantize_q8_0(g["q8_w"], K, 2).astype(np.float64)
    x = g["q8_x"].astype(np.float64)
    assert rel_err(g["q8_y"], x @ deq.T) < 2e-3
    up, gate = x @ deq.T, x @ O.dequantize_q8_0(g["q8_w2"], K, 2).astype(np.float64).T
    assert rel_err(g["upgate"], gate / (1 + np.exp(-gate)) * up) < 4e-3
    rms = np.sqrt((x * x).mean(-1, keepdims=True) + 1e-5)
    assert rel_err(g["norm_y"], x / rms * g["norm_w"]) < 2e-3
    a, b = g["tb_a"].astype(np.float64), g["tb_b"].astype(np.float64)
    assert rel_err(g["tb_y"], 0.125 * np.einsum("cmk,cnk->cmn", a, b)) < 2e-3
    assert rel_err(g["nn_y"], np.einsum("cmk,ckn->cmn", g["nn_a"].astype(np.float64), b)) < 2e-3
    s = g["softmax_y"].astype(np.float64)
    assert np.allclose(s.sum(-1), 1.0, atol=4e-3)


def test_tiny_llama_fixture_is_consistent():
    with open(os.path.join(GOLDEN, "tiny_llama_c2_greedy.json")) as f:
        gold = json.load(f)
    assert len(gold["prompt"]) == 16 and len(gold["oracle_ids"]) == 128
    assert gold["config"]["dim"] == 512 and gold["config"]["vocab"] == 32000
    assert all(3 <= t < 32000 for t in gold["prompt"])
    # the first generated id is the arg-max of the stored first-step logits
    assert gold["oracle_ids"][0] == gold["first_logits_top8_idx"][0]
    v = gold["first_logits_top8_val"]
    assert all(v[i] >= v[i + 1] for i in range(7))


# ------------------------------------------------------------------ GPU -----
def _f16(buf, shape):
    return buf.read(np.uint16, shape).view(np.float16)


@pytest.mark.gpu
def test_hip_q8_kernels_on_fixtures(dev, g):
    L = capi.lib()
    x, M, N = g["q8_x"], 2, 48
    dx = dev.upload(x)
    dw = [dev.upload_q8_0(g[k], N, K) for k in ("q8_w", "q8_w2", "q8_w3")]
    dy = dev.alloc(M * N * 2)
    capi.check(L.vkl_matmul_q8_0(dx.ptr, dw[0].ptr, M, N, K, K, N, 1.0, 0.0, 0, None, dy.ptr, None, dev.stream))
    got = _f16(dy, (M, N))
    assert ulp_diff_f16(got, g["q8_y"]).max() <= 1 and rel_err(got, g["q8_y"]) < 1e-2
    outs = [dev.alloc(M * N * 2) for _ in range(3)]
    capi.check(L.vkl_kqv_q8_0(dx.ptr, dw[0].ptr, dw[1].ptr, dw[2].ptr, M, N, K, outs[0].ptr, outs[1].ptr,
                              outs[2].ptr, dev.stream))
    for o, name in zip(outs, ("kqv_k", "kqv_q", "kqv_v")):
        assert rel_err(_f16(o, (M, N)), g[name]) < 1e-2
    capi.check(L.vkl_ffn_upgate_q8_0(dx.ptr, dw[0].ptr, dw[1].ptr, M, N, K, dy.ptr, dev.stream))
    assert rel_err(_f16(dy, (M, N)), g["upgate"]) < 1e-2
    toks = g["embed_toks"]
    dt = dev.upload(toks)
    de = dev.alloc(toks.size * K * 2)
    capi.check(L.vkl_embed_q8_0(dw[0].ptr, N, K, dt.ptr, toks.size, 0, de.ptr, dev.stream))
    assert np.array_equal(bits(_f16(de, (toks.size, K))), bits(g["embed_y"]))


@pytest.mark.gpu
def test_hip_small_ops_on_fixtures(dev, g):
    L = capi.lib()
    x = g["q8_x"]
    dx, dw = dev.upload(x), dev.upload(g["norm_w"])
    dy = dev.alloc(x.nbytes)
    capi.check(L.vkl_rmsnorm_f16(dx.ptr, dw.ptr, 2, K, 1e-5, dy.ptr, dev.stream))
    assert ulp_diff_f16(_f16(dy, x.shape), g["norm_y"]).max() <= 1
    fc, fs = O.rope_tables(64, 64)
    dr, dfc, dfs = dev.upload(g["rope_x"]), dev.upload(fc), dev.upload(fs)
    capi.check(L.vkl_rope_f16(dr.ptr, 4, 3, 64, dfc.ptr, dfs.ptr, 17, dev.stream))
    assert np.array_equal(bits(_f16(dr, (4, 3, 64))), bits(g["rope_y"]))
    s = g["softmax_x"]
    ds, do = dev.upload(s), dev.alloc(s.nbytes)
    capi.check(L.vkl_softmax_f16(ds.ptr, 4, 3, 20, 1, 17, do.ptr, dev.stream))
    got = _f16(do, s.shape)
    assert np.array_equal(got == 0, g["softmax_y"] == 0)
    assert rel_err(got, g["softmax_y"]) < 1e-2
    a, b = g["tb_a"], g["tb_b"]
    da, db, dy = dev.upload(a), dev.upload(b), dev.alloc(4 * 3 * 20 * 2)
    capi.check(L.vkl_matmul_f16_tb(da.ptr, db.ptr, 4, 3, 20, 64, 3 * 64, 64, 20 * 64, 64, 3 * 20, 20, 0.125, 0.0, 0,
                                   None, dy.ptr, None, dev.stream))
    assert rel_err(_f16(dy, (4, 3, 20)), g["tb_y"]) < 1e-2
    dp, dy = dev.upload(g["nn_a"]), dev.alloc(4 * 3 * 64 * 2)
    capi.check(L.vkl_matmul_f16_nn(dp.ptr, db.ptr, 4, 3, 64, 20, 3 * 20, 20, 20 * 64, 64, 3 * 64, 64, 1.0, 0.0, 0,
                                   dy.ptr, dev.stream))
    assert rel_err(_f16(dy, (4, 3, 64)), g["nn_y"]) < 1e-2


def test_host_quantizer_on_fixture(g):
    xq = g["quant_x"]
    lib = capi.lib()
    for r in range(xq.shape[0]):
        row = np.ascontiguousarray(xq[r])
        out = np.empty(lib.vkl_q8_0_row_bytes(row.size), np.uint8)
        lib.vkl_quantize_q8_0_h(row.ctypes.data, row.size, out.ctypes.data)
        assert np.array_equal(out, g["quant_y"][r])
