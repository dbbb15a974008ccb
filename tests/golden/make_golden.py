"""Writes the committed fixtures under tests/golden/ from the CPU oracle.

Run from the repository root: python tests/golden/make_golden.py
(and once more with --llama2-7b for the fixture of the 7B-shape workload).
The reference ships no golden vectors for this path (its tests draw unseeded
random inputs), so the fixtures hold the oracle's outputs on seeded synthetic
inputs; tests/test_golden.py checks both the oracle (CPU) and the HIP kernels
(GPU) against them.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import oracle as O  # noqa: E402
from util import q8_weights  # noqa: E402
from vkllama_amd import model as M  # noqa: E402

TINY = dict(dim=512, n_layers=8, n_heads=8, ffn=1376, vocab=32000, maxlen=512, eps=1e-5, wtype=8)


def tiny_llama():
    w = M.synth_weights(TINY, seed=1234)
    rng = np.random.default_rng(1234)
    prompt = rng.integers(3, 32000, 16).astype(np.uint32)
    om = O.OracleModel(TINY, w)
    ids, first = om.generate_greedy(prompt, 128)
    top = np.argsort(-first, kind="stable")[:8]
    out = {
        "config": TINY, "weight_seed": 1234, "prompt": [int(t) for t in prompt],
        "oracle_ids": [int(t) for t in ids],
        "first_logits_top8_idx": [int(i) for i in top],
        "first_logits_top8_val": [float(first[i]) for i in top],
    }
    with open(os.path.join(HERE, "tiny_llama_c2_greedy.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("tiny llama ids:", out["oracle_ids"][:16], "...")


# benchmark configuration 3: the Llama-2-7B shape with Q8_0 weights
LLAMA7B = dict(dim=4096, n_layers=32, n_heads=32, ffn=11008, vocab=32000, maxlen=4096, eps=1e-5, wtype=8)


def llama2_7b():
    """The first 32 greedy ids of the oracle on the 7B-shape workload of
    bench.py (weights of seed 1234, the 32 prompt ids of the same seed).
    About 7 GB of weights and a minute of CPU time."""
    w = M.synth_weights(LLAMA7B, seed=1234)
    rng = np.random.default_rng(1234)
    prompt = rng.integers(3, 32000, 32).astype(np.uint32)
    om = O.OracleModel(LLAMA7B, w)
    ids, first = om.generate_greedy(prompt, 32)
    top = np.argsort(-first, kind="stable")[:8]
    out = {
        "config": LLAMA7B, "weight_seed": 1234, "prompt": [int(t) for t in prompt],
        "oracle_ids": [int(t) for t in ids],
        "first_logits_top8_idx": [int(i) for i in top],
        "first_logits_top8_val": [float(first[i]) for i in top],
    }
    with open(os.path.join(HERE, "llama2_7b_q8_0_c3_greedy.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("7B ids:", out["oracle_ids"])


def ops():
    rng = np.random.default_rng(2024)
    d = {}
    N, K, M_ = 48, 256, 2
    raw, _ = q8_weights(rng, N, K)
    x = rng.standard_normal((M_, K)).astype(np.float16)
    d["q8_w"], d["q8_x"] = raw, x
    d["q8_y"] = O.matmul_q8_0(x, raw, K)
    raw2, _ = q8_weights(rng, N, K)
    raw3, _ = q8_weights(rng, N, K)
    d["q8_w2"], d["q8_w3"] = raw2, raw3
    k, q, v = O.kqv_q8_0(x, raw, raw2, raw3, K)
    d["kqv_k"], d["kqv_q"], d["kqv_v"] = k, q, v
    d["upgate"] = O.ffn_upgate_q8_0(x, raw, raw2, K)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    d["norm_w"] = w
    d["norm_y"] = O.rmsnorm(x, w, 1e-5)
    fc, fs = O.rope_tables(64, 64)
    r = rng.standard_normal((4, 3, 64)).astype(np.float16)
    d["rope_x"], d["rope_y"] = r, O.rope(r, fc, fs, 17)
    s = (rng.standard_normal((4, 3, 20)) * 2).astype(np.float16)
    d["softmax_x"], d["softmax_y"] = s, O.softmax(s, True, 17)
    a = rng.standard_normal((4, 3, 64)).astype(np.float16)
    b = rng.standard_normal((4, 20, 64)).astype(np.float16)
    d["tb_a"], d["tb_b"], d["tb_y"] = a, b, O.matmul_f16_tb(a, b, scale=0.125)
    p = rng.uniform(0, 0.2, (4, 3, 20)).astype(np.float16)
    d["nn_a"], d["nn_y"] = p, O.matmul_f16_nn(p, b)
    xq = rng.uniform(-5, 5, (3, 95)).astype(np.float32)
    d["quant_x"], d["quant_y"] = xq, O.quantize_q8_0(xq, 2)
    toks = np.array([0, 47, 7, 48, 2 ** 31], np.uint32)
    d["embed_toks"], d["embed_y"] = toks, O.embedding_q8_0(raw, K, toks, 0)
    np.savez_compressed(os.path.join(HERE, "ops_golden.npz"), **d)
    print("ops fixture:", sum(v.nbytes for v in d.values()), "bytes raw")


ORDERS = (0, 1, 2, 3, 4)


def llama2_7b_lane_orders():
    """How far the reference's own freedom moves the 7B-shape workload: its
    shaders add the 32 lanes of a subgroup with subgroupAdd, whose order
    Vulkan leaves open.  The committed sequence (oracle order 0) is fed, token
    by token, to the oracle in each of its lane orders; per step the
    fixture keeps the order-0 margin between the first and the second choice,
    every order's arg-max and its largest logit deviation from order 0.
    Five passes over 7 GB of weights: some minutes of CPU time."""
    w = M.synth_weights(LLAMA7B, seed=1234)
    with open(os.path.join(HERE, "llama2_7b_q8_0_c3_greedy.json")) as f:
        gold = json.load(f)
    prompt = np.array(gold["prompt"], np.uint32)
    ids = gold["oracle_ids"]
    logits = {}
    for order in ORDERS:
        O.set_lane_order(order)
        om = O.OracleModel(LLAMA7B, w)
        rows = [om.forward(prompt, 0).copy()]
        for i in range(31):
            rows.append(om.forward([ids[i]], 32 + i).copy())
        om.close()
        logits[order] = np.stack(rows)
        print("order", order, "arg-max:", [int(np.argmax(r)) for r in rows])
    O.set_lane_order(0)
    ref = logits[0]
    assert [int(np.argmax(r)) for r in ref] == ids
    srt = np.sort(ref, axis=1)
    out = {
        "config": LLAMA7B, "weight_seed": 1234, "prompt": gold["prompt"], "fed_ids": ids,
        "lane_orders": {"0": "pairwise halving (the oracle's default)", "1": "sequential", "2": "neighbours first",
                        "3": "sequential from the last lane", "4": "groups of eight, then the groups"},
        "max_logit": [float(np.abs(r).max()) for r in ref],
        "margin_order0": [float(srt[i, -1] - srt[i, -2]) for i in range(32)],
        "second_choice_order0": [int(np.argsort(-ref[i], kind="stable")[1]) for i in range(32)],
        "argmax": {str(o): [int(np.argmax(r)) for r in logits[o]] for o in ORDERS},
        "max_abs_dev_from_order0": {str(o): [float(np.abs(logits[o][i] - ref[i]).max()) for i in range(32)]
                                    for o in ORDERS[1:]},
    }
    with open(os.path.join(HERE, "llama2_7b_q8_0_c3_lane_orders.json"), "w") as f:
        json.dump(out, f, indent=1)
    for o in ORDERS[1:]:
        diff = [i for i in range(32) if out["argmax"][str(o)][i] != ids[i]]
        print("order %d differs from order 0 at steps %s; margins there %s" % (
            o, diff, [out["margin_order0"][i] for i in diff]))


if __name__ == "__main__":
    if "--llama2-7b-lane-orders" in sys.argv:
        llama2_7b_lane_orders()
    elif "--llama2-7b" in sys.argv:
        llama2_7b()
    else:
        ops()
        tiny_llama()
