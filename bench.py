#!/usr/bin/env python3
"""Benchmark of the llama2 token loop on one MI355X.

A step is one batch-1 greedy decode token.  The default workload is benchmark
config 3: Llama-2-7B shape (dim 4096, 32 layers, 32 heads, FFN 11008, vocab
32000, context 4096), random-init N(0, 0.02) weights quantised to Q8_0, fp16
activations and KV cache, a 32-token random-id prompt, then K greedy decode
tokens (K = 256 by default, contexts 33 .. 32+K).

Prints ONE JSON line.  `value` is decode tokens per second with weights and
KV cache resident in HBM, timed across the K steps between device
synchronisations, including the on-device arg-max and the token hand-over.
`roofline` covers the dominant kernel of the step (the phase kernel with the
largest share of the step time, in practice the fused up/gate projection):
algorithmic bytes of one launch divided by the average launch duration, which
is measured with HIP event pairs on the launch stream in a second pass over
the same K steps (the events would perturb the throughput pass).  The same
object also carries the whole step priced the same way (`step_*`).
`cpu_baseline` is the CPU oracle timed on this box's host cores on a bounded
sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # the four model-level benchmark configurations
    "llama2-tiny-q8_0": dict(dim=512, n_layers=8, n_heads=8, ffn=1376, vocab=32000, maxlen=512, eps=1e-5, wtype=8,
                             prompt=16, prefill_kv=0),
    "llama2-7b-q8_0": dict(dim=4096, n_layers=32, n_heads=32, ffn=11008, vocab=32000, maxlen=4096, eps=1e-5,
                           wtype=8, prompt=32, prefill_kv=0),
    # FP16 weights, 2048-token prompt
    "llama2-7b-f16": dict(dim=4096, n_layers=32, n_heads=32, ffn=11008, vocab=32000, maxlen=4096, eps=1e-5,
                          wtype=1, prompt=2048, prefill_kv=0),
    "llama2-13b-q8_0-ctx3968": dict(dim=5120, n_layers=40, n_heads=40, ffn=13824, vocab=32000, maxlen=4096,
                                    eps=1e-5, wtype=8, prompt=3968, prefill_kv=1),
}
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of a kernel from hardware counters (FETCH_SIZE +
# WRITE_SIZE, calibrated against a copy kernel), keyed by (workload, phase);
# filled in from the counter runs whose summaries are kept under profiles/
TRAFFIC = {("llama2-7b-q8_0", "upgate"): (96197201, "profiles/decode_phase_kernels_llama2-7b-q8_0_hbm_traffic.txt"),
           ("llama2-7b-q8_0", "layer"): (218700083, "profiles/decode_layer_kernel_llama2-7b-q8_0_hbm_traffic.txt")}


def cpu_baseline(cfg, weights, n_tokens, gpu_model=None, n_parity=16):
    """The CPU oracle (a plain-C restatement of the reference's arithmetic,
    OpenMP over output rows) decoding n_tokens after a 4-token prompt.  With a
    GPU model of the same weights the first n_parity steps are also run on the
    GPU, on the oracle's own token sequence, and compared: largest deviation of
    a logit relative to the largest logit, and how often the arg-max agrees."""
    from oracle import oracle as O
    om = O.OracleModel(cfg, weights)
    head = np.array([5, 17, 99, 3], np.uint32)
    om.forward(head, 0)
    parity = None
    if gpu_model is not None:
        gpu_model.forward(head, 0)
        parity = {"against": "the CPU oracle on the same weights, step by step on the oracle's own ids",
                  "steps": 0, "argmax_equal": 0, "max_rel_logit_err": 0.0,
                  "largest_oracle_margin_where_argmax_differs": 0.0,
                  "rule": "near-tie rule: every logit within 1e-2 of the largest logit, and the oracle's arg-max "
                          "unless the oracle's margin over the GPU's choice is at most 2x the largest absolute "
                          "deviation of a logit in that step",
                  "rule_holds": True}
    tok, pos = 7, 4
    dt = 0.0
    for i in range(n_tokens):
        t0 = time.perf_counter()
        logits = om.forward([tok], pos)
        dt += time.perf_counter() - t0
        if parity is not None and i < n_parity:
            got = gpu_model.forward([tok], pos)
            parity["steps"] += 1
            parity["max_rel_logit_err"] = max(parity["max_rel_logit_err"],
                                              float(np.abs(got - logits).max() / np.abs(logits).max()))
            g, o = int(np.argmax(got)), int(np.argmax(logits))
            parity["argmax_equal"] += int(g == o)
            dev_abs = float(np.abs(got - logits).max())
            if dev_abs > 1e-2 * float(np.abs(logits).max()) or float(logits[o] - logits[g]) > 2.0 * dev_abs:
                parity["rule_holds"] = False
            if g != o:
                parity["largest_oracle_margin_where_argmax_differs"] = max(
                    parity["largest_oracle_margin_where_argmax_differs"], float(logits[o] - logits[g]))
        tok = int(np.argmax(logits))
        pos += 1
    om.close()
    if parity is not None:
        parity["max_rel_logit_err"] = round(parity["max_rel_logit_err"], 5)
    return n_tokens / dt, dt, parity


def bench_single_matmul(args):
    """Benchmark configuration 1: y[1,4096] = x[1,4096] W[4096,4096]^T with W in Q8_0 (int8 uniform in
    [-127,127], fp16 scales U(0.001,0.01)), x ~ N(0,1) fp16, through vkl_matmul_q8_0.  A step is one call.  The
    HBM figure cycles through a ring of 32 distinct matrices (571 MB, more than every cache); the same call on
    one matrix over and over is reported beside it as the cache-resident figure."""
    import ctypes as C
    from vkllama_amd import capi
    from oracle import oracle as O
    N = K = 4096
    ring, steps, warmup = 32, args.steps, args.warmup
    rng = np.random.default_rng(args.seed)
    dev = capi.Device(0)
    L = capi.lib()
    x = rng.standard_normal((1, K)).astype(np.float16)
    dx, dy = dev.upload(x), dev.alloc(N * 2)
    raws, mats = [], []
    for i in range(ring):
        raw = np.zeros((N, K // 32, 34), np.uint8)
        raw[:, :, 2:] = rng.integers(-127, 128, (N, K // 32, 32)).astype(np.int8).view(np.uint8)
        raw[:, :, 0:2] = rng.uniform(0.001, 0.01, (N, K // 32)).astype(np.float16).view(np.uint8).reshape(N, K // 32, 2)
        if i == 0:
            raws.append(raw)
        mats.append(dev.upload_q8_0(raw, N, K))

    def run(n, same):
        for i in range(n):
            w = mats[0 if same else i % ring]
            capi.check(L.vkl_matmul_q8_0(dx.ptr, w.ptr, 1, N, K, K, N, C.c_float(1.0), C.c_float(0.0), 0, None,
                                         dy.ptr, None, dev.stream), "vkl_matmul_q8_0")

    def timed(n, same):
        run(warmup, same)
        dev.sync()
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        run(n, same)
        dev.record(e1)
        return dev.elapsed_ms(e0, e1) / n

    ms = timed(steps, False)
    ms_hot = timed(steps, True)
    run(1, True)
    got = dy.read(np.float16, (1, N))
    want = O.matmul_q8_0(x, raws[0].reshape(N, -1), K)
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))
                       / np.maximum(np.abs(want.astype(np.float64)), 1e-2 * np.abs(want).max())))
    nbytes = N * (K // 32) * 34 + K * 2 + N * 2           # 17,842,176
    t0 = time.perf_counter()
    n_cpu = 200
    for _ in range(n_cpu):
        O.matmul_q8_0(x, raws[0].reshape(N, -1), K)
    cpu_calls = n_cpu / (time.perf_counter() - t0)
    gbs = nbytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "q8_0_matmul_4096x4096_bs1_calls_per_second", "value": round(1e3 / ms, 1), "unit": "calls/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "q8_0 weights x f16 activations, f32 accumulate",
        "data": "synthetic: int8 U[-127,127], fp16 scales U(0.001,0.01), x N(0,1); ring of %d matrices" % ring,
        "config": {"workload": args.workload, "M": 1, "N": N, "K": K, "ring": ring},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "decode_phase_direct_kernel<7, 8, %d, false> (the decode step's weight-streaming kernel, stand-alone)" % min(4, (K + 4095) // 4096),
                     "avg_launch_us": round(ms * 1e3, 3), "launches_timed": steps, "bytes_per_launch": nbytes,
                     "cache_resident_avg_launch_us": round(ms_hot * 1e3, 3),
                     "cache_resident_gbs": round(nbytes / (ms_hot * 1e-3) / 1e9, 1)},
        "max_rel_err_vs_oracle": err,
        "cpu_baseline": {"value": round(cpu_calls, 1), "unit": "calls/s",
                         "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count())), "kind": "port",
                         "sample": "%d calls of the oracle's matmul on the first matrix" % n_cpu}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="llama2-7b-q8_0", choices=sorted(WORKLOADS) + ["matmul-q8_0-4096"])
    ap.add_argument("--decode-mode", type=int, default=-1, choices=(-1, 0, 1),
                    help="1: one launch per layer (contexts below the split-attention length), 0: one launch per phase, "
                         "-1: the library's default for the model's shape")
    ap.add_argument("--decode-graph", type=int, default=1, choices=(0, 1),
                    help="1: the decode loop is replayed from a captured HIP graph; 0: the same launches step by step "
                         "(for runs under a kernel tracer, which does not survive graph launches here)")
    ap.add_argument("--cpu-tokens", type=int, default=-1, help="decode tokens of the CPU baseline (0 = skip)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="N",
                    help="before the timed region, launch the library's copy kernel N times on 1 GiB "
                         "(the known-size launch that traffic counters are scaled by)")
    ap.add_argument("--seed", type=int, default=1234)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (batch-1 decode is a single dependency chain and "
                 "would shard by tensor parallelism, which is not built); got --gpus %d" % args.gpus)

    if args.workload == "matmul-q8_0-4096":
        return bench_single_matmul(args)

    from vkllama_amd import capi, model as M

    wl = dict(WORKLOADS[args.workload])
    n_prompt, prefill_kv = wl.pop("prompt"), wl.pop("prefill_kv")
    cfg = wl
    steps, warmup = args.steps, args.warmup
    if n_prompt + steps + 1 > cfg["maxlen"]:
        sys.exit("prompt %d + %d steps exceed the context length %d" % (n_prompt, steps, cfg["maxlen"]))

    t0 = time.perf_counter()
    weights = M.synth_weights(cfg, seed=args.seed)
    t_synth = time.perf_counter() - t0
    rng = np.random.default_rng(args.seed)
    prompt = rng.integers(3, cfg["vocab"], n_prompt).astype(np.uint32)

    t0 = time.perf_counter()
    m = M.Llama2(cfg, weights)
    if args.decode_mode >= 0:
        m.set_option("decode_mode", args.decode_mode)
    m.set_option("decode_graph", args.decode_graph)
    t_load = time.perf_counter() - t0

    if args.copy_calibration > 0:
        dev = capi.Device(0)
        a, b = dev.alloc(1 << 30), dev.alloc(1 << 30)
        a.zero()
        for _ in range(args.copy_calibration):
            capi.check(capi.lib().vkl_copy_kernel(b.ptr, a.ptr, 1 << 30, dev.stream), "vkl_copy_kernel")
        dev.sync()
        a.free(), b.free()

    # warm-up: prompt pass + W decode steps, untimed (the prompt pass twice: its
    # first two runs also load code objects and fill the tensor pool)
    m.generate_greedy(prompt, 1)
    m.generate_greedy(prompt, warmup + 1)
    # timed: prompt pass (reported as prefill), then exactly `steps` decode steps
    ids, prefill_ms, decode_ms = m.generate_greedy(prompt, steps + 1)
    tok_s = steps / (decode_ms * 1e-3)
    ms_per_step = decode_ms / steps

    # algorithmic bytes per decode step, averaged over the contexts of the timed steps
    ctx = np.arange(n_prompt + 1, n_prompt + steps + 1)
    step_bytes = float(np.mean([m.decode_step_bytes(int(L)) for L in (ctx[0], ctx[-1])]))
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9

    # second pass over the same steps with an event pair around every phase launch
    m.set_option("decode_graph", 0)      # event pairs need the step-by-step launches
    m.set_option("phase_timing", 1)
    m.phase_times()
    m.generate_greedy(prompt, steps + 1)
    m.set_option("phase_timing", 0)
    m.set_option("decode_graph", args.decode_graph)
    phases = m.phase_times()
    L_mid = int(ctx[len(ctx) // 2])
    per_phase = {}
    for name, (ms, n) in phases.items():
        if n:
            per_phase[name] = {"launches_per_step": n // steps, "avg_us": round(ms * 1e3 / n, 3),
                               "us_per_step": round(ms * 1e3 / steps, 1),
                               "bytes_per_launch": m.phase_bytes(name, L_mid)}
    if "attention" in per_phase and "wo" not in per_phase and phases.get("wo", (0, 0))[1] == 0:
        # short contexts: the attention phase and the Wo projection are one launch
        fused = per_phase.pop("attention")
        fused["bytes_per_launch"] += m.phase_bytes("wo", L_mid)
        per_phase = {"kqv": per_phase.pop("kqv"), "attention+wo": fused, **per_phase} if "kqv" in per_phase \
            else {"attention+wo": fused, **per_phase}
    if per_phase:
        dom = max(per_phase, key=lambda k: per_phase[k]["us_per_step"])
        # the dominant kernel again, launched back to back (every layer's weights
        # in turn) between ONE event pair: its duration without a pair's own cost
        rounds = max(2, steps // 8)
        if dom == "attention+wo":
            # (no stand-alone replay of the fused launch: its average between event pairs)
            dom_us, dom_n = per_phase[dom]["avg_us"], phases["attention"][1]
        else:
            m.phase_replay(dom, L_mid - 1, 1)
            dom_us, dom_n = m.phase_replay(dom, L_mid - 1, rounds)
        dom_bytes = per_phase[dom]["bytes_per_launch"]
        # the kernel's name as a profiler prints it: phase number, weight type,
        # 4096-value chunks of the staged activation row
        phase_no = {"kqv": 0, "attention": 1, "attention+wo": 1, "wo": 2, "upgate": 3, "down": 4, "lm_head": 5,
                    "layer": 8}[dom]
        kstage = cfg["ffn"] if dom == "down" else cfg["dim"]
        per = 34.0 / 32.0 if cfg["wtype"] == 8 else 2.0
        wbytes = (cfg["n_layers"] * (4.0 * cfg["dim"] ** 2 + 3.0 * cfg["dim"] * cfg["ffn"])
                  + cfg["vocab"] * cfg["dim"]) * per
        if dom == "layer":
            # (row chunks of 4096 values as the library picks them: see launch_layer_wt)
            xd, xf = (cfg["dim"] + 4095) // 4096, (cfg["ffn"] + 4095) // 4096
            xd, xf = (1, 1) if (xd, xf) == (1, 1) else ((1, 3) if xd == 1 and xf <= 3 else (2, 4))
            dom_kernel = "decode_layer_kernel<%d, %d, %d, %s> (the five phases of a layer in one launch)" % (
                8 if cfg["wtype"] == 8 else 1, xd, xf, "true" if wbytes > (288 << 20) else "false")
        elif dom == "attention+wo":
            dom_kernel = "decode_attn_wo_kernel<%d, %d> (attention + Wo)" % (8 if cfg["wtype"] == 8 else 1,
                                                                            min(4, (cfg["dim"] + 4095) // 4096))
        elif dom == "attention":
            dom_kernel = "decode_phase_kernel<1, %d> (attention)" % (8 if cfg["wtype"] == 8 else 1)
        else:
            # last argument: weights of a step beyond what the caches hold are
            # requested with the non-temporal hint (same rule as the library's)
            dom_kernel = "decode_phase_direct_kernel<%d, %d, %d, %s> (%s)" % (
                phase_no, 8 if cfg["wtype"] == 8 else 1, min(4, (kstage + 4095) // 4096),
                "true" if wbytes > (288 << 20) else "false", dom)
        dom_pair_us = per_phase[dom]["avg_us"]
    else:
        dom, dom_us, dom_n, dom_bytes = None, ms_per_step * 1e3, steps, step_bytes
        dom_kernel, dom_pair_us = "decode step (all launches of one token)", None
    dom_gbs = dom_bytes / (dom_us * 1e-6) / 1e9

    # the same loop through Model::operator() (token id from the host, 128 KB of
    # logits back to the host per token, host arg-max): the PCIe-inclusive rate
    n_host = min(32, steps)
    logits = m.forward(prompt, 0)
    tok, pos = int(np.argmax(logits)), n_prompt
    t0 = time.perf_counter()
    for _ in range(n_host):
        logits = m.forward([tok], pos)
        tok, pos = int(np.argmax(logits)), pos + 1
    host_tok_s = n_host / (time.perf_counter() - t0)

    result = {
        "metric": "decode_tokens_per_second_bs1",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("q8_0" if cfg["wtype"] == 8 else "f16") + " weights x f16 activations, f32 accumulate",
        "data": "synthetic: random-init N(0,0.02) weights" + (" quantised to Q8_0" if cfg["wtype"] == 8 else " in FP16")
                + ", random prompt ids",
        "config": {"workload": args.workload, "prompt_tokens": n_prompt, "decode_tokens": steps,
                   "decode_mode": ("one launch per layer" if "layer" in per_phase else "one launch per phase")
                                  + (", replayed from a HIP graph" if args.decode_graph else ""),
                   "dims": {k: cfg[k] for k in ("dim", "n_layers", "n_heads", "ffn", "vocab", "maxlen")}},
        "decode_tokens_per_second_host_interface": round(host_tok_s, 1),
        "prefill_tokens_per_second": round(n_prompt / (prefill_ms * 1e-3), 1),
        "roofline": {"bound": "hbm", "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom_gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC.get((args.workload, dom), (None, None))[0],
                     "traffic_source": ("quoted from the counter runs summarised in " + TRAFFIC[(args.workload, dom)][1]
                                        + ", not measured by this run") if (args.workload, dom) in TRAFFIC else None,
                     "kernel": dom_kernel,
                     "avg_launch_us": round(dom_us, 3), "launches_timed": dom_n,
                     "avg_launch_us_with_event_pair": dom_pair_us,
                     "bytes_per_launch": int(dom_bytes),
                     "step_achieved": round(achieved, 1), "step_frac": round(achieved / HBM_PEAK_GBS, 4),
                     "bytes_per_step": int(step_bytes)},
        "phases": per_phase,
        "load_seconds": {"synthesize": round(t_synth, 1), "upload": round(t_load, 1)},
        "first_ids": [int(t) for t in ids[:8]],
    }

    cpu_tokens = args.cpu_tokens
    if cpu_tokens < 0:
        cpu_tokens = 128 if cfg["dim"] >= 4096 else 1024
    cpu_tokens = min(cpu_tokens, cfg["maxlen"] - 8)     # 4-token prompt, then one position per token
    if cpu_tokens > 0:
        m.set_option("decode_graph", args.decode_graph)
        v, dt, parity = cpu_baseline(cfg, weights, cpu_tokens, m)
        result["parity"] = parity
        result["cpu_baseline"] = {
            "value": round(v, 3), "unit": "tok/s", "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count())),
            "kind": "port",
            "sample": "%d greedy decode tokens at context 5..%d after a 4-token prompt, same weights (%.1f s)"
                      % (cpu_tokens, 4 + cpu_tokens, dt)}
    m.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
