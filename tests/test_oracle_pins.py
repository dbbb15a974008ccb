"""Pins for the CPU oracle (oracle/vkl_oracle.c).

The reference holds no golden vectors for this path (its tests draw unseeded
random inputs and compare with Eigen), so each oracle function is pinned by
what the mathematics fixes: closed forms evaluated in float64 by independent
numpy code, invariants, special cases that reduce to an exact answer, and the
tolerances / edge cases the reference's own tests name (cited per test).
"""
import numpy as np
import pytest

from oracle import oracle as O
from util import q8_weights, rel_err, ulp_diff_f16


# ---------------------------------------------------------------- fp16 ------
def test_f16_to_f32_all_bit_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.f16_bits_to_f32(b) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rne_against_numpy_and_f16c(rng):
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),   # subnormal range
        (rng.standard_normal(5000) * 3e4).astype(np.float32),    # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e10, -1e10, np.inf, -np.inf,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25], np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    sw = np.array([O.f32_to_f16_bits(x) for x in xs], np.uint16)
    hw = np.array([O.f32_to_f16_bits(x, hw=True) for x in xs], np.uint16)
    assert np.array_equal(sw, want)
    assert np.array_equal(hw, want)


def test_reference_host_fp16_helper_truncates():
    # src/core/float.h:52-112 truncates the mantissa and clamps to 65504
    x = np.float32(1.0 + 2.0 ** -10 + 2.0 ** -11 + 2.0 ** -12)  # RNE rounds up, truncation does not
    assert O.f32_to_f16_bits(x) == np.float16(1.0 + 2 * 2.0 ** -10).view(np.uint16)
    assert O.ref_host_f32_to_f16_bits(x) == np.float16(1.0 + 2.0 ** -10).view(np.uint16)
    assert O.ref_host_f32_to_f16_bits(1e6) == np.float16(65504).view(np.uint16)


# ---------------------------------------------------------------- Q8_0 ------
def _split(raw, scale_bytes):
    bb = 32 + scale_bytes
    blocks = raw.reshape(-1, bb)
    q = blocks[:, scale_bytes:].view(np.int8)
    if scale_bytes == 4:
        d = blocks[:, :4].copy().view(np.float32).reshape(-1)
    else:
        d = blocks[:, :2].copy().view(np.float16).reshape(-1)
    return q, d


def test_quantize_invariants(rng):
    x = rng.uniform(-5, 5, size=(7, 96)).astype(np.float32)
    x[3, 32:64] = 0.0                                   # an all-zero block
    r4 = O.quantize_q8_0(x, 4)
    r2 = O.quantize_q8_0(x, 2)
    q4, d4 = _split(r4, 4)
    q2, d2 = _split(r2, 2)
    assert np.array_equal(q4, q2)                        # payload independent of the scale format
    assert np.array_equal(d4.astype(np.float16), d2)     # fp16 scale = RNE of the fp32 scale
    assert np.abs(q4.astype(np.int32)).max() <= 127
    xb = x.reshape(-1, 32)
    amax_pos = np.argmax(np.abs(xb), axis=1)
    rows = np.arange(xb.shape[0])
    nz = np.abs(xb).max(axis=1) > 0
    assert np.all(np.abs(q4[rows, amax_pos][nz]) == 127)                 # arg-max element -> +-127
    assert np.all(np.sign(q4[rows, amax_pos][nz]) == np.sign(xb[rows, amax_pos][nz]))
    assert np.all(d4[~nz] == 0) and np.all(q4[~nz] == 0)                 # zero block -> scale 0, q 0
    err = np.abs(xb - q4.astype(np.float64) * d4[:, None].astype(np.float64))
    assert np.all(err <= d4[:, None] / 2 * (1 + 1e-5) + 1e-12)           # |x - q d| <= d/2
    assert np.allclose(d4[nz], np.abs(xb).max(axis=1)[nz] / 127.0, rtol=1e-7)


def test_quantize_roundtrip_like_reference_test(rng):
    # tests/test_quants.cpp:26-52: n = 95 values in U(-5,5), |x - deq(q(x))| < 1e-1
    x = rng.uniform(-5, 5, size=(1, 95)).astype(np.float32)
    for sb in (2, 4):
        raw = O.quantize_q8_0(x, sb)
        assert raw.shape[1] == 3 * (32 + sb)
        q, _ = _split(raw, sb)
        assert q[2, 31] == 0                             # tail padded with zero
        back = O.dequantize_q8_0(raw, 95, sb)
        assert np.abs(back - x).max() < 1e-1


def test_quantize_rounds_half_away_from_zero():
    x = np.zeros((1, 32), np.float32)
    x[0, 0] = 127.0                                       # scale 1, inverse exactly 1
    x[0, 1:7] = [0.5, -0.5, 1.5, 2.5, -2.5, 126.5]
    q, d = _split(O.quantize_q8_0(x, 4), 4)
    assert d[0] == 1.0
    assert list(q[0, :7]) == [127, 1, -1, 2, 3, -3, 127]  # roundf, not round-half-even


# ------------------------------------------------------------- embedding ----
def test_embedding_q8_gather_and_unk(rng):
    V, W = 50, 96
    raw, deq = q8_weights(rng, V, W)
    toks = np.array([0, 49, 7, 50, 2 ** 31, 7], np.uint32)     # 50 and 2^31 are out of range -> UNK = 0
    got = O.embedding_q8_0(raw, W, toks, unk=0)
    want_rows = np.array([0, 49, 7, 0, 0, 7])
    # fp16(q*d): the fp32 product is exact, so float64 -> fp16 gives the same bits
    want = deq[want_rows][:, :W].astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_embedding_f16_gather(rng):
    table = rng.standard_normal((20, 64)).astype(np.float16)
    toks = np.array([3, 19, 20, 0], np.uint32)
    got = O.embedding_f16(table, toks, unk=5)
    assert np.array_equal(got, table[[3, 19, 5, 0]])


# --------------------------------------------------------------- matmul -----
@pytest.mark.parametrize("M,N,K", [(1, 37, 256), (3, 64, 1376), (2, 10, 4096)])
def test_matmul_q8_0_vs_float64(rng, M, N, K):
    raw, deq = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    want = x.astype(np.float64) @ deq[:, :K].T
    got = O.matmul_q8_0(x, raw, K)
    # fp32 accumulation error is far below fp16 rounding: at most 1 ulp off the rounded fp64 result
    assert ulp_diff_f16(got, want.astype(np.float16)).max() <= 1
    assert rel_err(got, want) < 1e-2


def test_matmul_q8_0_one_hot_is_exact_column(rng):
    N, K = 12, 128
    raw, deq = q8_weights(rng, N, K)
    for k in (0, 31, 32, 77, 127):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        got = O.matmul_q8_0(x, raw, K)
        assert np.array_equal(got[0], deq[:, k].astype(np.float16))


def test_matmul_q8_0_scale_bias_silu(rng):
    N, K = 16, 64
    raw, deq = q8_weights(rng, N, K, 0.01, 0.05)
    x = rng.standard_normal((1, K)).astype(np.float16)
    base = x.astype(np.float64) @ deq.T
    v = base * 0.5 + 0.25
    got = O.matmul_q8_0(x, raw, K, scale=0.5, bias=0.25, act=0)
    assert rel_err(got, v) < 2e-3
    got = O.matmul_q8_0(x, raw, K, scale=0.5, bias=0.25, act=1)
    assert rel_err(got, v / (1 + np.exp(-v))) < 2e-3


def test_kqv_equals_three_matmuls_and_keeps_output_order(rng):
    N, K, M = 24, 128, 2
    ws = [q8_weights(rng, N, K)[0] for _ in range(3)]
    x = rng.standard_normal((M, K)).astype(np.float16)
    k, q, v = O.kqv_q8_0(x, ws[0], ws[1], ws[2], K)
    for got, w in zip((k, q, v), ws):
        assert np.array_equal(got.view(np.uint16), O.matmul_q8_0(x, w, K).view(np.uint16))


def test_ffn_upgate_q8_0(rng):
    N, K, M = 40, 128, 2
    (up, dup), (gate, dgate) = q8_weights(rng, N, K, 0.01, 0.03), q8_weights(rng, N, K, 0.01, 0.03)
    x = rng.standard_normal((M, K)).astype(np.float16)
    u = x.astype(np.float64) @ dup.T
    g = x.astype(np.float64) @ dgate.T
    want = g / (1 + np.exp(-g)) * u                      # tests/test_feedforward.cpp:114-119
    got = O.ffn_upgate_q8_0(x, up, gate, K)
    assert rel_err(got, want) < 3e-3
    # argument order: SiLU acts on the SECOND weight (gate); swapping must change the result
    swapped = O.ffn_upgate_q8_0(x, gate, up, K)
    assert rel_err(swapped, want) > 1e-2


@pytest.mark.parametrize("C,M,N,K", [(1, 9, 9, 128), (3, 2, 5, 64), (2, 1, 7, 192)])
def test_matmul_f16_tb_vs_float64(rng, C, M, N, K):
    # tests/test_matmul.cpp:190-208 runs {C1,M9,N9,K128}, transpose_b
    a = rng.standard_normal((C, M, K)).astype(np.float16)
    b = rng.standard_normal((C, N, K)).astype(np.float16)
    want = np.einsum("cmk,cnk->cmn", a.astype(np.float64), b.astype(np.float64)) * 0.125
    got = O.matmul_f16_tb(a, b, scale=0.125)
    assert got.shape == (C, M, N)
    assert ulp_diff_f16(got, want.astype(np.float16)).max() <= 1


@pytest.mark.parametrize("C,M,N,K", [(2, 3, 64, 130), (1, 1, 16, 17), (4, 2, 8, 300)])
def test_matmul_f16_nn_vs_float64(rng, C, M, N, K):
    a = rng.standard_normal((C, M, K)).astype(np.float16)
    b = rng.standard_normal((C, K, N)).astype(np.float16)
    want = np.einsum("cmk,ckn->cmn", a.astype(np.float64), b.astype(np.float64))
    got = O.matmul_f16_nn(a, b)
    assert ulp_diff_f16(got, want.astype(np.float16)).max() <= 1


def test_ffn_upgate_f16(rng):
    M, N, K = 2, 33, 128
    x = rng.standard_normal((M, K)).astype(np.float16)
    up = (rng.standard_normal((N, K)) * 0.1).astype(np.float16)
    gate = (rng.standard_normal((N, K)) * 0.1).astype(np.float16)
    u = x.astype(np.float64) @ up.astype(np.float64).T
    g = x.astype(np.float64) @ gate.astype(np.float64).T
    got = O.ffn_upgate_f16(x, up, gate)
    assert rel_err(got, g / (1 + np.exp(-g)) * u) < 3e-3


# ---------------------------------------------------------------- RMSNorm ---
def test_rmsnorm_closed_form_and_unit_rms(rng):
    rows, W = 5, 1000                                     # W not a multiple of the 512-thread stride
    x = (rng.standard_normal((rows, W)) * 3).astype(np.float16)
    w = rng.uniform(0.5, 1.5, W).astype(np.float32)
    xf = x.astype(np.float64)
    want = xf * w / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-5)   # tests/test_rmsnorm.cpp:77-86
    got = O.rmsnorm(x, w, 1e-5)
    assert ulp_diff_f16(got, want.astype(np.float16)).max() <= 1
    ones = O.rmsnorm(x, np.ones(W, np.float32), 0.0).astype(np.float64)
    assert np.allclose(np.sqrt((ones ** 2).mean(axis=1)), 1.0, atol=2e-3)
    # eps matters: a zero row stays zero instead of producing NaN
    z = O.rmsnorm(np.zeros((1, W), np.float16), w, 1e-5)
    assert np.all(z == 0)


# ------------------------------------------------------------------ RoPE ----
def test_rope_tables_closed_form():
    maxlen, dim = 600, 64
    fc, fs = O.rope_tables(maxlen, dim)
    p = np.arange(maxlen, dtype=np.float64)[:, None]
    freq = 10000.0 ** (-np.arange(0, dim, 2, dtype=np.float64) / dim)[None, :]
    assert np.abs(fc - np.cos(p * freq)).max() < 2e-4     # float angle p*freq carries ~p*6e-8 error
    assert np.abs(fs - np.sin(p * freq)).max() < 2e-4
    assert np.all(fc[0] == 1.0) and np.all(fs[0] == 0.0)


def test_rope_identity_norm_and_composition(rng):
    C, H, W, maxlen = 3, 4, 64, 256
    fc, fs = O.rope_tables(maxlen, W)
    x = rng.standard_normal((C, H, W)).astype(np.float16)
    # position 0 is the identity, exactly (only row 0 sits at position 0)
    y0 = O.rope(x[:, :1], fc, fs, 0)
    assert np.array_equal(y0, x[:, :1])
    # rotation preserves each adjacent pair's norm (tests/test_rope.cpp:21-49 rotates pairs (2i, 2i+1))
    y = O.rope(x, fc, fs, 100).astype(np.float64)
    xn = x.astype(np.float64)
    n_in = xn[..., 0::2] ** 2 + xn[..., 1::2] ** 2
    n_out = y[..., 0::2] ** 2 + y[..., 1::2] ** 2
    assert np.allclose(n_in, n_out, rtol=5e-3, atol=1e-4)
    # closed form in float64 for row y at position y + offset
    pos = (np.arange(H) + 100)[None, :, None]
    freq = 10000.0 ** (-np.arange(0, W, 2, dtype=np.float64) / W)[None, None, :]
    c, s = np.cos(pos * freq), np.sin(pos * freq)
    want = np.empty_like(xn)
    want[..., 0::2] = xn[..., 0::2] * c - xn[..., 1::2] * s
    want[..., 1::2] = xn[..., 0::2] * s + xn[..., 1::2] * c
    assert np.abs(y - want).max() < 4e-3                  # tests/test_rope.cpp:202 uses 1e-3 on U(-1,1)
    # composition R(p1) R(p2) = R(p1 + p2) up to two fp16 roundings
    a = O.rope(O.rope(x[:, :1], fc, fs, 30), fc, fs, 70).astype(np.float64)
    b = O.rope(x[:, :1], fc, fs, 100).astype(np.float64)
    assert np.abs(a - b).max() < 8e-3


# --------------------------------------------------------------- KV cache ---
def test_kvcache_update_wraps():
    # tests/test_update_kv_cache.cpp:117-118: offsets 0 and 1022 of 1024
    C, HO, H, W = 2, 1024, 5, 8
    cache = np.zeros((C, HO, W), np.float16)
    kv = (np.arange(C * H * W).reshape(C, H, W) % 97 + 1).astype(np.float16)
    out = O.update_kvcache(cache, kv, 1022)
    assert np.array_equal(out[:, 1022], kv[:, 0]) and np.array_equal(out[:, 1023], kv[:, 1])
    assert np.array_equal(out[:, 0], kv[:, 2]) and np.array_equal(out[:, 2], kv[:, 4])
    assert np.count_nonzero(out) == kv.size
    out0 = O.update_kvcache(cache, kv, 0)
    assert np.array_equal(out0[:, :H], kv)


# ---------------------------------------------------------------- softmax ---
def test_softmax_closed_form_and_mask(rng):
    C, H, W, off = 2, 5, 70, 64
    x = (rng.standard_normal((C, H, W)) * 2).astype(np.float16)
    got = O.softmax(x, True, off).astype(np.float64)
    xf = x.astype(np.float64)
    for y in range(H):
        keep = np.arange(W) <= y + off                   # softmax_fp16.comp:53,65: masked iff i > row + OFFSET
        e = np.exp(xf[:, y] - xf[:, y].max(axis=1, keepdims=True)) * keep
        want = e / e.sum(axis=1, keepdims=True)
        assert np.abs(got[:, y] - want).max() < 1e-3      # tests/test_softmax.cpp:105 allows 1e-2
        assert np.all(got[:, y][:, ~keep] == 0)
        assert abs(got[:, y].sum(axis=1) - 1).max() < 5e-3
    unmasked = O.softmax(x, False, 0).astype(np.float64)
    assert np.allclose(unmasked.sum(axis=2), 1.0, atol=5e-3)
    assert np.all(unmasked > 0)


# ------------------------------------------------- element-wise / arg / T ---
def test_elementwise_ops(rng):
    a = rng.standard_normal(1000).astype(np.float16)
    b = (rng.standard_normal(1000) + 3).astype(np.float16)
    af, bf = a.astype(np.float32), b.astype(np.float32)
    for op, want in enumerate([af + bf, af - bf, af * bf, af / bf]):
        assert np.array_equal(O.elementwise(a, b, op).view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_argmax_first_maximum(rng):
    x = rng.standard_normal((6, 3000)).astype(np.float16)
    x[2, 17] = x[2, 2500] = 30.0                           # tie -> lowest index (argmax_stage1.comp:44)
    x[4, :] = -1.0
    want = np.argmax(x.astype(np.float32), axis=1)        # tests/test_argop.cpp:94-102: first maximum
    assert list(O.argmax_f16(x)) == list(want)
    assert O.argmax_f16(x)[2] == 17 and O.argmax_f16(x)[4] == 0
    assert O.argmax_f32(x[2].astype(np.float32)) == 17


def test_transpose102(rng):
    x = rng.standard_normal((3, 5, 8)).astype(np.float16)
    assert np.array_equal(O.transpose102(x), x.transpose(1, 0, 2))


# ------------------------------------------------------------------ model ---
def _tiny(rng, wtype=8, dim=64, L=2, H=4, F=96, V=128, maxlen=32):
    from llama_ref import make_weights
    cfg = dict(dim=dim, n_layers=L, n_heads=H, ffn=F, vocab=V, maxlen=maxlen, eps=1e-5, wtype=wtype)
    return cfg, make_weights(rng, cfg)


@pytest.mark.parametrize("wtype", [8, 1])
def test_model_matches_textbook_float64_forward(rng, wtype):
    """Whole-model wiring (weight roles, rope pairing, score scale, causal
    mask, residuals, eps values, lm_head) against an independent float64
    implementation; decode steps only, where the reference has no quirk."""
    from llama_ref import forward_f64
    cfg, (w, wf) = _tiny(rng, wtype)
    m = O.OracleModel(cfg, w)
    toks = [5, 17, 99, 3, 64]
    ref_cache = {}
    for pos, t in enumerate(toks):
        got = m.forward([t], pos)
        want = forward_f64(cfg, wf, [t], pos, ref_cache)
        assert np.abs(got - want).max() < 0.03 * np.abs(want).max()
        assert np.corrcoef(got, want)[0, 1] > 0.999


def test_model_prefill_vs_decode_and_lastblock_quirk(rng):
    cfg, (w, wf) = _tiny(rng)
    toks = np.array([5, 17, 99, 3, 64, 8], np.uint32)
    step = O.OracleModel(cfg, w)
    for pos, t in enumerate(toks):
        logits_step = step.forward([t], pos)
    quirk = O.OracleModel(cfg, w, lastblock_rope_quirk=True)
    fixed = O.OracleModel(cfg, w, lastblock_rope_quirk=False)
    lq = quirk.forward(toks, 0)
    lf = fixed.forward(toks, 0)
    S = len(toks)
    # the caches of a prefill equal the caches of token-by-token decoding: exactly in layer 0
    # (row-wise identical arithmetic), within fp16 noise deeper down
    assert np.array_equal(step.kcache(0)[:, :S], fixed.kcache(0)[:, :S])
    assert np.array_equal(step.vcache(0)[:, :S], fixed.vcache(0)[:, :S])
    for l in range(cfg["n_layers"]):
        assert np.abs(step.kcache(l)[:, :S].astype(np.float32) - fixed.kcache(l)[:, :S].astype(np.float32)).max() < 2e-2
        assert np.array_equal(quirk.kcache(l), fixed.kcache(l))   # the quirk touches the query only
    # without the quirk a prefill predicts what decoding predicts
    assert np.abs(lf - logits_step).max() < 2e-2 * max(1.0, np.abs(logits_step).max())
    # with it (multiheadattention_v2.cpp:222-233,251 + rope_fp16.comp:34) the last query is rotated
    # at position `offset` instead of offset+S-1, which changes the logits for S > 1 ...
    assert np.abs(lq - lf).max() > 10 * np.abs(lf - logits_step).max()
    # ... and nothing for S == 1
    a = O.OracleModel(cfg, w, True).forward(toks[:1], 0)
    b = O.OracleModel(cfg, w, False).forward(toks[:1], 0)
    assert np.array_equal(a, b)


def test_generate_greedy_follows_the_app_loop(rng):
    cfg, (w, wf) = _tiny(rng)
    prompt = np.array([5, 17, 99, 3], np.uint32)
    m = O.OracleModel(cfg, w)
    ids, first = m.generate_greedy(prompt, 6)
    # app/llama2_infer.cpp:141-176: prompt at offset 0, then one token at offset toks.size()-1
    m2 = O.OracleModel(cfg, w)
    logits = m2.forward(prompt, 0)
    assert np.array_equal(first, logits)
    seq = list(prompt)
    out = []
    for _ in range(6):
        tok = int(np.argmax(logits))                      # first maximum
        out.append(tok)
        seq.append(tok)
        logits = m2.forward([tok], len(seq) - 1)
    assert list(ids) == out


def test_lane_orders_are_reassociations_of_one_sum():
    """The oracle's lane-order switch (the reference's subgroupAdd leaves the
    order open) only re-associates the 32 partial sums: with weights and
    activations that make every partial sum an exactly representable integer
    all orders give the same bits, and on random data every order agrees with
    the fp64 product to fp32 accuracy while at least one differs from order 0
    in its last bits."""
    rng = np.random.default_rng(11)
    N, K = 64, 1024
    q = rng.integers(-8, 9, size=(N, K // 32, 32), dtype=np.int8)
    raw = np.empty((N, K // 32, 34), np.uint8)
    raw[:, :, :2] = np.array([1.0], np.float16).view(np.uint8)      # scale 1
    raw[:, :, 2:] = q.view(np.uint8)
    raw = raw.reshape(N, -1)
    x_int = rng.integers(-4, 5, size=(1, K)).astype(np.float16)
    x_rnd = rng.standard_normal((1, K)).astype(np.float16)
    try:
        exact = [O.matmul_q8_0(x_int, raw, K).view(np.uint16).copy() for o in range(5) if O.set_lane_order(o) is None]
        assert all(np.array_equal(e, exact[0]) for e in exact)
        want = x_rnd.astype(np.float64) @ q.reshape(N, K).astype(np.float64).T
        outs = []
        for o in range(5):
            O.set_lane_order(o)
            y = O.matmul_q8_0(x_rnd, raw, K).astype(np.float64)
            assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()        # fp16 output rounding
            outs.append(y)
    finally:
        O.set_lane_order(0)
    # (fp16 outputs hide most last-bit differences of the fp32 sums; the orders
    # are distinct code paths all the same: see the fixture test in
    # test_golden.py for their effect through 32 layers)
    assert len(outs) == 5
