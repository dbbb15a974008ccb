"""Parity of every HIP operator kernel with the CPU oracle, through the C ABI.

Bars: bit-exact for Q8_0 repacking, embedding gather,
KV-cache writes, arg-max ids and plain copies; fp16 outputs within 1e-2
relative of the oracle (measured against max(|ref|, 1e-2 max|ref|)).
"""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from util import q8_weights, rel_err, ulp_diff_f16, within_one_ulp_or_cancelled
from vkllama_amd import capi

pytestmark = pytest.mark.gpu

F16_REL_TOL = 1e-2


def L():
    return capi.lib()


def f16(buf, shape):
    return buf.read(np.uint16, shape).view(np.float16)


# ------------------------------------------------------------------ Q8_0 ----
@pytest.mark.parametrize("rows,K", [(5, 32), (64, 1376), (33, 4096), (7, 100)])
def test_q8_pack_unpack_roundtrip_bit_exact(dev, rng, rows, K):
    raw, _ = q8_weights(rng, rows, K)
    nb = (K + 31) // 32
    staging = dev.upload(raw)
    planar = dev.alloc(raw.nbytes)
    back = dev.alloc(raw.nbytes)
    capi.check(L().vkl_q8_0_pack(staging.ptr, planar.ptr, rows, K, dev.stream))
    capi.check(L().vkl_q8_0_unpack(planar.ptr, back.ptr, rows, K, dev.stream))
    p = planar.read(np.uint8, raw.nbytes)
    blocks = raw.reshape(rows * nb, 34)
    assert np.array_equal(p[:rows * nb * 32].reshape(-1, 32), blocks[:, 2:])      # int8 plane
    assert np.array_equal(p[rows * nb * 32:].reshape(-1, 2), blocks[:, :2])       # scale plane
    assert np.array_equal(back.read(np.uint8, raw.shape), raw)


# -------------------------------------------------------------- embedding ---
def test_embedding_q8_bit_exact(dev, rng):
    V, W = 300, 512
    raw, _ = q8_weights(rng, V, W)
    toks = np.array([0, 299, 7, 300, 2 ** 31 + 5, 7, 128], np.uint32)
    table = dev.upload_q8_0(raw, V, W)
    dt = dev.upload(toks)
    out = dev.alloc(toks.size * W * 2)
    capi.check(L().vkl_embed_q8_0(table.ptr, V, W, dt.ptr, toks.size, 0, out.ptr, dev.stream))
    want = O.embedding_q8_0(raw, W, toks, 0)
    assert np.array_equal(f16(out, want.shape).view(np.uint16), want.view(np.uint16))


def test_embedding_f16_bit_exact(dev, rng):
    V, W = 100, 200
    table = rng.standard_normal((V, W)).astype(np.float16)
    toks = np.array([3, 99, 100, 0], np.uint32)
    dtab, dt = dev.upload(table), dev.upload(toks)
    out = dev.alloc(toks.size * W * 2)
    capi.check(L().vkl_embed_f16(dtab.ptr, V, W, dt.ptr, toks.size, 5, out.ptr, dev.stream))
    assert np.array_equal(f16(out, (4, W)), O.embedding_f16(table, toks, 5))


# ----------------------------------------------------------------- RMSNorm --
@pytest.mark.parametrize("rows,W", [(1, 4096), (16, 512), (3, 1000), (2, 5120), (33, 4096), (2, 1004), (3, 8200), (2, 8192)])
def test_rmsnorm(dev, rng, rows, W):
    x = (rng.standard_normal((rows, W)) * 2).astype(np.float16)
    w = rng.uniform(0.5, 1.5, W).astype(np.float32)
    dx, dw = dev.upload(x), dev.upload(w)
    out = dev.alloc(x.nbytes)
    capi.check(L().vkl_rmsnorm_f16(dx.ptr, dw.ptr, rows, W, 1e-5, out.ptr, dev.stream))
    got, want = f16(out, x.shape), O.rmsnorm(x, w, 1e-5)
    assert ulp_diff_f16(got, want).max() <= 1
    assert rel_err(got, want) < F16_REL_TOL


# ------------------------------------------------------------ Q8_0 matmul ---
def _run_matmul_q8(dev, x, raw, N, K, scale=1.0, bias=0.0, act=0, residual=None, want32=False):
    M = x.shape[0]
    dx = dev.upload(x)
    dw = dev.upload_q8_0(raw, N, K)
    dy = dev.alloc(M * N * 2)
    dres = dev.upload(residual) if residual is not None else None
    d32 = dev.alloc(M * N * 4) if want32 else None
    capi.check(L().vkl_matmul_q8_0(dx.ptr, dw.ptr, M, N, K, K, N, scale, bias, act,
                                   dres.ptr if dres else None, dy.ptr, d32.ptr if d32 else None, dev.stream))
    y = f16(dy, (M, N))
    return (y, d32.read(np.float32, (M, N))) if want32 else y


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (1, 37, 256), (1, 512, 1376), (1, 1376, 512), (3, 64, 1376),
                                   (16, 130, 512), (1, 6, 11008), (5, 9, 100)])
def test_matmul_q8_0(dev, rng, M, N, K):
    raw, deq = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    got = _run_matmul_q8(dev, x, raw, N, K)
    want = O.matmul_q8_0(x, raw, K)
    assert rel_err(got, want) < F16_REL_TOL
    assert within_one_ulp_or_cancelled(got, want).all()   # same products, fp32 sums in another order
    exact = x.astype(np.float64) @ deq[:, :K].T
    assert rel_err(got, exact) < F16_REL_TOL


def test_matmul_q8_0_one_hot_exact_and_subnormal_activations(dev, rng):
    N, K = 40, 256
    raw, deq = q8_weights(rng, N, K)
    for k in (0, 15, 16, 31, 32, 255):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        got = _run_matmul_q8(dev, x, raw, N, K)
        assert np.array_equal(got[0], deq[:, k].astype(np.float16))
    # activations in the fp16 subnormal range must still contribute
    x = (rng.standard_normal((1, K)) * 2e-5).astype(np.float16)
    raw2, _ = q8_weights(rng, N, K, 0.5, 1.0)
    got = _run_matmul_q8(dev, x, raw2, N, K)
    want = O.matmul_q8_0(x, raw2, K)
    assert rel_err(got, want) < F16_REL_TOL


def test_matmul_q8_0_epilogue(dev, rng):
    M, N, K = 2, 96, 512
    raw, _ = q8_weights(rng, N, K, 0.01, 0.03)
    x = rng.standard_normal((M, K)).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = _run_matmul_q8(dev, x, raw, N, K, scale=0.5, bias=0.25, act=1)
    want = O.matmul_q8_0(x, raw, K, 0.5, 0.25, 1)
    assert rel_err(got, want) < F16_REL_TOL
    got, got32 = _run_matmul_q8(dev, x, raw, N, K, residual=res, want32=True)
    want = O.elementwise(O.matmul_q8_0(x, raw, K), res, 0)
    assert rel_err(got, want) < F16_REL_TOL
    assert np.array_equal(got32, got.astype(np.float32))  # the widening cast is exact


# ------------------------------------------------- prompt-pass GEMM (MFMA) --
@pytest.mark.parametrize("M,N,K", [(9, 128, 32), (16, 130, 512), (64, 256, 4096), (100, 200, 1376), (300, 1376, 512),
                                   (129, 64, 11008), (65, 32000, 512),
                                   (7, 200, 1376), (32, 129, 768), (5, 64, 256), (31, 300, 11008), (2, 1000, 5120),
                                   (270, 12300, 64), (600, 13000, 192), (1030, 6144, 448), (777, 8200, 320),
                                   (300, 8192, 64), (256, 4096, 2048),
                                   (9, 6416, 1024), (32, 12288, 768), (3, 16368, 1280),
                                   (64, 12288, 768), (33, 6416, 1024), (50, 16368, 1280),
                                   (96, 12288, 768), (65, 6416, 1024), (80, 16368, 1280), (128, 12288, 768), (110, 6416, 1024),
                                   (24, 4000, 768), (64, 4000, 768), (90, 4000, 1024), (110, 16400, 64)])
def test_gemm_q8_0_many_rows(dev, rng, M, N, K):
    """Several token rows run on the matrix cores (quants as exact fp16
    integers, block sums by MFMA, block scale in fp32); the shapes cover the
    few-row kernels (K a multiple of 256 or not, a last slice that is half
    empty, row counts that do not fill the last workgroup), half- and
    full-height tiles, the k-split, and (the last five: about two hundred
    256 x 128 tiles and more, or half as many 128 x 128 ones, K a multiple of
    64) the form that loads its tiles straight into LDS, with ragged M and N,
    one to seven k-steps, and its k range split in two; the last three: at
    most 32 token rows against 512 and more groups of 16 weight rows, K a
    multiple of 256: workgroups that run over the whole of K (2, 3 and 4
    groups each, the last workgroup not full), and the same with 33 to 96
    token rows (two and three blocks of 32 rows per workgroup) and with 97 to 128 (a
    second launch for the rows past 96); the last three: one group per workgroup
    (the Wo product of a short prompt) with one, two and three blocks of 32 rows."""
    raw, deq = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    got = _run_matmul_q8(dev, x, raw, N, K)
    if M * N * K <= 3e8 or K == 2048 or M <= 128:
        want = O.matmul_q8_0(x, raw, K)
        assert rel_err(got, want) < F16_REL_TOL
    exact = x.astype(np.float64) @ deq[:, :K].T
    assert rel_err(got, exact) < 2e-3


@pytest.mark.parametrize("M,N,K", [(40, 200, 512), (72, 200, 2048), (20, 200, 2048), (260, 12300, 64),
                                   (260, 4096, 2048), (20, 8224, 1024), (40, 8224, 1024), (100, 8224, 1024), (20, 4000, 1024)])
def test_gemm_q8_0_epilogue_and_strides(dev, rng, M, N, K):
    """scale / bias / activation, residual, widened copy and row strides: on
    the tile kernel without (K 512) and with the k-split, on the few-row
    kernel (20 rows; these two finish in the reduction kernel) and on the
    256-row tiles (260 rows: 16-byte stores, and single ones where the output
    rows are not 16-byte aligned; with K 2048 the k range split in two, which
    finishes in the reduction kernel as well), and on the few-row kernel whose
    workgroups run over the whole of K (20, 40 and, in two launches, 100 rows x 8224)"""
    raw, _ = q8_weights(rng, N, K, 0.01, 0.03)
    x = rng.standard_normal((M, K)).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = _run_matmul_q8(dev, x, raw, N, K, scale=0.5, bias=0.25, act=1)
    assert rel_err(got, O.matmul_q8_0(x, raw, K, 0.5, 0.25, 1)) < F16_REL_TOL
    got, got32 = _run_matmul_q8(dev, x, raw, N, K, residual=res, want32=True)
    want = O.elementwise(O.matmul_q8_0(x, raw, K), res, 0)
    assert rel_err(got, want) < F16_REL_TOL
    assert np.array_equal(got32, got.astype(np.float32))
    # rows of x and y embedded in wider buffers
    xs, ys = K + 64, N + 8
    xw = np.zeros((M, xs), np.float16)
    xw[:, :K] = x
    dx, dw = dev.upload(xw), dev.upload_q8_0(raw, N, K)
    dy = dev.alloc(M * ys * 2)
    dy.zero()
    capi.check(L().vkl_matmul_q8_0(dx.ptr, dw.ptr, M, N, K, xs, ys, 1.0, 0.0, 0, None, dy.ptr, None, dev.stream))
    yw = f16(dy, (M, ys))
    assert rel_err(yw[:, :N], O.matmul_q8_0(x, raw, K)) < F16_REL_TOL
    assert not yw[:, N:].any()
    # output rows that are not 16-byte aligned: single stores, the same values
    ys2 = N + 4 if N % 8 == 0 else N + 3
    dy2 = dev.alloc(M * ys2 * 2)
    dy2.zero()
    capi.check(L().vkl_matmul_q8_0(dx.ptr, dw.ptr, M, N, K, xs, ys2, 1.0, 0.0, 0, None, dy2.ptr, None, dev.stream))
    yw2 = f16(dy2, (M, ys2))
    assert np.array_equal(yw2[:, :N].view(np.uint16), yw[:, :N].view(np.uint16))
    assert not yw2[:, N:].any()


@pytest.mark.parametrize("M,N,K", [(40, 512, 512), (130, 96, 1376), (258, 4200, 64), (130, 5200, 64),
                                   (32, 4096, 4096), (7, 4112, 768), (17, 5120, 1024), (2, 2736, 1024),
                                   (64, 4096, 4096), (45, 4112, 768), (96, 4096, 4096), (70, 4112, 768), (128, 4096, 4096),
                                   (100, 4112, 768)])
def test_kqv_q8_0_many_rows(dev, rng, M, N, K):
    """(the last four: at most 32 token rows and 512 and more groups of 16
    weight rows over the three matrices: workgroups over the whole of K, 3, 4, 4
    and 3 consecutive groups each, also across the end of a matrix; then the same
    form with 64, 45, 96 and 70 token rows, and 128 and 100 in two launches)"""
    ws = [q8_weights(rng, N, K)[0] for _ in range(3)]
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx = dev.upload(x)
    dws = [dev.upload_q8_0(w, N, K) for w in ws]
    outs = [dev.alloc(M * N * 2) for _ in range(3)]
    capi.check(L().vkl_kqv_q8_0(dx.ptr, dws[0].ptr, dws[1].ptr, dws[2].ptr, M, N, K, outs[0].ptr, outs[1].ptr,
                                outs[2].ptr, dev.stream))
    want = O.kqv_q8_0(x, ws[0], ws[1], ws[2], K)
    for o, w in zip(outs, want):
        assert rel_err(f16(o, (M, N)), w) < F16_REL_TOL


@pytest.mark.parametrize("M,N,K", [(33, 1376, 512), (128, 160, 4096), (200, 64, 512), (300, 6200, 128), (200, 7800, 64),
                                   (32, 11008, 4096), (5, 2064, 768), (20, 4112, 1024), (32, 13824, 1280),
                                   (64, 11008, 4096), (40, 2064, 768), (33, 4112, 1024), (48, 13824, 1280), (96, 11008, 4096),
                                   (70, 2064, 768), (100, 8256, 128), (66, 13824, 256), (127, 11008, 512)])
def test_ffn_upgate_q8_0_many_rows(dev, rng, M, N, K):
    """(the last four: at most 32 token rows against 128 and more groups of
    16 row pairs: workgroups over the whole of K with 3, 1, 2 and 4 groups of
    each matrix; then 33 to 64 token rows on the same form with 3, 1 and 2
    groups, on the tile kernel where it would take 4, and 96 and 70 rows in two launches;
    the last three: 65 to 127 rows in one partly empty row of 128-row tiles of the many-row kernel)"""
    up, _ = q8_weights(rng, N, K)
    gate, _ = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dup, dg = dev.upload(x), dev.upload_q8_0(up, N, K), dev.upload_q8_0(gate, N, K)
    out = dev.alloc(M * N * 2)
    capi.check(L().vkl_ffn_upgate_q8_0(dx.ptr, dup.ptr, dg.ptr, M, N, K, out.ptr, dev.stream))
    assert rel_err(f16(out, (M, N)), O.ffn_upgate_q8_0(x, up, gate, K)) < F16_REL_TOL


def test_kqv_q8_0(dev, rng):
    M, N, K = 3, 512, 512
    ws = [q8_weights(rng, N, K)[0] for _ in range(3)]
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx = dev.upload(x)
    dws = [dev.upload_q8_0(w, N, K) for w in ws]
    outs = [dev.alloc(M * N * 2) for _ in range(3)]
    capi.check(L().vkl_kqv_q8_0(dx.ptr, dws[0].ptr, dws[1].ptr, dws[2].ptr, M, N, K, outs[0].ptr, outs[1].ptr,
                                outs[2].ptr, dev.stream))
    want = O.kqv_q8_0(x, ws[0], ws[1], ws[2], K)
    for o, w in zip(outs, want):
        assert rel_err(f16(o, (M, N)), w) < F16_REL_TOL


@pytest.mark.parametrize("M,N,K", [(1, 1376, 512), (4, 300, 256), (1, 11008, 4096)])
def test_ffn_upgate_q8_0(dev, rng, M, N, K):
    up, _ = q8_weights(rng, N, K, 0.005, 0.02)
    gate, _ = q8_weights(rng, N, K, 0.005, 0.02)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dup, dg = dev.upload(x), dev.upload_q8_0(up, N, K), dev.upload_q8_0(gate, N, K)
    out = dev.alloc(M * N * 2)
    capi.check(L().vkl_ffn_upgate_q8_0(dx.ptr, dup.ptr, dg.ptr, M, N, K, out.ptr, dev.stream))
    assert rel_err(f16(out, (M, N)), O.ffn_upgate_q8_0(x, up, gate, K)) < F16_REL_TOL


# ------------------------------------------------------------ fp16 matmul ---
@pytest.mark.parametrize("C,M,N,K", [(1, 9, 9, 128), (8, 1, 300, 64), (4, 7, 50, 128), (1, 1, 512, 4096),
                                     (2, 3, 5, 100), (1, 2, 9, 36)])
def test_matmul_f16_tb(dev, rng, C, M, N, K):
    a = rng.standard_normal((C, M, K)).astype(np.float16)
    b = rng.standard_normal((C, N, K)).astype(np.float16)
    da, db = dev.upload(a), dev.upload(b)
    dy = dev.alloc(C * M * N * 2)
    capi.check(L().vkl_matmul_f16_tb(da.ptr, db.ptr, C, M, N, K, M * K, K, N * K, K, M * N, N, 0.125, 0.0, 0,
                                     None, dy.ptr, None, dev.stream))
    assert rel_err(f16(dy, (C, M, N)), O.matmul_f16_tb(a, b, scale=0.125)) < F16_REL_TOL


@pytest.mark.parametrize("M,N,K", [(16, 130, 512), (100, 200, 1376), (300, 96, 4096), (64, 1376, 512),
                                   (512, 12800, 64), (600, 13000, 96), (600, 13000, 128), (777, 8200, 320),
                                   (256, 24576, 192), (1030, 6144, 448), (300, 6144, 128), (130, 12000, 192), (200, 4096, 2048),
                                   (100, 11392, 128), (66, 12000, 192)])
def test_matmul_f16_tb_many_rows(dev, rng, M, N, K):
    """FP16 weights, many token rows: the matrix-core paths (from about two
    hundred 256 x 128 output tiles on, or half as many 128 x 128 ones, with K a
    multiple of 64, the form that loads its tiles straight into LDS; ragged M
    and N included; (200, 4096, 2048) with its k range split in two; the last
    two: 65 to 127 rows in one partly empty row of 128-row tiles)."""
    a = rng.standard_normal((1, M, K)).astype(np.float16)
    b = (rng.standard_normal((1, N, K)) * 0.05).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    da, db, dr = dev.upload(a), dev.upload(b), dev.upload(res)
    dy, d32 = dev.alloc(M * N * 2), dev.alloc(M * N * 4)
    capi.check(L().vkl_matmul_f16_tb(da.ptr, db.ptr, 1, M, N, K, M * K, K, N * K, K, M * N, N, 1.0, 0.0, 0,
                                     dr.ptr, dy.ptr, d32.ptr, dev.stream))
    prod = O.matmul_f16_tb(a, b)[0]
    want = O.elementwise(prod, res, 0)
    got = f16(dy, (M, N))
    # The product is rounded to fp16 before the residual is added.  Where its
    # fp32 value lies next to a rounding boundary the summation order decides
    # the direction, and a sum that cancels (product 2.5, residual -2.45) then
    # differs by a whole fp16 step of the PRODUCT: the error is measured against
    # the larger of |product| and |result|.
    denom = np.maximum(np.maximum(np.abs(want.astype(np.float64)), np.abs(prod.astype(np.float64))),
                       1e-2 * float(np.abs(want.astype(np.float64)).max()))
    assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / denom)) < F16_REL_TOL
    assert np.array_equal(d32.read(np.float32, (M, N)), got.astype(np.float32))


@pytest.mark.parametrize("M,N,K", [(33, 1376, 512), (130, 96, 4096), (600, 6500, 128), (257, 12300, 256), (200, 6000, 128),
                                   (90, 6000, 128), (127, 11008, 256)])
def test_ffn_upgate_f16_many_rows(dev, rng, M, N, K):
    x = rng.standard_normal((M, K)).astype(np.float16)
    up = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    gate = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    dx, du, dg = dev.upload(x), dev.upload(up), dev.upload(gate)
    out = dev.alloc(M * N * 2)
    capi.check(L().vkl_ffn_upgate_f16(dx.ptr, du.ptr, dg.ptr, M, N, K, out.ptr, dev.stream))
    assert rel_err(f16(out, (M, N)), O.ffn_upgate_f16(x, up, gate)) < F16_REL_TOL


@pytest.mark.parametrize("H,S,Lk,hd,maxlen", [(4, 40, 40, 64, 64), (3, 130, 200, 128, 256), (2, 9, 77, 64, 128)])
def test_attention_products_many_rows(dev, rng, H, S, Lk, hd, maxlen):
    """Prompt-pass attention: scores = Q K^T over a cache view and P V, batched
    over heads on the matrix cores (Lk % 8 != 0 takes the scalar kernel for P V)."""
    q = rng.standard_normal((H, S, hd)).astype(np.float16)
    kc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    vc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    dq, dk, dv = dev.upload(q), dev.upload(kc), dev.upload(vc)
    ds = dev.alloc(H * S * Lk * 2)
    sc = 1.0 / np.sqrt(hd)
    capi.check(L().vkl_matmul_f16_tb(dq.ptr, dk.ptr, H, S, Lk, hd, S * hd, hd, maxlen * hd, hd, S * Lk, Lk,
                                     sc, 0.0, 0, None, ds.ptr, None, dev.stream))
    want_s = O.matmul_f16_tb(q, np.ascontiguousarray(kc[:, :Lk]), scale=sc)
    assert rel_err(f16(ds, (H, S, Lk)), want_s) < F16_REL_TOL
    p = rng.uniform(0, 2.0 / Lk, (H, S, Lk)).astype(np.float16)
    dp, do = dev.upload(p), dev.alloc(H * S * hd * 2)
    capi.check(L().vkl_matmul_f16_nn(dp.ptr, dv.ptr, H, S, hd, Lk, S * Lk, Lk, maxlen * hd, hd, S * hd, hd,
                                     1.0, 0.0, 0, do.ptr, dev.stream))
    want_o = O.matmul_f16_nn(p, np.ascontiguousarray(vc[:, :Lk]))
    assert rel_err(f16(do, (H, S, hd)), want_o) < F16_REL_TOL


@pytest.mark.parametrize("H,S,Lk,hd,maxlen,flat", [
    (8, 40, 40, 64, 64, True), (3, 130, 200, 128, 256, False), (2, 9, 77, 64, 128, True),
    (8, 300, 300, 128, 320, True), (16, 1, 150, 128, 160, True), (8, 257, 385, 64, 512, False)])
def test_attn_prefill_causal(dev, rng, H, S, Lk, hd, maxlen, flat):
    """One-launch prompt attention against the three separate operators of the
    oracle (scores with fp16 rounding, masked softmax, P V).  A score whose
    fp32 value lies next to an fp16 rounding boundary rounds either way
    depending on the summation order of the dot product, which moves one
    probability by 2^-11 relative; the tolerance is therefore 1e-2 relative to
    max(|o|, 0.1 * sum_l p[l] |v[l]|), the size of the terms summed, not to a
    possibly cancelled |o| alone."""
    q = rng.standard_normal((H, S, hd)).astype(np.float16)
    kc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    vc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    kc[:, Lk:] = np.float16(np.nan)   # rows past L must not be touched
    vc[:, Lk:] = np.float16(np.nan)
    dq, dk, dv = dev.upload(q), dev.upload(kc), dev.upload(vc)
    do = dev.alloc(H * S * hd * 2)
    sc = 1.0 / np.sqrt(hd)
    ors, ohs = (H * hd, hd) if flat else (hd, S * hd)
    capi.check(L().vkl_attn_prefill_causal_f16(dq.ptr, dk.ptr, dv.ptr, H, S, Lk, hd, S * hd, hd, maxlen * hd, hd,
                                               maxlen * hd, hd, sc, do.ptr, ors, ohs, dev.stream))
    scores = O.matmul_f16_tb(q, np.ascontiguousarray(kc[:, :Lk]), scale=sc)
    p = O.softmax(scores, True, Lk - S)
    want = O.matmul_f16_nn(p, np.ascontiguousarray(vc[:, :Lk]))
    got = f16(do, (S, H, hd)).transpose(1, 0, 2) if flat else f16(do, (H, S, hd))
    assert np.isfinite(got.astype(np.float32)).all()
    terms = np.einsum("hsl,hld->hsd", p.astype(np.float64), np.abs(vc[:, :Lk].astype(np.float64)))
    denom = np.maximum(np.abs(want.astype(np.float64)), 0.1 * terms)
    assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / denom)) < F16_REL_TOL


def test_matmul_f16_tb_reads_cache_view(dev, rng):
    """scores = Q K^T over the first L rows of a [H, maxlen, hd] cache."""
    H, maxlen, hd, Lk, S = 4, 64, 64, 37, 3
    q = rng.standard_normal((H, S, hd)).astype(np.float16)
    cache = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    dq, dc = dev.upload(q), dev.upload(cache)
    dy = dev.alloc(H * S * Lk * 2)
    capi.check(L().vkl_matmul_f16_tb(dq.ptr, dc.ptr, H, S, Lk, hd, S * hd, hd, maxlen * hd, hd, S * Lk, Lk,
                                     1 / 8.0, 0.0, 0, None, dy.ptr, None, dev.stream))
    want = O.matmul_f16_tb(q, np.ascontiguousarray(cache[:, :Lk]), scale=1 / 8.0)
    assert rel_err(f16(dy, (H, S, Lk)), want) < F16_REL_TOL


@pytest.mark.parametrize("C,M,N,K", [(4, 3, 64, 37), (2, 1, 128, 300), (1, 2, 20, 17)])
def test_matmul_f16_nn(dev, rng, C, M, N, K):
    a = rng.uniform(0, 0.1, (C, M, K)).astype(np.float16)
    b = rng.standard_normal((C, K, N)).astype(np.float16)
    da, db = dev.upload(a), dev.upload(b)
    dy = dev.alloc(C * M * N * 2)
    capi.check(L().vkl_matmul_f16_nn(da.ptr, db.ptr, C, M, N, K, M * K, K, K * N, N, M * N, N, 1.0, 0.0, 0, dy.ptr,
                                     dev.stream))
    assert rel_err(f16(dy, (C, M, N)), O.matmul_f16_nn(a, b)) < F16_REL_TOL


def test_ffn_upgate_f16(dev, rng):
    M, N, K = 2, 300, 512
    x = rng.standard_normal((M, K)).astype(np.float16)
    up = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    gate = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    dx, du, dg = dev.upload(x), dev.upload(up), dev.upload(gate)
    out = dev.alloc(M * N * 2)
    capi.check(L().vkl_ffn_upgate_f16(dx.ptr, du.ptr, dg.ptr, M, N, K, out.ptr, dev.stream))
    assert rel_err(f16(out, (M, N)), O.ffn_upgate_f16(x, up, gate)) < F16_REL_TOL


# ------------------------------------------------- RoPE / KV / softmax ------
@pytest.mark.parametrize("C,H,W,off", [(8, 16, 64, 0), (32, 1, 128, 100), (3, 5, 64, 1019)])
def test_rope_bit_exact(dev, rng, C, H, W, off):
    # tests/test_rope.cpp:211-217 uses offsets 0 / 100 / 1020
    fc, fs = O.rope_tables(1024, W)
    x = rng.standard_normal((C, H, W)).astype(np.float16)
    dx, dfc, dfs = dev.upload(x), dev.upload(fc), dev.upload(fs)
    capi.check(L().vkl_rope_f16(dx.ptr, C, H, W, dfc.ptr, dfs.ptr, off, dev.stream))
    want = O.rope(x, fc, fs, off)
    assert np.array_equal(f16(dx, x.shape).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("S,H,hd,maxlen,off,clip,qpos", [
    (16, 8, 64, 64, 0, False, 0), (5, 3, 128, 256, 100, False, 100), (7, 4, 128, 128, 121, True, 121),
    (7, 4, 64, 128, 9, True, 15)])
def test_rope_kvwrite_bit_exact(dev, rng, S, H, hd, maxlen, off, clip, qpos):
    """RoPE of Q and K plus the cache write on [S, H*hd] projection outputs equals
    Transpose -> Rope -> UpdateKVCache of the oracle bit for bit; with clip only
    the last q row is rotated (at position qpos)."""
    fc, fs = O.rope_tables(maxlen, hd)
    q, k, v = (rng.standard_normal((S, H, hd)).astype(np.float16) for _ in range(3))
    kc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    vc = rng.standard_normal((H, maxlen, hd)).astype(np.float16)
    dq, dk, dv, dkc, dvc = (dev.upload(a) for a in (q, k, v, kc, vc))
    dfc, dfs = dev.upload(fc), dev.upload(fs)
    q_row0, q_rows = (S - 1, 1) if clip else (0, S)
    capi.check(L().vkl_rope_kvwrite_f16(dq.ptr, dk.ptr, dv.ptr, S, H, hd, H * hd, q_row0, q_rows, qpos, off,
                                        dfc.ptr, dfs.ptr, maxlen, dkc.ptr, dvc.ptr, maxlen, dev.stream))
    kt, vt, qt = O.transpose102(k), O.transpose102(v), O.transpose102(q)       # [H, S, hd]
    want_k = O.update_kvcache(kc, O.rope(kt, fc, fs, off), off)
    want_v = O.update_kvcache(vc, vt, off)
    assert np.array_equal(f16(dkc, kc.shape).view(np.uint16), want_k.view(np.uint16))
    assert np.array_equal(f16(dvc, vc.shape).view(np.uint16), want_v.view(np.uint16))
    got_q = f16(dq, q.shape)
    want_q = q.copy()
    rot = O.rope(np.ascontiguousarray(qt[:, q_row0:q_row0 + q_rows]), fc, fs, qpos)  # [H, rows, hd]
    want_q[q_row0:q_row0 + q_rows] = rot.transpose(1, 0, 2)
    assert np.array_equal(got_q.view(np.uint16), want_q.view(np.uint16))
    assert np.array_equal(f16(dk, k.shape), k) and np.array_equal(f16(dv, v.shape), v)


@pytest.mark.parametrize("off", [0, 1022, 500])
def test_kv_update_bit_exact(dev, rng, off):
    C, HO, H, W = 8, 1024, 5, 64
    cache = rng.standard_normal((C, HO, W)).astype(np.float16)
    kv = rng.standard_normal((C, H, W)).astype(np.float16)
    dc, dk = dev.upload(cache), dev.upload(kv)
    capi.check(L().vkl_kv_update_f16(dc.ptr, dk.ptr, C, HO, H, W, off, dev.stream))
    assert np.array_equal(f16(dc, cache.shape), O.update_kvcache(cache, kv, off))


@pytest.mark.parametrize("C,H,W,off,mask", [(8, 16, 16, 0, 1), (32, 1, 289, 288, 1), (2, 5, 70, 64, 1),
                                            (3, 4, 1000, 0, 0)])
def test_softmax(dev, rng, C, H, W, off, mask):
    x = (rng.standard_normal((C, H, W)) * 2).astype(np.float16)
    dx = dev.upload(x)
    out = dev.alloc(x.nbytes)
    capi.check(L().vkl_softmax_f16(dx.ptr, C, H, W, mask, off, out.ptr, dev.stream))
    got, want = f16(out, x.shape), O.softmax(x, mask, off)
    assert np.array_equal(got == 0, want == 0)            # masked entries are exactly zero
    assert rel_err(got, want) < F16_REL_TOL
    assert ulp_diff_f16(got, want).max() <= 1


# ------------------------------------------- element-wise, casts, arg, ... --
def test_elementwise_and_casts_bit_exact(dev, rng):
    n = 5000
    a = rng.standard_normal(n).astype(np.float16)
    b = (rng.standard_normal(n) + 3).astype(np.float16)
    for op in range(4):
        da, db = dev.upload(a), dev.upload(b)
        capi.check(L().vkl_elementwise_f16(da.ptr, db.ptr, n, op, dev.stream))
        assert np.array_equal(f16(db, n).view(np.uint16), O.elementwise(a, b, op).view(np.uint16))
    da = dev.upload(a)
    out = dev.alloc(n * 2)
    capi.check(L().vkl_elementwise_const_f16(da.ptr, 0.5, n, 2, out.ptr, dev.stream))
    assert np.array_equal(f16(out, n), (a.astype(np.float32) * np.float32(0.5)).astype(np.float16))
    o32 = dev.alloc(n * 4)
    capi.check(L().vkl_cast_f16_f32(da.ptr, o32.ptr, n, dev.stream))
    assert np.array_equal(o32.read(np.float32, n), a.astype(np.float32))
    f = rng.standard_normal(n).astype(np.float32)
    df = dev.upload(f)
    capi.check(L().vkl_cast_f32_f16(df.ptr, out.ptr, n, dev.stream))
    assert np.array_equal(f16(out, n), f.astype(np.float16))


def test_argop_bit_exact(dev, rng):
    rows, W = 7, 32000
    x = rng.standard_normal((rows, W)).astype(np.float16)
    x[2, 17] = x[2, 25000] = 30.0
    x[4, :] = -1.0
    x[5, 31999] = 50.0
    dx = dev.upload(x)
    out = dev.alloc(rows * 4)
    capi.check(L().vkl_argop_f16(dx.ptr, rows, W, 0, out.ptr, dev.stream))
    assert list(out.read(np.uint32, rows)) == list(O.argmax_f16(x))
    capi.check(L().vkl_argop_f16(dx.ptr, rows, W, 1, out.ptr, dev.stream))
    assert list(out.read(np.uint32, rows)) == list(np.argmin(x.astype(np.float32), axis=1))


def test_slice_and_transpose_bit_exact(dev, rng):
    C, H, W = 5, 9, 40
    x = rng.standard_normal((C, H, W)).astype(np.float16)
    dx = dev.upload(x)
    out = dev.alloc(x.nbytes)
    capi.check(L().vkl_slice_f16(dx.ptr, C, H, W, 1, 2, 3, 3, 4, 30, out.ptr, dev.stream))
    assert np.array_equal(f16(out, (3, 4, 30)), x[1:4, 2:6, 3:33])
    capi.check(L().vkl_transpose102_f16(dx.ptr, C, H, W, out.ptr, dev.stream))
    assert np.array_equal(f16(out, (H, C, W)), O.transpose102(x))


def test_invalid_arguments_are_rejected_before_launch(dev):
    buf = dev.alloc(1024)
    assert L().vkl_slice_f16(buf.ptr, 2, 2, 2, 1, 0, 0, 2, 1, 1, buf.ptr, dev.stream) == 1   # c0+CE > C
    assert L().vkl_rope_f16(buf.ptr, 1, 1, 3, buf.ptr, buf.ptr, 0, dev.stream) == 1          # odd width
    assert L().vkl_kv_update_f16(buf.ptr, buf.ptr, 1, 2, 3, 4, 0, dev.stream) == 1           # kv longer than cache
    assert L().vkl_matmul_q8_0(buf.ptr, buf.ptr, 1, 4, 32, 16, 4, 1.0, 0.0, 0, None, buf.ptr, None,
                               dev.stream) == 1                                              # row stride < K
    dev.sync()


# ------------------------------------------------- Concat / ReadKVCache / Reduce
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_concat_parts_bit_exact(dev, rng, axis):
    """tests/test_concat.cpp of the reference: inputs joined along one axis."""
    shapes = [[3, 5, 16], [3, 5, 16], [3, 5, 16]]
    shapes[1][axis] += 4
    shapes[2][axis] = 1
    xs = [rng.standard_normal(sh).astype(np.float16) for sh in shapes]
    want = np.concatenate(xs, axis=axis)
    OC, OH, OW = want.shape
    out = dev.alloc(want.nbytes)
    off = 0
    for x in xs:
        Cc, H, W = x.shape
        capi.check(L().vkl_concat_part_f16(dev.upload(x).ptr, Cc, H, W, H * W, W, out.ptr, OH * OW, OW, off, dev.stream))
        off += (Cc * OH * OW, H * OW, W)[axis]
    assert np.array_equal(f16(out, want.shape).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("off,n", [(0, 16), (13, 6), (31, 16), (5, 1)])
def test_read_kvcache_bit_exact(dev, rng, off, n):
    C_, H, W = 4, 16, 64
    cache = rng.standard_normal((C_, H, W)).astype(np.float16)
    out = dev.alloc(C_ * n * W * 2)
    capi.check(L().vkl_read_kvcache_f16(dev.upload(cache).ptr, C_, H, W, off, n, out.ptr, dev.stream))
    want = cache[:, (np.arange(n) + off) % H]
    assert np.array_equal(f16(out, want.shape).view(np.uint16), want.view(np.uint16))
    assert L().vkl_read_kvcache_f16(dev.upload(cache).ptr, C_, H, W, 0, H + 1, out.ptr, dev.stream) != 0


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("shape", [(3, 7, 300), (1, 1, 5), (2, 64, 4096)])
def test_reduce_last_axis(dev, rng, op, shape):
    """tests/test_reduce.cpp of the reference (tolerance 1e-2); max and min are exact."""
    x = rng.standard_normal(shape).astype(np.float16)
    out = dev.alloc(shape[0] * shape[1] * 2)
    capi.check(L().vkl_reduce_f16(dev.upload(x).ptr, *shape, op, out.ptr, dev.stream))
    got = f16(out, shape[:2]).astype(np.float64)
    x64 = x.astype(np.float64)
    want = (x64.sum(-1), x64.max(-1), x64.min(-1), x64.mean(-1))[op]
    if op in (1, 2):
        assert np.array_equal(got, want)
    else:
        scale = np.abs(x64).sum(-1) / (shape[2] if op == 3 else 1)
        assert np.all(np.abs(got - want) <= 1e-2 * np.maximum(np.abs(want), 0.1 * scale) + 1e-3)



# ------------------------------------ full sizes, through exact properties ---
def test_q8_roundtrip_full_size(dev, rng):
    """The 7B down-projection matrix (4096 x 11008): GGUF blocks -> planar
    device layout -> GGUF blocks, bit for bit."""
    rows, K = 4096, 11008
    raw, _ = q8_weights(rng, rows, K)
    staging = dev.upload(raw)
    planar = dev.alloc(raw.nbytes)
    back = dev.alloc(raw.nbytes)
    capi.check(L().vkl_q8_0_pack(staging.ptr, planar.ptr, rows, K, dev.stream))
    capi.check(L().vkl_q8_0_unpack(planar.ptr, back.ptr, rows, K, dev.stream))
    assert np.array_equal(back.read(np.uint8, raw.shape), raw)


@pytest.mark.parametrize("M", [1, 20, 48, 200, 1024])
@pytest.mark.parametrize("N,K", [(4096, 4096), (4096, 11008)])
def test_matmul_q8_0_full_size_scaling_and_rows(dev, rng, M, N, K):
    """7B shapes on every product kernel (one row: the decode step's streaming
    kernel; few rows; tiles with and without the k-split).  Doubling x doubles
    every product, sum and (normal) rounded result exactly, so y(2x) must equal
    2 y(x) bit for bit; and a row's result does not depend on the other rows of the
    call (the same row alone, on the same kernel family, gives the same bits)."""
    raw, _ = q8_weights(rng, N, K, 0.002, 0.006)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dw = dev.upload_q8_0(raw, N, K)

    def run(xx):
        dx = dev.upload(xx)
        dy = dev.alloc(xx.shape[0] * N * 2)
        capi.check(L().vkl_matmul_q8_0(dx.ptr, dw.ptr, xx.shape[0], N, K, K, N, 1.0, 0.0, 0,
                                       None, dy.ptr, None, dev.stream))
        return f16(dy, (xx.shape[0], N)).copy()

    y1 = run(x)
    y2 = run((x * np.float16(2)).astype(np.float16))
    assert np.isfinite(y1.astype(np.float32)).all()
    # (a subnormal fp16 result has a fixed absolute precision: doubling the
    # exact value may round the other way there, within one unit)
    normal = np.abs(y1.astype(np.float32)) >= 2.0 ** -14
    d = (y1 * np.float16(2)).view(np.uint16).astype(np.int32) - y2.view(np.uint16).astype(np.int32)
    assert not d[normal].any()
    assert np.abs(d[~normal]).max(initial=0) <= 1
    # permuting the rows of x permutes the rows of y
    perm = rng.permutation(M)
    assert np.array_equal(run(x[perm]).view(np.uint16), y1[perm].view(np.uint16))


@pytest.mark.parametrize("M", [1, 32, 300])
def test_kqv_q8_0_full_size_scaling(dev, rng, M):
    """Fused K/Q/V projection at the 7B width: y(2x) = 2 y(x) bit for bit
    (normal results) for all three outputs."""
    N = K = 4096
    dws = [dev.upload_q8_0(q8_weights(rng, N, K, 0.002, 0.006)[0], N, K) for _ in range(3)]
    x = rng.standard_normal((M, K)).astype(np.float16)

    def run(xx):
        dx = dev.upload(xx)
        outs = [dev.alloc(M * N * 2) for _ in range(3)]
        capi.check(L().vkl_kqv_q8_0(dx.ptr, dws[0].ptr, dws[1].ptr, dws[2].ptr, M, N, K, outs[0].ptr,
                                    outs[1].ptr, outs[2].ptr, dev.stream))
        return [f16(o, (M, N)).copy() for o in outs]

    for y1, y2 in zip(run(x), run((x * np.float16(2)).astype(np.float16))):
        normal = np.abs(y1.astype(np.float32)) >= 2.0 ** -14
        d = (y1 * np.float16(2)).view(np.uint16).astype(np.int32) - y2.view(np.uint16).astype(np.int32)
        assert not d[normal].any()
        assert np.abs(d[~normal]).max(initial=0) <= 1


def test_attn_prefill_causal_full_size_is_causal(dev, rng):
    """Prompt attention at 32 heads x 1024 positions x 128: the output of a
    position depends on nothing behind it.  Changing q, k and v from position
    700 on must leave the outputs of positions 0..699 bit for bit."""
    H, S, hd, cut = 32, 1024, 128, 700
    sc = 1.0 / np.sqrt(hd)

    def run(q, k, v):
        dq, dk, dv = dev.upload(q), dev.upload(k), dev.upload(v)
        do = dev.alloc(H * S * hd * 2)
        capi.check(L().vkl_attn_prefill_causal_f16(dq.ptr, dk.ptr, dv.ptr, H, S, S, hd, S * hd, hd, S * hd, hd,
                                                   S * hd, hd, sc, do.ptr, hd, S * hd, dev.stream))
        return f16(do, (H, S, hd)).copy()

    q, k, v = (rng.standard_normal((H, S, hd)).astype(np.float16) for _ in range(3))
    a = run(q, k, v)
    q2, k2, v2 = q.copy(), k.copy(), v.copy()
    for t in (q2, k2, v2):
        t[:, cut:] = rng.standard_normal((H, S - cut, hd)).astype(np.float16)
    b = run(q2, k2, v2)
    assert np.isfinite(a.astype(np.float32)).all()
    assert np.array_equal(a[:, :cut].view(np.uint16), b[:, :cut].view(np.uint16))
    assert not np.array_equal(a[:, cut:].view(np.uint16), b[:, cut:].view(np.uint16))
