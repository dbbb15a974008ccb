"""vkl_matmul_q8_0_noalloc: the Q8_0 product for callers that cannot allocate
device memory.  Its partial sums go through the library's static device array
instead of an allocated workspace; kernels and results are those of
vkl_matmul_q8_0, so the outputs must agree bit for bit -- on two calls in a
row, the second with a smaller input (the array keeps the first call's
contents), and on a many-row problem that takes the k-split tile kernel.
Problems whose partial sums exceed the array are refused."""
import numpy as np
import pytest

from util import q8_weights
from vkllama_amd import capi

pytestmark = pytest.mark.gpu

HIP_ERROR_INVALID_VALUE = 1


def f16(buf, shape):
    return buf.read(np.uint16, shape).view(np.float16)


def _both(dev, rng, M, N, K, residual=False):
    L = capi.lib()
    raw, _ = q8_weights(rng, N, K, 0.002, 0.006)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dw = dev.upload(x), dev.upload_q8_0(raw, N, K)
    res = rng.standard_normal((M, N)).astype(np.float16) if residual else None
    dr = dev.upload(res) if residual else None
    out = []
    for fn in (L.vkl_matmul_q8_0, L.vkl_matmul_q8_0_noalloc):
        dy = dev.alloc(M * N * 2)
        dy.zero()
        capi.check(fn(dx.ptr, dw.ptr, M, N, K, K, N, 1.0, 0.0, 0, dr.ptr if dr else None, dy.ptr, None,
                      dev.stream), fn.__name__)
        out.append(f16(dy, (M, N)).copy())
    return out


def test_noalloc_equals_the_allocating_entry_point_on_two_calls_in_a_row(dev, rng):
    # few-row kernel with K slices: 20 rows against a 2048 x 4096 matrix (2.1 MB of partial sums; with 4096 rows
    # and more the workgroups run over the whole of K and need no scratch) ...
    a, b = _both(dev, rng, 20, 2048, 4096)
    assert np.isfinite(a.astype(np.float32)).all() and a.any()
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    # ... then a smaller problem over the same scratch, with the residual epilogue
    a, b = _both(dev, rng, 7, 1024, 512, residual=True)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    # the tile kernel with its k range split (100 rows: 3.3 MB of partial tiles)
    a, b = _both(dev, rng, 100, 4096, 1024)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    # one row needs no scratch, nor do few rows against many weight rows
    a, b = _both(dev, rng, 1, 4096, 4096)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    a, b = _both(dev, rng, 20, 4096, 4096, residual=True)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_noalloc_refuses_what_does_not_fit(dev, rng):
    # 32 rows x 32000 columns x 4 slices of K: 16 MB of partial sums > 8 MiB (32 MB with slices of 512)
    M, N, K = 32, 32000, 4096
    raw, _ = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dw, dy = dev.upload(x), dev.upload_q8_0(raw, N, K), dev.alloc(M * N * 2)
    rc = capi.lib().vkl_matmul_q8_0_noalloc(dx.ptr, dw.ptr, M, N, K, K, N, 1.0, 0.0, 0, None, dy.ptr, None,
                                            dev.stream)
    assert rc == HIP_ERROR_INVALID_VALUE
