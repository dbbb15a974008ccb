"""vkl_matmul_q8_0_noalloc: the Q8_0 product for callers that cannot allocate
device memory.  Its partial sums go through the library's static device array
instead of an allocated workspace; kernels and results are those of
vkl_matmul_q8_0.

What is pinned here, per kernel family that uses scratch (the two whole-line
few-row kernels, the k-split tile kernel and the k-split direct-to-LDS kernel;
the few-row kernel with slices of 1024 takes Q8_0 weights only where the
whole-line form's sums exceed 64 MiB, far beyond the static array): the no-allocation call comes FIRST, on a fresh stream
that has never run a product (so no per-stream workspace exists yet); free
device memory is the same before and after it; the static array, marked with a
pattern beforehand, has been written; and the output equals that of the
allocating entry point bit for bit -- also on a second, smaller call over the
same array.  Problems whose partial sums exceed the array are refused."""
import ctypes as C

import numpy as np
import pytest

from util import q8_weights
from vkllama_amd import capi

pytestmark = pytest.mark.gpu

HIP_ERROR_INVALID_VALUE = 1
SCRATCH = 8 << 20


def f16(buf, shape):
    return buf.read(np.uint16, shape).view(np.float16)


def free_bytes():
    f, t = C.c_size_t(0), C.c_size_t(0)
    capi.check(capi.lib().vkl_mem_info(C.byref(f), C.byref(t)), "vkl_mem_info")
    return f.value


def static_scratch():
    p, n = C.c_void_p(), C.c_size_t(0)
    capi.check(capi.lib().vkl_debug_static_scratch(C.byref(p), C.byref(n)), "vkl_debug_static_scratch")
    assert n.value == SCRATCH
    return p


def plan(M, N, K, workspace):
    p = capi.GemmPlan()
    capi.check(capi.lib().vkl_gemm_plan(M, N, K, 8, 1, 0, workspace, C.byref(p)), "vkl_gemm_plan")
    return p


def _noalloc_then_alloc(dev, rng, M, N, K, family, residual=False):
    """The no-allocation call on a stream of its own, checked for what it
    must not do, then the allocating call; returns both outputs."""
    L = capi.lib()
    p = plan(M, N, K, SCRATCH)
    assert p.family == family, (p.family, family)
    own = plan(M, N, K, 0)      # the allocating entry point's plan: the same kernels and split
    assert (own.family, own.tile_rows, own.ksplit) == (p.family, p.tile_rows, p.ksplit)
    raw, _ = q8_weights(rng, N, K, 0.002, 0.006)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dw = dev.upload(x), dev.upload_q8_0(raw, N, K)
    res = rng.standard_normal((M, N)).astype(np.float16) if residual else None
    dr = dev.upload(res) if residual else None
    dy0, dy1 = dev.alloc(M * N * 2), dev.alloc(M * N * 2)
    dy0.zero(), dy1.zero()
    probe = dev.alloc(64)
    scratch = static_scratch()
    # mark the head of the static array: partial sums of the first output
    # columns land there in every family
    capi.check(L.vkl_memset(scratch, 0xA5, 4096, dev.stream), "vkl_memset")
    dev.sync()
    fresh = C.c_void_p()
    capi.check(L.vkl_stream_create(C.byref(fresh)), "vkl_stream_create")
    before = free_bytes()
    capi.check(L.vkl_matmul_q8_0_noalloc(dx.ptr, dw.ptr, M, N, K, K, N, 1.0, 0.0, 0, dr.ptr if dr else None,
                                         dy0.ptr, None, fresh), "vkl_matmul_q8_0_noalloc")
    capi.check(L.vkl_stream_sync(fresh), "vkl_stream_sync")
    after = free_bytes()
    assert after == before, "the no-allocation entry point changed free device memory by %d bytes" % (before - after)
    if p.workspace_bytes:
        capi.check(L.vkl_memcpy_d2d(probe.ptr, scratch, 64, dev.stream), "vkl_memcpy_d2d")
        head = probe.read(np.uint8, (64,))
        assert not np.all(head == 0xA5), "the static scratch array was not written"
    capi.check(L.vkl_stream_destroy(fresh), "vkl_stream_destroy")
    capi.check(L.vkl_matmul_q8_0(dx.ptr, dw.ptr, M, N, K, K, N, 1.0, 0.0, 0, dr.ptr if dr else None, dy1.ptr, None,
                                 dev.stream), "vkl_matmul_q8_0")
    return f16(dy0, (M, N)).copy(), f16(dy1, (M, N)).copy()


# kernel families of vkl_gemm_plan
ROWSFULL, ROWS128, ROWS64, SLICES, WIDE, TILE, STREAM = 1, 2, 3, 4, 5, 6, 7


@pytest.mark.parametrize("M,N,K,family,residual", [
    (20, 2048, 4096, ROWS128, False),    # whole-line few-row kernel, four independent waves (K % 256 == 0)
    (7, 1024, 544, ROWS64, True),        # whole-line few-row kernel, K not a multiple of 256; smaller, after the first
    (100, 4096, 1024, TILE, True),       # tile kernel with its k range split
    (128, 4096, 4096, WIDE, False),      # direct-to-LDS kernel with its k range split (8 MiB of partial tiles)
    (1, 4096, 4096, STREAM, False),      # one row: no scratch
    (20, 4096, 4096, ROWSFULL, True),    # few rows against many weight rows: no scratch
])
def test_noalloc_allocates_nothing_uses_the_static_array_and_equals_the_allocating_call(dev, rng, M, N, K, family,
                                                                                        residual):
    a, b = _noalloc_then_alloc(dev, rng, M, N, K, family, residual)
    assert np.isfinite(a.astype(np.float32)).all() and a.any()
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


@pytest.mark.parametrize("M,N,K", [(32, 32000, 4096),    # 32 MB of partial sums (8 slices of 512)
                                   (24, 9000, 4096)])    # 9.2 MB: just beyond the array
def test_noalloc_refuses_what_does_not_fit(dev, rng, M, N, K):
    """The allocating entry point's plan for these problems needs more scratch
    than the static array holds.  They are refused, not run on another kernel:
    the results would no longer be those of vkl_matmul_q8_0 bit for bit."""
    assert plan(M, N, K, 0).workspace_bytes > SCRATCH
    raw, _ = q8_weights(rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dx, dw, dy = dev.upload(x), dev.upload_q8_0(raw, N, K), dev.alloc(M * N * 2)
    rc = capi.lib().vkl_matmul_q8_0_noalloc(dx.ptr, dw.ptr, M, N, K, K, N, 1.0, 0.0, 0, None, dy.ptr, None,
                                            dev.stream)
    assert rc == HIP_ERROR_INVALID_VALUE
