"""Which kernel a matrix product of the prompt pass runs on.

Five kernel families sit behind the launchers of include/vkl_hip.h, chosen by
row count, shape and scratch size.  Parity tests reach each family by choosing
shapes, but they cannot tell when a changed threshold sends a real workload to
a slower family: the results stay right.  This table pins the choice for the
Llama-2 7B and 13B shapes (the four products of a block, Q8_0 and FP16
weights) over the row counts at which the families hand over.  It is read from
vkl_gemm_plan, the host function the launchers themselves follow; no GPU is
needed.  A deliberate change of a threshold changes this table with it.

Entry: family:tile_rows/ksplit/launches; families: 1 whole-K workgroups, 2 / 3
/ 4 K slices + a reduction launch, 5 direct-to-LDS tiles, 6 the general tile
kernel, 7 one weight-streaming pass per token row.
"""
import ctypes as C

import pytest

from vkllama_amd import capi


Plan = capi.GemmPlan

ROWS = [1, 2, 32, 33, 64, 65, 96, 97, 127, 128, 512, 2048, 3968]
SHAPES = {"7b": (4096, 11008), "13b": (5120, 13824)}

EXPECTED = {
    ("7b", 8, "kqv"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:96/1/1 1:96/1/1 1:96/1/2 1:96/1/2 1:96/1/2 5:256/1/1 5:256/1/1 5:256/1/1",
    ("7b", 8, "wo"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:96/1/1 1:96/1/1 5:128/4/2 5:128/4/2 5:128/4/2 5:128/2/2 5:256/1/1 5:256/1/1",
    ("7b", 8, "upgate"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:64/1/2 1:64/1/2 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1 5:256/1/1",
    ("7b", 8, "down"): "7:1/1/1 2:32/22/2 2:32/22/2 6:64/8/2 6:64/8/2 6:64/8/2 6:64/8/2 6:64/8/2 6:64/8/2 5:128/4/2 5:256/4/2 5:256/1/1 5:256/1/1",
    ("7b", 1, "kqv"): "7:1/1/1 7:1/1/2 4:32/4/2 6:64/5/2 6:64/5/2 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1 5:256/1/1",
    ("7b", 1, "wo"): "7:1/1/1 7:1/1/2 4:32/4/2 6:64/8/2 6:64/8/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/2/2 5:256/1/1 5:256/1/1",
    ("7b", 1, "upgate"): "7:1/1/1 7:1/1/2 4:32/4/2 6:64/1/1 6:64/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1",
    ("7b", 1, "down"): "7:1/1/1 7:1/1/2 4:32/11/2 6:64/8/2 6:64/8/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/2/2 5:256/1/1 5:256/1/1",
    ("13b", 8, "kqv"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:96/1/1 1:96/1/1 1:96/1/2 1:96/1/2 1:96/1/2 5:256/1/1 5:256/1/1 5:256/1/1",
    ("13b", 8, "wo"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:96/1/1 1:96/1/1 1:96/1/2 1:96/1/2 1:96/1/2 5:256/2/2 5:256/1/1 5:256/1/1",
    ("13b", 8, "upgate"): "7:1/1/1 1:32/1/1 1:32/1/1 6:64/2/2 6:64/2/2 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1 5:256/1/1",
    ("13b", 8, "down"): "7:1/1/1 1:32/1/1 1:32/1/1 1:64/1/1 1:64/1/1 1:96/1/1 1:96/1/1 1:96/1/2 1:96/1/2 1:96/1/2 5:256/2/2 5:256/1/1 5:256/1/1",
    ("13b", 1, "kqv"): "7:1/1/1 7:1/1/2 4:32/5/2 6:64/4/2 6:64/4/2 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1 5:256/1/1",
    ("13b", 1, "wo"): "7:1/1/1 7:1/1/2 4:32/5/2 6:64/8/2 6:64/8/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/1/1 5:128/1/1 5:128/1/1",
    ("13b", 1, "upgate"): "7:1/1/1 7:1/1/2 4:32/5/2 6:64/1/1 6:64/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:128/1/1 5:256/1/1 5:256/1/1 5:256/1/1",
    ("13b", 1, "down"): "7:1/1/1 7:1/1/2 4:32/14/2 6:64/8/2 6:64/8/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:128/4/2 5:256/2/2 5:128/1/1 5:128/1/1",
}


def plan(M, N, K, wtype, nmat=1, upgate=0, workspace=0):
    lib = capi.lib()
    p = Plan()
    assert lib.vkl_gemm_plan(M, N, K, wtype, nmat, upgate, workspace, C.byref(p)) == 0
    return p


def product(model, name):
    dim, ffn = SHAPES[model]
    return {"kqv": (dim, dim, 3, 0), "wo": (dim, dim, 1, 0), "upgate": (ffn, dim, 1, 1),
            "down": (dim, ffn, 1, 0)}[name]


@pytest.mark.parametrize("key", sorted(EXPECTED))
def test_kernel_family_per_llama_shape_and_row_count(key):
    model, wtype, name = key
    N, K, nmat, upgate = product(model, name)
    got = []
    for M in ROWS:
        p = plan(M, N, K, wtype, nmat, upgate)
        got.append("%d:%d/%d/%d" % (p.family, p.tile_rows, p.ksplit, p.launches))
    assert " ".join(got) == EXPECTED[key]


def test_the_plan_is_what_the_workspace_query_and_the_launcher_share():
    """Partial sums never exceed the scratch the plan was made for: the
    library's own 64 MiB, or a caller's (8 MiB for the no-allocation entry
    point); a smaller scratch means fewer parts or another family, never an
    overrun."""
    for model in SHAPES:
        for name in ("kqv", "wo", "upgate", "down"):
            N, K, nmat, upgate = product(model, name)
            for wtype in (8, 1):
                for M in ROWS[1:]:
                    own = plan(M, N, K, wtype, nmat, upgate)
                    assert own.workspace_bytes <= 64 << 20
                    assert (own.ksplit > 1) == (own.workspace_bytes > 0)
                    small = plan(M, N, K, wtype, nmat, upgate, workspace=8 << 20)
                    assert small.workspace_bytes <= 8 << 20, (model, name, wtype, M)
                    assert small.family != 0
                    assert small.launches == (2 if small.ksplit > 1 else small.launches)


def test_single_rows_stream_and_bad_arguments_are_refused():
    p = plan(1, 4096, 4096, 8)
    assert (p.family, p.launches) == (7, 1)
    p = plan(2, 4096, 4096, 1)      # fp16 weights: the matrix cores take over from 3 rows
    assert (p.family, p.launches) == (7, 2)
    lib = capi.lib()
    q = Plan()
    assert lib.vkl_gemm_plan(0, 4096, 4096, 8, 1, 0, 0, C.byref(q)) != 0
    assert lib.vkl_gemm_plan(4, 4096, 4096, 5, 1, 0, 0, C.byref(q)) != 0
    assert lib.vkl_gemm_plan(4, 4096, 4096, 8, 2, 0, 0, C.byref(q)) != 0
    assert lib.vkl_gemm_plan(4, 4096, 4096, 8, 3, 1, 0, C.byref(q)) != 0
