"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and its host-only entry points agree with the oracle.  No
kernel is launched here."""
import os
import re

import numpy as np

import ctypes as C

from oracle import oracle as O
from vkllama_amd import capi, model as M

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vkl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared("vkl_hip.h")
    assert len(names) > 40
    lib = capi.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.SIGNATURES) == names               # the binding covers the header, no more, no less


def test_decode_header_symbols_are_exported():
    names = _declared("vkl_decode.h")
    assert "vkl_decode_step" in names and "vkl_decode_phase_replay" in names
    raw = C.CDLL(capi.HIP_LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n


def test_model_header_symbols_are_exported_and_bound():
    names = _declared("vkl_model.h")
    lib = M.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(M.SIGNATURES) == names


def test_model_capi_rejects_bad_arguments_without_a_gpu():
    """Argument checks that come before any device call (absl status codes)."""
    lib = M.lib()
    INVALID_ARGUMENT = 3
    out = C.c_void_p()
    assert lib.vkl_model_create(0, None, None, 0, C.byref(out)) == INVALID_ARGUMENT
    logits = np.zeros(4, np.float32)
    toks = np.zeros(1, np.uint32)
    assert lib.vkl_model_forward(None, toks.ctypes.data, 1, 0, logits.ctypes.data) == INVALID_ARGUMENT
    assert lib.vkl_model_set_option(None, b"fused_decode", 1) == INVALID_ARGUMENT
    assert lib.vkl_model_vocab(None) == 0
    assert lib.vkl_model_decode_step_bytes(None, 5) == 0
    assert lib.vkl_model_last_error(None) == b"null model"
    lib.vkl_model_destroy(None)                           # a no-op


def test_synthetic_weight_generator_is_counter_based():
    """Element i of a stream depends on (seed, i) only: any slice can be
    regenerated on its own, rows of a Q8_0 matrix equal the quantised fp32
    stream, and the moments are those of N(0, std)."""
    lib = M.lib()
    n = 1 << 16
    a = np.empty(n, np.float32)
    lib.vkl_synth_normal_f32(77, n, 0.02, a.ctypes.data)
    b = np.empty(n // 2, np.float32)
    lib.vkl_synth_normal_f32(77, n // 2, 0.02, b.ctypes.data)
    assert np.array_equal(a[:n // 2], b)
    c = np.empty(n, np.float32)
    lib.vkl_synth_normal_f32(78, n, 0.02, c.ctypes.data)
    assert not np.array_equal(a, c)
    assert abs(a.mean()) < 5e-4 and abs(a.std() - 0.02) < 5e-4
    assert abs(float(np.mean(a ** 4)) / a.var() ** 2 - 3.0) < 0.15      # kurtosis of a normal
    h = np.empty(n, np.uint16)
    lib.vkl_synth_normal_f16(77, n, 0.02, h.ctypes.data)
    assert np.array_equal(h.view(np.float16), a.astype(np.float16))
    rows, K = 8, 96
    raw = np.empty(rows * capi.lib().vkl_q8_0_row_bytes(K), np.uint8)
    lib.vkl_synth_normal_q8_0(77, rows, K, 0.02, raw.ctypes.data)
    want = O.quantize_q8_0(a[:rows * K].reshape(rows, K), 2)
    assert np.array_equal(raw.reshape(rows, -1), want)


def test_host_quantizer_bit_exact_vs_oracle(rng):
    x = np.concatenate([rng.uniform(-5, 5, 4096 + 95), np.zeros(32), [127.0, 0.5, -0.5, 2.5, -2.5, 126.5]]
                       ).astype(np.float32)
    n = x.size
    out = np.empty(capi.lib().vkl_q8_0_row_bytes(n), np.uint8)
    capi.lib().vkl_quantize_q8_0_h(x.ctypes.data, n, out.ctypes.data)
    want = O.quantize_q8_0(x[None, :], 2)[0]
    assert np.array_equal(out, want)
    back = np.empty(n, np.float32)
    capi.lib().vkl_dequantize_q8_0_h(out.ctypes.data, n, back.ctypes.data)
    assert np.array_equal(back, O.dequantize_q8_0(want[None, :], n, 2)[0])


