"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and its host-only entry points agree with the oracle.  No
kernel is launched here."""
import os
import re

import numpy as np

from oracle import oracle as O
from vkllama_amd import capi

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


