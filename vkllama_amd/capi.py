"""ctypes binding of the C ABI in include/vkl_hip.h (libvkllama_hip.so).

There is no CPU fallback: if the library is missing, or a call returns a
non-zero hipError_t, an exception is raised.
"""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# VKL_LIB_DIR: another directory holding a build of both libraries (comparing two builds on one GPU)
LIB_DIR = os.environ.get("VKL_LIB_DIR", os.path.join(_PKG, "lib"))
HIP_LIB_PATH = os.path.join(LIB_DIR, "libvkllama_hip.so")

vp = C.c_void_p
sz = C.c_size_t
u32 = C.c_uint32
u64 = C.c_uint64
f32 = C.c_float
i32 = C.c_int


class DeviceInfo(C.Structure):
    _fields_ = [("device", i32), ("compute_units", i32), ("wavefront_size", i32), ("max_lds_bytes", i32),
                ("total_mem", sz), ("name", C.c_char * 128), ("arch", C.c_char * 64)]


# name -> (restype, argtypes); every symbol include/vkl_hip.h declares
class GemmPlan(C.Structure):
    """vkl_gemm_plan_t of include/vkl_hip.h"""
    _fields_ = [("family", C.c_int), ("tile_rows", C.c_int), ("ksplit", C.c_int), ("groups", C.c_int),
                ("launches", C.c_int), ("workspace_bytes", C.c_size_t)]


SIGNATURES = {
    "vkl_device_count": (i32, [C.POINTER(i32)]),
    "vkl_device_open": (i32, [i32, C.POINTER(DeviceInfo)]),
    "vkl_error_string": (C.c_char_p, [i32]),
    "vkl_stream_create": (i32, [C.POINTER(vp)]),
    "vkl_stream_destroy": (i32, [vp]),
    "vkl_stream_sync": (i32, [vp]),
    "vkl_device_sync": (i32, []),
    "vkl_malloc": (i32, [C.POINTER(vp), sz]),
    "vkl_free": (i32, [vp]),
    "vkl_host_malloc_h": (i32, [C.POINTER(vp), sz]),
    "vkl_host_free_h": (i32, [vp]),
    "vkl_memcpy_h2d": (i32, [vp, vp, sz, vp]),
    "vkl_memcpy_d2h": (i32, [vp, vp, sz, vp]),
    "vkl_memcpy_d2d": (i32, [vp, vp, sz, vp]),
    "vkl_memset": (i32, [vp, i32, sz, vp]),
    "vkl_copy_kernel": (i32, [vp, vp, sz, vp]),
    "vkl_event_create": (i32, [C.POINTER(vp)]),
    "vkl_event_destroy": (i32, [vp]),
    "vkl_event_record": (i32, [vp, vp]),
    "vkl_event_sync": (i32, [vp]),
    "vkl_event_elapsed_ms": (i32, [vp, vp, C.POINTER(f32)]),
    "vkl_quantize_q8_0_h": (None, [vp, sz, vp]),
    "vkl_dequantize_q8_0_h": (None, [vp, sz, vp]),
    "vkl_q8_0_row_bytes": (sz, [sz]),
    "vkl_q8_0_pack": (i32, [vp, vp, sz, sz, vp]),
    "vkl_q8_0_unpack": (i32, [vp, vp, sz, sz, vp]),
    "vkl_embed_q8_0": (i32, [vp, u32, u32, vp, u32, u32, vp, vp]),
    "vkl_embed_f16": (i32, [vp, u32, u32, vp, u32, u32, vp, vp]),
    "vkl_rmsnorm_f16": (i32, [vp, vp, i32, i32, f32, vp, vp]),
    "vkl_matmul_q8_0": (i32, [vp, vp, i32, i32, i32, sz, sz, f32, f32, i32, vp, vp, vp, vp]),
    "vkl_matmul_q8_0_noalloc": (i32, [vp, vp, i32, i32, i32, sz, sz, f32, f32, i32, vp, vp, vp, vp]),
    "vkl_mem_info": (i32, [C.POINTER(sz), C.POINTER(sz)]),
    "vkl_debug_static_scratch": (i32, [C.POINTER(vp), C.POINTER(sz)]),
    "vkl_gemm_plan": (i32, [i32, i32, i32, i32, i32, i32, sz, C.POINTER(GemmPlan)]),
    "vkl_kqv_q8_0": (i32, [vp, vp, vp, vp, i32, i32, i32, vp, vp, vp, vp]),
    "vkl_ffn_upgate_q8_0": (i32, [vp, vp, vp, i32, i32, i32, vp, vp]),
    "vkl_rope_kvwrite_f16": (i32, [vp, vp, vp, i32, i32, i32, sz, i32, i32, u32, u32, vp, vp, i32, vp, vp, i32, vp]),
    "vkl_sample_f32": (i32, [vp, i32, i32, f32, u64, u32, vp, vp, vp, vp, vp, vp]),
    "vkl_concat_part_f16": (i32, [vp, i32, i32, i32, sz, sz, vp, sz, sz, sz, vp]),
    "vkl_read_kvcache_f16": (i32, [vp, i32, i32, i32, u32, u32, vp, vp]),
    "vkl_reduce_f16": (i32, [vp, i32, i32, i32, i32, vp, vp]),
    "vkl_attn_prefill_causal_f16": (i32, [vp, vp, vp, i32, i32, i32, i32, sz, sz, sz, sz, sz, sz, f32, vp, sz, sz, vp]),
    "vkl_matmul_f16_tb": (i32, [vp, vp, i32, i32, i32, i32, sz, sz, sz, sz, sz, sz, f32, f32, i32, vp, vp, vp, vp]),
    "vkl_matmul_f16_nn": (i32, [vp, vp, i32, i32, i32, i32, sz, sz, sz, sz, sz, sz, f32, f32, i32, vp, vp]),
    "vkl_ffn_upgate_f16": (i32, [vp, vp, vp, i32, i32, i32, vp, vp]),
    "vkl_rope_f16": (i32, [vp, i32, i32, i32, vp, vp, u32, vp]),
    "vkl_kv_update_f16": (i32, [vp, vp, i32, i32, i32, i32, u32, vp]),
    "vkl_softmax_f16": (i32, [vp, i32, i32, i32, i32, u32, vp, vp]),
    "vkl_elementwise_f16": (i32, [vp, vp, sz, i32, vp]),
    "vkl_elementwise_const_f16": (i32, [vp, f32, sz, i32, vp, vp]),
    "vkl_cast_f16_f32": (i32, [vp, vp, sz, vp]),
    "vkl_cast_f32_f16": (i32, [vp, vp, sz, vp]),
    "vkl_argop_f16": (i32, [vp, i32, i32, i32, vp, vp]),
    "vkl_slice_f16": (i32, [vp, i32, i32, i32, i32, i32, i32, i32, i32, i32, vp, vp]),
    "vkl_transpose102_f16": (i32, [vp, i32, i32, i32, vp, vp]),
}


class VklError(RuntimeError):
    pass


def load_library(path=HIP_LIB_PATH, signatures=None):
    """dlopen the HIP library and type every exported entry point."""
    if not os.path.exists(path):
        raise VklError("%s is missing: build it with __graft_entry__.build() "
                       "(there is no CPU fallback)" % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in (signatures or SIGNATURES).items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load_library()
    return _lib


def check(err, what=""):
    if err != 0:
        msg = lib().vkl_error_string(err)
        raise VklError("%s failed: hip error %d (%s)" % (what or "vkl call", err, msg.decode() if msg else "?"))


class Device:
    """Opens a GPU, owns one stream; helper for tests and the benchmark."""

    def __init__(self, dev=0):
        n = i32(0)
        check(lib().vkl_device_count(C.byref(n)), "vkl_device_count")
        if n.value <= 0:
            raise VklError("no HIP device visible")
        self.info = DeviceInfo()
        check(lib().vkl_device_open(dev, C.byref(self.info)), "vkl_device_open")
        s = vp()
        check(lib().vkl_stream_create(C.byref(s)), "vkl_stream_create")
        self.stream = s

    def sync(self):
        check(lib().vkl_stream_sync(self.stream), "vkl_stream_sync")

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        buf = DeviceBuffer(self, arr.nbytes)
        buf.write(arr)
        return buf

    def upload_q8_0(self, raw, rows, K):
        """raw: uint8 GGUF blocks [rows, K/32*34] -> planar device buffer."""
        raw = np.ascontiguousarray(raw, np.uint8)
        staging = self.upload(raw)
        planar = DeviceBuffer(self, raw.nbytes)
        check(lib().vkl_q8_0_pack(staging.ptr, planar.ptr, rows, K, self.stream), "vkl_q8_0_pack")
        self.sync()
        staging.free()
        return planar

    def event(self):
        e = vp()
        check(lib().vkl_event_create(C.byref(e)), "vkl_event_create")
        return e

    def record(self, ev):
        check(lib().vkl_event_record(ev, self.stream), "vkl_event_record")

    def elapsed_ms(self, e0, e1):
        check(lib().vkl_event_sync(e1), "vkl_event_sync")
        ms = f32(0)
        check(lib().vkl_event_elapsed_ms(e0, e1, C.byref(ms)), "vkl_event_elapsed_ms")
        return ms.value


class DeviceBuffer:
    def __init__(self, dev, nbytes):
        self.dev = dev
        self.nbytes = int(nbytes)
        p = vp()
        check(lib().vkl_malloc(C.byref(p), self.nbytes), "vkl_malloc")
        self.ptr = p

    def write(self, arr, sync=True):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        check(lib().vkl_memcpy_h2d(self.ptr, arr.ctypes.data, arr.nbytes, self.dev.stream), "vkl_memcpy_h2d")
        if sync:
            self.dev.sync()

    def read(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib().vkl_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, self.dev.stream), "vkl_memcpy_d2h")
        self.dev.sync()
        return out

    def zero(self):
        check(lib().vkl_memset(self.ptr, 0, self.nbytes, self.dev.stream), "vkl_memset")

    def free(self):
        if self.ptr:
            check(lib().vkl_free(self.ptr), "vkl_free")
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
