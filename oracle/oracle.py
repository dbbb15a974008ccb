"""ctypes binding of the CPU oracle (oracle/libvkl_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg, never by the vkllama_amd package.
All fp16 data travels as numpy uint16/float16 arrays; Q8_0 rows are uint8
arrays of 34-byte GGUF blocks.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvkl_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (no GPU involved)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_u8p = C.POINTER(C.c_uint8)
_u16p = C.POINTER(C.c_uint16)
_u32p = C.POINTER(C.c_uint32)
_f32p = C.POINTER(C.c_float)
_vpp = C.POINTER(C.c_void_p)


def _p(a, t):
    return a.ctypes.data_as(t)


def _u16(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def _decl(name, res, *args):
    f = getattr(_lib, name)
    f.restype = res
    f.argtypes = list(args)
    return f


_f32_to_f16 = _decl("vko_f32_to_f16", C.c_uint16, C.c_float)
_f32_to_f16_hw = _decl("vko_f32_to_f16_hw", C.c_uint16, C.c_float)
_f16_to_f32 = _decl("vko_f16_to_f32", C.c_float, C.c_uint16)
_ref_host_f32_to_f16 = _decl("vko_ref_host_f32_to_f16", C.c_uint16, C.c_float)
_decl("vko_q8_0_quantize_row", None, _f32p, C.c_size_t, _u8p, C.c_int)
_decl("vko_q8_0_dequantize_row", None, _u8p, C.c_size_t, _f32p, C.c_int)
_decl("vko_embedding_q8_0", None, _u8p, C.c_uint32, C.c_uint32, _u32p, C.c_uint32, C.c_uint32, _u16p)
_decl("vko_embedding_f16", None, _u16p, C.c_uint32, C.c_uint32, _u32p, C.c_uint32, C.c_uint32, _u16p)
_decl("vko_rmsnorm_f16", None, _u16p, _f32p, C.c_int, C.c_int, C.c_float, _u16p)
_decl("vko_set_lane_order", None, C.c_int)
_decl("vko_matmul_q8_0", None, _u16p, _u8p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int, _u16p)
_decl("vko_kqv_q8_0", None, _u16p, _u8p, _u8p, _u8p, C.c_int, C.c_int, C.c_int, _u16p, _u16p, _u16p)
_decl("vko_ffn_upgate_q8_0", None, _u16p, _u8p, _u8p, C.c_int, C.c_int, C.c_int, _u16p)
for _n in ("vko_matmul_f16_tb", "vko_matmul_f16_nn"):
    _decl(_n, None, _u16p, _u16p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_size_t,
          C.c_size_t, C.c_size_t, C.c_float, C.c_float, C.c_int, _u16p)
_decl("vko_ffn_upgate_f16", None, _u16p, _u16p, _u16p, C.c_int, C.c_int, C.c_int, _u16p)
_decl("vko_rope_tables", None, C.c_int, C.c_int, _f32p, _f32p)
_decl("vko_rope_f16", None, _u16p, C.c_int, C.c_int, C.c_int, _f32p, _f32p, C.c_uint32)
_decl("vko_update_kvcache_f16", None, _u16p, _u16p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint32)
_decl("vko_softmax_f16", None, _u16p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint32, _u16p)
_decl("vko_elementwise_f16", None, _u16p, _u16p, C.c_size_t, C.c_int, _u16p)
_decl("vko_argmax_f16", None, _u16p, C.c_int, C.c_int, _u32p)
_decl("vko_argmax_f32", C.c_uint32, _f32p, C.c_int)
_decl("vko_transpose102_f16", None, _u16p, C.c_int, C.c_int, C.c_int, _u16p)


def f32_to_f16_bits(x, hw=False):
    return int((_f32_to_f16_hw if hw else _f32_to_f16)(float(np.float32(x))))


def f16_bits_to_f32(h):
    return float(_f16_to_f32(int(h)))


def ref_host_f32_to_f16_bits(x):
    return int(_ref_host_f32_to_f16(float(np.float32(x))))


def q8_0_row_bytes(n, scale_bytes=2):
    return (n + 31) // 32 * (32 + scale_bytes)


def quantize_q8_0(x, scale_bytes=2):
    """x: [rows, n] float32 -> uint8 [rows, blocks*(32+scale_bytes)]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    out = np.empty((x2.shape[0], q8_0_row_bytes(x2.shape[1], scale_bytes)), np.uint8)
    for r in range(x2.shape[0]):
        _lib.vko_q8_0_quantize_row(_p(x2[r], _f32p), x2.shape[1], _p(out[r], _u8p), scale_bytes)
    return out.reshape(x.shape[:-1] + (out.shape[1],))


def dequantize_q8_0(q, n, scale_bytes=2):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    q2 = q.reshape(-1, q.shape[-1])
    out = np.empty((q2.shape[0], n), np.float32)
    for r in range(q2.shape[0]):
        _lib.vko_q8_0_dequantize_row(_p(q2[r], _u8p), n, _p(out[r], _f32p), scale_bytes)
    return out.reshape(q.shape[:-1] + (n,))


def embedding_q8_0(table, VW, toks, unk=0):
    table = np.ascontiguousarray(table, np.uint8)
    toks = np.ascontiguousarray(toks, np.uint32)
    out = np.empty((toks.size, VW), np.uint16)
    _lib.vko_embedding_q8_0(_p(table, _u8p), table.shape[0], VW, _p(toks, _u32p), toks.size, unk, _p(out, _u16p))
    return out.view(np.float16)


def embedding_f16(table, toks, unk=0):
    table = _u16(table)
    toks = np.ascontiguousarray(toks, np.uint32)
    out = np.empty((toks.size, table.shape[1]), np.uint16)
    _lib.vko_embedding_f16(_p(table, _u16p), table.shape[0], table.shape[1], _p(toks, _u32p), toks.size, unk,
                           _p(out, _u16p))
    return out.view(np.float16)


def rmsnorm(x, w, eps):
    x = _u16(x)
    w = np.ascontiguousarray(w, np.float32)
    rows, W = x.reshape(-1, x.shape[-1]).shape
    out = np.empty_like(x)
    _lib.vko_rmsnorm_f16(_p(x, _u16p), _p(w, _f32p), rows, W, eps, _p(out, _u16p))
    return out.view(np.float16)


def set_lane_order(order):
    """Order in which the dot-product kernels add the 32 lanes of a subgroup
    (the reference's subgroupAdd leaves it open): 0 pairwise halving (default),
    1 sequential, 2 neighbours first, 3 sequential from the last lane, 4 groups
    of eight then the groups.  Process-wide."""
    _lib.vko_set_lane_order(int(order))


def matmul_q8_0(x, w, K, scale=1.0, bias=0.0, act=0):
    """x [M,K] fp16, w uint8 [N, K/32*34] -> [M,N] fp16."""
    x = _u16(x)
    w = np.ascontiguousarray(w, np.uint8)
    M, N = x.shape[0], w.shape[0]
    y = np.empty((M, N), np.uint16)
    _lib.vko_matmul_q8_0(_p(x, _u16p), _p(w, _u8p), M, N, K, scale, bias, act, _p(y, _u16p))
    return y.view(np.float16)


def kqv_q8_0(x, wk, wq, wv, K):
    x = _u16(x)
    M, N = x.shape[0], wk.shape[0]
    k, q, v = (np.empty((M, N), np.uint16) for _ in range(3))
    _lib.vko_kqv_q8_0(_p(x, _u16p), _p(wk, _u8p), _p(wq, _u8p), _p(wv, _u8p), M, N, K, _p(k, _u16p), _p(q, _u16p),
                      _p(v, _u16p))
    return k.view(np.float16), q.view(np.float16), v.view(np.float16)


def ffn_upgate_q8_0(x, wup, wgate, K):
    x = _u16(x)
    M, N = x.shape[0], wup.shape[0]
    out = np.empty((M, N), np.uint16)
    _lib.vko_ffn_upgate_q8_0(_p(x, _u16p), _p(wup, _u8p), _p(wgate, _u8p), M, N, K, _p(out, _u16p))
    return out.view(np.float16)


def ffn_upgate_f16(x, wup, wgate):
    x, wup, wgate = _u16(x), _u16(wup), _u16(wgate)
    M, K = x.shape
    N = wup.shape[0]
    out = np.empty((M, N), np.uint16)
    _lib.vko_ffn_upgate_f16(_p(x, _u16p), _p(wup, _u16p), _p(wgate, _u16p), M, N, K, _p(out, _u16p))
    return out.view(np.float16)


def matmul_f16_tb(a, b, scale=1.0, bias=0.0, act=0):
    """a [C,M,K], b [C,N,K] dense -> [C,M,N]."""
    a, b = _u16(a), _u16(b)
    Cc, M, K = a.shape
    N = b.shape[1]
    y = np.empty((Cc, M, N), np.uint16)
    _lib.vko_matmul_f16_tb(_p(a, _u16p), _p(b, _u16p), Cc, M, N, K, M * K, K, N * K, K, scale, bias, act,
                           _p(y, _u16p))
    return y.view(np.float16)


def matmul_f16_nn(a, b, scale=1.0, bias=0.0, act=0):
    """a [C,M,K], b [C,K,N] dense -> [C,M,N]."""
    a, b = _u16(a), _u16(b)
    Cc, M, K = a.shape
    N = b.shape[2]
    y = np.empty((Cc, M, N), np.uint16)
    _lib.vko_matmul_f16_nn(_p(a, _u16p), _p(b, _u16p), Cc, M, N, K, M * K, K, K * N, N, scale, bias, act,
                           _p(y, _u16p))
    return y.view(np.float16)


def rope_tables(maxlen, dim):
    fc = np.empty((maxlen, dim // 2), np.float32)
    fs = np.empty((maxlen, dim // 2), np.float32)
    _lib.vko_rope_tables(maxlen, dim, _p(fc, _f32p), _p(fs, _f32p))
    return fc, fs


def rope(x, fc, fs, offset):
    x = _u16(x).copy()
    Cc, H, W = x.shape
    _lib.vko_rope_f16(_p(x, _u16p), Cc, H, W, _p(fc, _f32p), _p(fs, _f32p), offset)
    return x.view(np.float16)


def update_kvcache(cache, kv, offset):
    cache = _u16(cache).copy()
    kv = _u16(kv)
    Cc, HO, W = cache.shape
    _lib.vko_update_kvcache_f16(_p(cache, _u16p), _p(kv, _u16p), Cc, HO, kv.shape[1], W, offset)
    return cache.view(np.float16)


def softmax(x, seq_mask, offset):
    x = _u16(x)
    Cc, H, W = x.shape
    out = np.empty_like(x)
    _lib.vko_softmax_f16(_p(x, _u16p), Cc, H, W, int(seq_mask), offset, _p(out, _u16p))
    return out.view(np.float16)


def elementwise(x, y, op=0):
    x, y = _u16(x), _u16(y)
    out = np.empty_like(x)
    _lib.vko_elementwise_f16(_p(x, _u16p), _p(y, _u16p), x.size, op, _p(out, _u16p))
    return out.view(np.float16)


def argmax_f16(x):
    x = _u16(x)
    rows, W = x.reshape(-1, x.shape[-1]).shape
    out = np.empty(rows, np.uint32)
    _lib.vko_argmax_f16(_p(x, _u16p), rows, W, _p(out, _u32p))
    return out


def argmax_f32(x):
    x = np.ascontiguousarray(x, np.float32)
    return int(_lib.vko_argmax_f32(_p(x, _f32p), x.size))


def transpose102(x):
    x = _u16(x)
    Cc, H, W = x.shape
    out = np.empty((H, Cc, W), np.uint16)
    _lib.vko_transpose102_f16(_p(x, _u16p), Cc, H, W, _p(out, _u16p))
    return out.view(np.float16)


class _CModel(C.Structure):
    _fields_ = [
        ("dim", C.c_int), ("n_layers", C.c_int), ("n_heads", C.c_int), ("head_dim", C.c_int),
        ("ffn", C.c_int), ("vocab", C.c_int), ("maxlen", C.c_int),
        ("eps", C.c_float), ("final_eps", C.c_float), ("wtype", C.c_int),
        ("lastblock_rope_quirk", C.c_int),
        ("tok_embd", C.c_void_p), ("output", C.c_void_p), ("output_norm", C.c_void_p),
        ("wq", _vpp), ("wk", _vpp), ("wv", _vpp), ("wo", _vpp),
        ("w_gate", _vpp), ("w_up", _vpp), ("w_down", _vpp),
        ("attn_norm", _vpp), ("ffn_norm", _vpp),
    ]


_lib.vko_state_create.restype = C.c_void_p
_lib.vko_state_create.argtypes = [C.POINTER(_CModel)]
_lib.vko_state_destroy.argtypes = [C.c_void_p]
_lib.vko_forward.restype = C.c_int
_lib.vko_forward.argtypes = [C.POINTER(_CModel), C.c_void_p, _u32p, C.c_int, C.c_size_t, _f32p]
_lib.vko_generate_greedy.restype = C.c_int
_lib.vko_generate_greedy.argtypes = [C.POINTER(_CModel), C.c_void_p, _u32p, C.c_int, C.c_int, _u32p, _f32p]
_lib.vko_state_kcache.restype = _u16p
_lib.vko_state_kcache.argtypes = [C.c_void_p, C.c_int]
_lib.vko_state_vcache.restype = _u16p
_lib.vko_state_vcache.argtypes = [C.c_void_p, C.c_int]
_lib.vko_state_hidden.restype = _u16p
_lib.vko_state_hidden.argtypes = [C.c_void_p, C.POINTER(C.c_int)]


class OracleModel:
    """Llama2 model on the CPU oracle.

    cfg: dict with dim, n_layers, n_heads, ffn, vocab, maxlen, eps, wtype
    weights: dict name -> numpy array, GGUF tensor names
    (token_embd.weight, output.weight, output_norm.weight,
    blk.N.{attn_norm,attn_q,attn_k,attn_v,attn_output,ffn_norm,ffn_gate,
    ffn_down,ffn_up}.weight); matrices are uint8 Q8_0 rows or fp16, norm
    weights fp32.
    """

    def __init__(self, cfg, weights, lastblock_rope_quirk=True):
        self.cfg = dict(cfg)
        self._keep = []
        L = cfg["n_layers"]

        def ptr(a):
            a = np.ascontiguousarray(a)
            self._keep.append(a)
            return a.ctypes.data

        def ptr_array(fmt):
            arr = (C.c_void_p * L)(*[ptr(weights[fmt % i]) for i in range(L)])
            self._keep.append(arr)
            return C.cast(arr, _vpp)

        m = _CModel()
        m.dim, m.n_layers, m.n_heads = cfg["dim"], L, cfg["n_heads"]
        m.head_dim = cfg["dim"] // cfg["n_heads"]
        m.ffn, m.vocab, m.maxlen = cfg["ffn"], cfg["vocab"], cfg["maxlen"]
        m.eps, m.final_eps = cfg.get("eps", 1e-5), 1e-6
        m.wtype = cfg.get("wtype", 8)
        m.lastblock_rope_quirk = 1 if lastblock_rope_quirk else 0
        m.tok_embd = ptr(weights["token_embd.weight"])
        m.output = ptr(weights["output.weight"])
        m.output_norm = ptr(np.asarray(weights["output_norm.weight"], np.float32))
        m.wq = ptr_array("blk.%d.attn_q.weight")
        m.wk = ptr_array("blk.%d.attn_k.weight")
        m.wv = ptr_array("blk.%d.attn_v.weight")
        m.wo = ptr_array("blk.%d.attn_output.weight")
        m.w_gate = ptr_array("blk.%d.ffn_gate.weight")
        m.w_up = ptr_array("blk.%d.ffn_up.weight")
        m.w_down = ptr_array("blk.%d.ffn_down.weight")
        m.attn_norm = ptr_array("blk.%d.attn_norm.weight")
        m.ffn_norm = ptr_array("blk.%d.ffn_norm.weight")
        self._m = m
        self._s = _lib.vko_state_create(C.byref(m))

    def close(self):
        if self._s:
            _lib.vko_state_destroy(self._s)
            self._s = None

    def __del__(self):
        self.close()

    def forward(self, toks, offset):
        toks = np.ascontiguousarray(toks, np.uint32)
        logits = np.empty(self.cfg["vocab"], np.float32)
        rc = _lib.vko_forward(C.byref(self._m), self._s, _p(toks, _u32p), toks.size, offset, _p(logits, _f32p))
        if rc:
            raise RuntimeError("oracle forward failed: %d" % rc)
        return logits

    def generate_greedy(self, prompt, n_gen):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        ids = np.empty(n_gen, np.uint32)
        first = np.empty(self.cfg["vocab"], np.float32)
        rc = _lib.vko_generate_greedy(C.byref(self._m), self._s, _p(prompt, _u32p), prompt.size, n_gen,
                                      _p(ids, _u32p), _p(first, _f32p))
        if rc:
            raise RuntimeError("oracle generate failed: %d" % rc)
        return ids, first

    def _cache(self, fn, layer):
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        n = c["n_heads"] * c["maxlen"] * hd
        p = fn(self._s, layer)
        return np.ctypeslib.as_array(p, shape=(n,)).reshape(c["n_heads"], c["maxlen"], hd).copy().view(np.float16)

    def set_cache(self, layer, value, rows):
        """Replaces one layer's K (value False) or V cache with `rows`
        (float16 [heads, maxlen, head_dim]): puts the model at a late position
        without the prompt pass that leads there."""
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        rows = np.ascontiguousarray(rows, np.float16)
        assert rows.shape == (c["n_heads"], c["maxlen"], hd)
        p = (_lib.vko_state_vcache if value else _lib.vko_state_kcache)(self._s, layer)
        C.memmove(p, rows.ctypes.data, rows.nbytes)

    def kcache(self, layer):
        return self._cache(_lib.vko_state_kcache, layer)

    def vcache(self, layer):
        return self._cache(_lib.vko_state_vcache, layer)

    def hidden(self):
        rows = C.c_int(0)
        p = _lib.vko_state_hidden(self._s, C.byref(rows))
        return np.ctypeslib.as_array(p, shape=(rows.value * self.cfg["dim"],)).reshape(rows.value, -1).copy().view(
            np.float16)
