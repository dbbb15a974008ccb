"""GGUF files for the llama2 path: a writer (to make model files from weight
dictionaries, e.g. the synthetic ones) and a ctypes view of the reader that
libvkllama_host.so exports with gguf-tools' calling interface.

File format (version 3, little endian): header (magic "GGUF", version,
tensor count, key count), key/value pairs, tensor infos (name, dims with the
innermost first, ggml type, offset), padding to `general.alignment`, tensor
data.  Tensor names and keys are the ones models/llama2.h:367-370,401-403,
486-512 of the reference reads.
"""
import ctypes as C
import struct

import numpy as np

GGML_F32, GGML_F16, GGML_Q8_0 = 0, 1, 8
T_UINT32, T_FLOAT32, T_STRING, T_ARRAY, T_INT32 = 4, 6, 8, 9, 5


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _kv(key, vtype, payload):
    return _s(key) + struct.pack("<I", vtype) + payload


def write_gguf(path, cfg, weights, alignment=32, tokens=None):
    """cfg: dim, n_layers, n_heads, ffn, vocab, maxlen, eps, wtype (8 = Q8_0,
    1 = F16); weights: {tensor name: numpy array} with matrices as raw Q8_0
    block bytes (uint8 [rows, K/32*34]) or float16 [rows, K] and norm weights
    as float32 [dim] (the layout vkllama_amd.model.synth_weights produces)."""
    from .model import matrix_shape, tensor_names
    kvs = [
        _kv("general.architecture", T_STRING, _s("llama")),
        _kv("general.name", T_STRING, _s("vkllama-synthetic")),
        _kv("general.alignment", T_UINT32, struct.pack("<I", alignment)),
        _kv("llama.context_length", T_UINT32, struct.pack("<I", cfg["maxlen"])),
        _kv("llama.embedding_length", T_UINT32, struct.pack("<I", cfg["dim"])),
        _kv("llama.feed_forward_length", T_UINT32, struct.pack("<I", cfg["ffn"])),
        _kv("llama.block_count", T_UINT32, struct.pack("<I", cfg["n_layers"])),
        _kv("llama.attention.head_count", T_UINT32, struct.pack("<I", cfg["n_heads"])),
        _kv("llama.attention.head_count_kv", T_UINT32, struct.pack("<I", cfg["n_heads"])),
        _kv("llama.attention.layer_norm_rms_epsilon", T_FLOAT32, struct.pack("<f", cfg["eps"])),
        _kv("llama.rope.dimension_count", T_UINT32, struct.pack("<I", cfg["dim"] // cfg["n_heads"])),
    ]
    if tokens is not None:   # an array of strings and an array of scalars, as tokenizer keys are
        kvs.append(_kv("tokenizer.ggml.tokens", T_ARRAY,
                       struct.pack("<IQ", T_STRING, len(tokens)) + b"".join(_s(t) for t in tokens)))
        kvs.append(_kv("tokenizer.ggml.token_type", T_ARRAY,
                       struct.pack("<IQ", T_INT32, len(tokens)) + struct.pack("<%di" % len(tokens), *([1] * len(tokens)))))
    names = tensor_names(cfg["n_layers"])
    infos, blobs, off = [], [], 0
    for n in names:
        a = np.ascontiguousarray(weights[n])
        if n.endswith("norm.weight"):
            gtype, dims = GGML_F32, [a.size]
        else:
            rows, K = matrix_shape(cfg, n)
            gtype, dims = (GGML_Q8_0 if a.dtype == np.uint8 else GGML_F16), [K, rows]
        infos.append(_s(n) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
                     + struct.pack("<IQ", gtype, off))
        blobs.append((off, a))
        off = (off + a.nbytes + alignment - 1) // alignment * alignment
    head = b"GGUF" + struct.pack("<IQQ", 3, len(names), len(kvs)) + b"".join(kvs) + b"".join(infos)
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        base = f.tell()
        for o, a in blobs:
            f.seek(base + o)
            f.write(a.tobytes())
        f.truncate(base + off)
    return path


# ---- reader (ctypes view of gguf_open / gguf_get_key / gguf_get_tensor) ------
class GgufKey(C.Structure):
    _fields_ = [("name", C.c_void_p), ("namelen", C.c_size_t), ("type", C.c_uint32), ("val", C.c_void_p)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_void_p), ("namelen", C.c_size_t), ("type", C.c_uint32), ("ndim", C.c_uint32),
                ("dim", C.c_uint64 * 8), ("offset", C.c_uint64), ("bsize", C.c_uint64),
                ("num_weights", C.c_uint64), ("weights_data", C.c_void_p)]


def read_gguf(path):
    """{'version', 'keys': {name: (type, value or None)}, 'tensors': {name:
    dict(type, dims, bsize, data=uint8 array copy)}}; raises OSError if the
    file is not a GGUF file this reader understands."""
    from .model import lib
    L = lib()
    L.gguf_open.restype = C.c_void_p
    L.gguf_open.argtypes = [C.c_char_p]
    L.gguf_close.argtypes = [C.c_void_p]
    L.gguf_get_key.argtypes = [C.c_void_p, C.POINTER(GgufKey)]
    L.gguf_get_tensor.argtypes = [C.c_void_p, C.POINTER(GgufTensor)]
    L.gguf_version.argtypes = [C.c_void_p]
    L.gguf_version.restype = C.c_uint32
    g = L.gguf_open(path.encode())
    if not g:
        raise OSError("not a readable GGUF file: %s" % path)
    try:
        out = {"version": int(L.gguf_version(g)), "keys": {}, "tensors": {}}
        k = GgufKey()
        while L.gguf_get_key(g, C.byref(k)):
            name = C.string_at(k.name, k.namelen).decode()
            val = None
            if k.type == T_UINT32:
                val = C.cast(k.val, C.POINTER(C.c_uint32))[0]
            elif k.type == T_FLOAT32:
                val = C.cast(k.val, C.POINTER(C.c_float))[0]
            elif k.type == T_STRING:
                n = C.cast(k.val, C.POINTER(C.c_uint64))[0]
                val = C.string_at(k.val + 8, n).decode()
            out["keys"][name] = (int(k.type), val)
        t = GgufTensor()
        while L.gguf_get_tensor(g, C.byref(t)):
            name = C.string_at(t.name, t.namelen).decode()
            data = np.frombuffer(C.string_at(t.weights_data, t.bsize), np.uint8)
            out["tensors"][name] = dict(type=int(t.type), dims=[int(t.dim[i]) for i in range(t.ndim)],
                                        bsize=int(t.bsize), data=data)
        return out
    finally:
        L.gguf_close(g)
