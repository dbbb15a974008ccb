"""ctypes binding of include/vkl_model.h (libvkllama_host.so): the llama2
token loop behind the C++ drop-in classes.  No CPU fallback: a missing
library or a failing call raises."""
import ctypes as C
import os

import numpy as np

from . import capi

HOST_LIB_PATH = os.path.join(capi.LIB_DIR, "libvkllama_host.so")

vp, sz, u32, u64, i32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int


class TensorDesc(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", u32), ("dim0", u64), ("dim1", u64), ("data", vp), ("bsize", u64)]


class HParams(C.Structure):
    _fields_ = [("head_count", u32), ("block_count", u32), ("context_length", u32), ("rms_eps", C.c_float)]


SIGNATURES = {
    "vkl_model_create": (i32, [i32, C.POINTER(HParams), C.POINTER(TensorDesc), sz, C.POINTER(vp)]),
    "vkl_model_load_gguf": (i32, [i32, C.c_char_p, C.POINTER(vp)]),
    "vkl_model_destroy": (None, [vp]),
    "vkl_model_last_error": (C.c_char_p, [vp]),
    "vkl_model_vocab": (sz, [vp]),
    "vkl_model_forward": (i32, [vp, vp, sz, sz, vp]),
    "vkl_model_generate_greedy": (i32, [vp, vp, sz, sz, vp, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "vkl_model_generate_sampled": (i32, [vp, vp, sz, sz, i32, C.c_float, u64, vp, C.POINTER(C.c_double),
                                         C.POINTER(C.c_double)]),
    "vkl_model_set_option": (i32, [vp, C.c_char_p, i32]),
    "vkl_model_decode_recoveries": (sz, [vp]),
    "vkl_model_write_kv_cache": (i32, [vp, sz, i32, vp, sz]),
    "vkl_model_read_kv_cache": (i32, [vp, sz, i32, vp, sz]),
    "vkl_model_decode_step_bytes": (sz, [vp, sz]),
    "vkl_model_phase_times": (i32, [vp, vp, vp]),
    "vkl_model_phase_bytes": (sz, [vp, i32, sz]),
    "vkl_model_phase_replay": (i32, [vp, i32, sz, i32, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]),
    "vkl_synth_normal_f32": (None, [u64, sz, C.c_float, vp]),
    "vkl_synth_normal_f16": (None, [u64, sz, C.c_float, vp]),
    "vkl_synth_normal_q8_0": (None, [u64, sz, sz, C.c_float, vp]),
    "vkl_sampler_create": (i32, [i32, C.c_float, i32, u64, C.POINTER(vp)]),
    "vkl_sampler_destroy": (None, [vp]),
    "vkl_sampler_sample": (i32, [vp, vp, sz]),
    "vkl_sampler_candidates": (sz, [vp, vp, vp, sz]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        capi.lib()  # libvkllama_hip.so first, globally, so the host library resolves against it
        _lib = capi.load_library(HOST_LIB_PATH, SIGNATURES)
    return _lib


def tensor_names(n_layers):
    names = ["token_embd.weight", "output.weight", "output_norm.weight"]
    for i in range(n_layers):
        for t in ("attn_norm", "attn_q", "attn_k", "attn_v", "attn_output", "ffn_norm", "ffn_gate", "ffn_down",
                  "ffn_up"):
            names.append("blk.%d.%s.weight" % (i, t))
    return names


def matrix_shape(cfg, name):
    """(rows, cols) of a weight matrix; GGUF dim0 = cols, dim1 = rows."""
    d, F, V = cfg["dim"], cfg["ffn"], cfg["vocab"]
    if name in ("token_embd.weight", "output.weight"):
        return V, d
    if "ffn_gate" in name or "ffn_up" in name:
        return F, d
    if "ffn_down" in name:
        return d, F
    return d, d


def synth_weights(cfg, seed=1234, std=0.02, norm_value=1.0):
    """Random-init Llama-2-shaped weights, N(0, std), in the storage format
    cfg['wtype'] names (8 = Q8_0 GGUF blocks, 1 = fp16); norm weights are
    fp32 and equal to norm_value.  Deterministic in (cfg, seed)."""
    w = {}
    for idx, name in enumerate(tensor_names(cfg["n_layers"])):
        if name.endswith("_norm.weight"):
            w[name] = np.full(cfg["dim"], norm_value, np.float32)
            continue
        N, K = matrix_shape(cfg, name)
        if cfg.get("wtype", 8) == 8:
            out = np.empty((N, (K + 31) // 32 * 34), np.uint8)
            lib().vkl_synth_normal_q8_0(seed + idx, N, K, std, out.ctypes.data)
        else:
            out = np.empty((N, K), np.uint16)
            lib().vkl_synth_normal_f16(seed + idx, N * K, std, out.ctypes.data)
            out = out.view(np.float16)
        w[name] = out
    return w


class Sampler:
    """Host sampler over a row of logits (TopkSampler / TopPSampler of the
    reference's models/samplers.h).  kind "topk" with k, or "topp" with p;
    seed=None seeds from the system's random device as the reference does."""

    def __init__(self, kind, param, seed=None):
        h = vp()
        err = lib().vkl_sampler_create({"topk": 0, "topp": 1}[kind], float(param), int(seed is not None),
                                       int(seed or 0), C.byref(h))
        if err:
            raise ValueError("bad sampler parameters: %s %r" % (kind, param))
        self._h = h

    def sample(self, logits):
        logits = np.ascontiguousarray(logits, np.float32).reshape(-1)
        return int(lib().vkl_sampler_sample(self._h, logits.ctypes.data, logits.size))

    def candidates(self):
        """(ids, probabilities) of the last draw's candidate set, most likely first"""
        n = lib().vkl_sampler_candidates(self._h, None, None, 0)
        ids, probs = np.empty(n, np.int32), np.empty(n, np.float32)
        lib().vkl_sampler_candidates(self._h, ids.ctypes.data, probs.ctypes.data, n)
        return ids, probs

    def close(self):
        if self._h:
            lib().vkl_sampler_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Llama2:
    """vkllama::Model through the C ABI.

    cfg: dim, n_layers, n_heads, ffn, vocab, maxlen, eps, wtype
    weights: GGUF tensor name -> numpy array (uint8 Q8_0 blocks / float16 /
    float32 for the norm weights)."""

    def __init__(self, cfg, weights, dev=0):
        self.cfg = dict(cfg)
        self._h = None
        names = tensor_names(cfg["n_layers"])
        descs = (TensorDesc * len(names))()
        keep = []
        for i, n in enumerate(names):
            a = np.ascontiguousarray(weights[n])
            keep.append(a)
            if n.endswith("_norm.weight"):
                a = np.ascontiguousarray(a, np.float32)
                keep.append(a)
                t, d0, d1 = 0, a.size, 1
            else:
                rows, cols = matrix_shape(cfg, n)
                t = 8 if a.dtype == np.uint8 else 1
                d0, d1 = cols, rows
            descs[i] = TensorDesc(n.encode(), t, d0, d1, a.ctypes.data, a.nbytes)
        hp = HParams(cfg["n_heads"], cfg["n_layers"], cfg["maxlen"], cfg.get("eps", 1e-5))
        h = vp()
        rc = lib().vkl_model_create(dev, C.byref(hp), descs, len(names), C.byref(h))
        self._h = h
        if rc:
            raise capi.VklError("vkl_model_create failed (%d): %s" % (rc, self._err()))

    @classmethod
    def from_gguf(cls, path, dev=0):
        """Loads a GGUF file the way app/llama2_infer.cpp of the reference does
        (keys and tensors through the gguf reader, then Model::init)."""
        self = cls.__new__(cls)
        self._h = None
        h = vp()
        rc = lib().vkl_model_load_gguf(dev, path.encode(), C.byref(h))
        self._h = h
        if rc:
            msg = self._err()
            self.close()
            raise capi.VklError("vkl_model_load_gguf failed (%d): %s" % (rc, msg))
        self.cfg = {"vocab": int(lib().vkl_model_vocab(self._h))}
        return self

    def _err(self):
        m = lib().vkl_model_last_error(self._h)
        return m.decode() if m else "?"

    def _check(self, rc, what):
        if rc:
            raise capi.VklError("%s failed (%d): %s" % (what, rc, self._err()))

    def close(self):
        if self._h:
            lib().vkl_model_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_option(self, name, value):
        self._check(lib().vkl_model_set_option(self._h, name.encode(), int(value)), "set_option")

    def forward(self, toks, offset):
        toks = np.ascontiguousarray(toks, np.uint32)
        logits = np.empty(self.cfg["vocab"], np.float32)
        self._check(lib().vkl_model_forward(self._h, toks.ctypes.data, toks.size, offset, logits.ctypes.data),
                    "vkl_model_forward")
        return logits

    def generate_greedy(self, prompt, n_gen):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        ids = np.empty(n_gen, np.uint32)
        t_pre, t_dec = C.c_double(0), C.c_double(0)
        self._check(lib().vkl_model_generate_greedy(self._h, prompt.ctypes.data, prompt.size, n_gen,
                                                    ids.ctypes.data, C.byref(t_pre), C.byref(t_dec)),
                    "vkl_model_generate_greedy")
        return ids, t_pre.value, t_dec.value

    def generate_sampled(self, prompt, n_gen, topk=40, topp=None, seed=0):
        """Generation with the token drawn on the device: from the topk largest
        logits, or (topp given) from the top-p set; seed fixes the sequence."""
        prompt = np.ascontiguousarray(prompt, np.uint32)
        ids = np.empty(n_gen, np.uint32)
        t_pre, t_dec = C.c_double(0), C.c_double(0)
        self._check(lib().vkl_model_generate_sampled(self._h, prompt.ctypes.data, prompt.size, n_gen, int(topk),
                                                     -1.0 if topp is None else float(topp), int(seed),
                                                     ids.ctypes.data, C.byref(t_pre), C.byref(t_dec)),
                    "vkl_model_generate_sampled")
        return ids, t_pre.value, t_dec.value

    def read_kv_cache(self, layer, value):
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        out = np.empty((c["n_heads"], c["maxlen"], hd), np.uint16)
        self._check(lib().vkl_model_read_kv_cache(self._h, layer, int(value), out.ctypes.data, out.size),
                    "vkl_model_read_kv_cache")
        return out.view(np.float16)

    def write_kv_cache(self, layer, value, rows):
        """rows: float16 [heads, maxlen, head_dim], the whole cache of the layer"""
        rows = np.ascontiguousarray(rows, np.float16)
        self._check(lib().vkl_model_write_kv_cache(self._h, layer, int(value), rows.ctypes.data, rows.size),
                    "vkl_model_write_kv_cache")

    def decode_recoveries(self):
        return int(lib().vkl_model_decode_recoveries(self._h))

    def decode_step_bytes(self, L):
        return int(lib().vkl_model_decode_step_bytes(self._h, L))

    PHASES = ("kqv", "attention", "wo", "upgate", "down", "lm_head", "argmax", "unused", "layer")

    def phase_times(self):
        """{phase: (milliseconds summed, launches)} since the last call; filled
        while the option "phase_timing" is on."""
        ms = np.zeros(len(self.PHASES), np.float64)
        n = np.zeros(len(self.PHASES), np.uint64)
        self._check(lib().vkl_model_phase_times(self._h, ms.ctypes.data, n.ctypes.data), "phase_times")
        return {k: (float(ms[i]), int(n[i])) for i, k in enumerate(self.PHASES)}

    def phase_replay(self, kind, pos, rounds):
        """Average microseconds per launch of one phase kernel launched back
        to back (all layers, `rounds` times) between one pair of HIP events."""
        ms, n = C.c_double(0), C.c_uint64(0)
        self._check(lib().vkl_model_phase_replay(self._h, self.PHASES.index(kind), pos, rounds, C.byref(ms),
                                                 C.byref(n)), "phase_replay")
        return ms.value * 1e3, int(n.value)

    def phase_bytes(self, kind, L):
        return int(lib().vkl_model_phase_bytes(self._h, self.PHASES.index(kind), L))
