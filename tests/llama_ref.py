"""Synthetic Llama-2-shaped weights and an independent float64 forward pass.

forward_f64 is a textbook implementation (RMSNorm, rotary embedding on
adjacent pairs, causal softmax attention with a KV cache, SwiGLU, tied to the
GGUF tensor names) written with numpy in float64.  It shares no code with the
oracle and is used only to pin the oracle's wiring.
"""
import numpy as np

from oracle import oracle as O


def tensor_names(n_layers):
    names = ["token_embd.weight", "output.weight", "output_norm.weight"]
    for i in range(n_layers):
        for t in ("attn_norm", "attn_q", "attn_k", "attn_v", "attn_output", "ffn_norm", "ffn_gate", "ffn_down",
                  "ffn_up"):
            names.append("blk.%d.%s.weight" % (i, t))
    return names


def matrix_shape(cfg, name):
    d, F, V = cfg["dim"], cfg["ffn"], cfg["vocab"]
    if name in ("token_embd.weight", "output.weight"):
        return V, d
    if "ffn_gate" in name or "ffn_up" in name:
        return F, d
    if "ffn_down" in name:
        return d, F
    return d, d


def make_weights(rng, cfg, std=0.02, norm_jitter=0.1):
    """Returns (w, wf): w holds the tensors in their storage format (Q8_0 GGUF
    blocks as uint8 [N, K/32*34] or fp16 [N, K]; norm weights fp32), wf the
    same values as float64 (dequantised)."""
    w, wf = {}, {}
    for name in tensor_names(cfg["n_layers"]):
        if name.endswith("_norm.weight"):
            v = (1.0 + norm_jitter * rng.standard_normal(cfg["dim"])).astype(np.float32)
            w[name], wf[name] = v, v.astype(np.float64)
            continue
        N, K = matrix_shape(cfg, name)
        x = (rng.standard_normal((N, K)) * std).astype(np.float32)
        if cfg.get("wtype", 8) == 8:
            raw = O.quantize_q8_0(x, 2)
            w[name] = raw
            wf[name] = O.dequantize_q8_0(raw, K, 2).astype(np.float64)
        else:
            h = x.astype(np.float16)
            w[name], wf[name] = h, h.astype(np.float64)
    return w, wf


def _rmsnorm(x, w, eps):
    return x * w / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def forward_f64(cfg, wf, toks, offset, cache):
    """Logits of the last token; `cache` (dict) carries K/V between calls."""
    d, H, L = cfg["dim"], cfg["n_heads"], cfg["n_layers"]
    hd = d // H
    x = wf["token_embd.weight"][np.asarray(toks, np.int64)]           # [S, d]
    S = x.shape[0]
    pos = np.arange(offset, offset + S, dtype=np.float64)
    freq = 10000.0 ** (-np.arange(0, hd, 2, dtype=np.float64) / hd)
    ang = pos[:, None] * freq[None, :]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]         # [S, 1, hd/2]

    def rope(t):                                                        # t [S, H, hd]
        out = np.empty_like(t)
        out[..., 0::2] = t[..., 0::2] * cos - t[..., 1::2] * sin
        out[..., 1::2] = t[..., 0::2] * sin + t[..., 1::2] * cos
        return out

    for l in range(L):
        p = "blk.%d." % l
        n1 = _rmsnorm(x, wf[p + "attn_norm.weight"], cfg["eps"])
        q = rope((n1 @ wf[p + "attn_q.weight"].T).reshape(S, H, hd))
        k = rope((n1 @ wf[p + "attn_k.weight"].T).reshape(S, H, hd))
        v = (n1 @ wf[p + "attn_v.weight"].T).reshape(S, H, hd)
        kc = np.concatenate([cache.get((l, "k"), np.zeros((0, H, hd))), k])[:offset + S]
        vc = np.concatenate([cache.get((l, "v"), np.zeros((0, H, hd))), v])[:offset + S]
        cache[(l, "k")], cache[(l, "v")] = kc, vc
        sc = np.einsum("shd,lhd->hsl", q, kc) / np.sqrt(hd)
        mask = np.arange(offset + S)[None, :] > (np.arange(S)[:, None] + offset)
        sc = np.where(mask[None], -np.inf, sc)
        pr = np.exp(sc - sc.max(axis=-1, keepdims=True))
        pr /= pr.sum(axis=-1, keepdims=True)
        att = np.einsum("hsl,lhd->shd", pr, vc).reshape(S, d)
        x = x + att @ wf[p + "attn_output.weight"].T
        n2 = _rmsnorm(x, wf[p + "ffn_norm.weight"], cfg["eps"])
        g = n2 @ wf[p + "ffn_gate.weight"].T
        u = n2 @ wf[p + "ffn_up.weight"].T
        x = x + (g / (1 + np.exp(-g)) * u) @ wf[p + "ffn_down.weight"].T
    xn = _rmsnorm(x[-1], wf["output_norm.weight"], 1e-6)
    return xn @ wf["output.weight"].T
