"""Generation from a GGUF model file, the job of app/llama2_infer.cpp of the
reference:

    python -m vkllama_amd.infer MODEL.gguf N_TOKENS --ids 1 15043 3186
    python -m vkllama_amd.infer MODEL.gguf N_TOKENS --tokenizer tokenizer.model --prompt "Hello"
    python -m vkllama_amd.infer MODEL.gguf N_TOKENS --ids 1 15043 --topk 40 --seed 7

The default is the reference's TopkSampler(1), i.e. greedy, which runs with
the token pick on the device; --topk K / --topp P draw on the host from the
logits of every step like the reference's samplers.

With a sentencepiece model the prompt is encoded (BOS first, as the reference
does) and the result decoded; otherwise token ids go in and come out.
"""
import argparse
import sys

import numpy as np


def generate_sampled(m, ids, n_tokens, topk=None, topp=None, seed=None):
    """Token loop of app/llama2_infer.cpp:140-177 with a host sampler: logits of
    the last row come back every step and the sampler picks the next token."""
    import time
    from . import model as M
    sampler = M.Sampler("topp", topp, seed) if topp is not None else M.Sampler("topk", topk, seed)
    toks, offset, out = list(ids), 0, []
    t0 = time.perf_counter()
    t1 = t0
    for i in range(n_tokens):
        logits = m.forward(np.array(toks, np.uint32), offset)
        if i == 0:
            t1 = time.perf_counter()
        nxt = sampler.sample(logits)
        out.append(nxt)
        offset += len(toks)
        toks = [nxt]
    t2 = time.perf_counter()
    sampler.close()
    return np.array(out, np.uint32), (t1 - t0) * 1e3, (t2 - t1) * 1e3


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model")
    ap.add_argument("n_tokens", type=int)
    ap.add_argument("--ids", type=int, nargs="*", help="prompt as token ids")
    ap.add_argument("--tokenizer", help="sentencepiece model file")
    ap.add_argument("--prompt", help="prompt text (needs --tokenizer)")
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--topk", type=int, help="draw from the K most likely tokens (1 = greedy)")
    ap.add_argument("--topp", type=float, help="draw from the smallest set of tokens with probability mass P")
    ap.add_argument("--seed", type=int, help="seed of the sampler (default: random device)")
    ap.add_argument("--device-sampler", action="store_true",
                    help="draw on the device (no logits download per token); needs --seed or uses seed 0")
    args = ap.parse_args(argv)

    sp = None
    if args.tokenizer:
        import sentencepiece
        sp = sentencepiece.SentencePieceProcessor()
        sp.Load(args.tokenizer)
    if args.prompt is not None:
        if sp is None:
            ap.error("--prompt needs --tokenizer")
        ids = [sp.bos_id()] + sp.Encode(args.prompt)
    elif args.ids:
        ids = args.ids
    else:
        ap.error("give --ids or --prompt")

    from . import model as M
    m = M.Llama2.from_gguf(args.model, args.device)
    sampled = args.topp is not None or (args.topk or 1) > 1
    if sampled and args.device_sampler:
        out, prefill_ms, decode_ms = m.generate_sampled(np.array(ids, np.uint32), args.n_tokens, args.topk or 40,
                                                        args.topp, args.seed or 0)
    elif sampled:
        out, prefill_ms, decode_ms = generate_sampled(m, ids, args.n_tokens, args.topk, args.topp, args.seed)
    else:
        out, prefill_ms, decode_ms = m.generate_greedy(np.array(ids, np.uint32), args.n_tokens)
    m.close()
    print("ids:", " ".join(str(int(t)) for t in out))
    if sp is not None:
        print(sp.Decode([int(t) for t in out]))
    n = max(args.n_tokens - 1, 1)
    print("prompt %d tokens in %.1f ms; %d tokens in %.1f ms (%.1f tok/s)"
          % (len(ids), prefill_ms, args.n_tokens - 1, decode_ms, n / max(decode_ms, 1e-9) * 1e3), file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
