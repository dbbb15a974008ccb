"""Greedy generation from a GGUF model file, the job of app/llama2_infer.cpp
of the reference:

    python -m vkllama_amd.infer MODEL.gguf N_TOKENS --ids 1 15043 3186
    python -m vkllama_amd.infer MODEL.gguf N_TOKENS --tokenizer tokenizer.model --prompt "Hello"

With a sentencepiece model the prompt is encoded (BOS first, as the reference
does) and the result decoded; otherwise token ids go in and come out.
"""
import argparse
import sys

import numpy as np


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model")
    ap.add_argument("n_tokens", type=int)
    ap.add_argument("--ids", type=int, nargs="*", help="prompt as token ids")
    ap.add_argument("--tokenizer", help="sentencepiece model file")
    ap.add_argument("--prompt", help="prompt text (needs --tokenizer)")
    ap.add_argument("--device", type=int, default=0)
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
