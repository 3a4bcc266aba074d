#!/usr/bin/env python3
"""Generate from a model directory of any served architecture (``config.json`` decides: the registry in
``jacobiforcing_amd.modeling``), through ``LLM.generate`` and its scheduler.

    python -m jacobiforcing_amd.drivers.generate --model DIR --prompts prompts.json --max-tokens 64
    python -m jacobiforcing_amd.drivers.generate --model DIR --synthetic 8 --prompt-len 200 --temperature 0.8

``prompts.json`` holds a list of token-id lists (or of strings, when the directory has a tokenizer).  Prints one JSON object per
request ({"prompt_tokens", "token_ids", "text"}) and a last line with tokens per second.  A ragged family (Lokizen, Vumalix, Bamanex, Mikipel) runs prompt
portions and decoded tokens of different requests in one batch per step; ``--max-num-batched-tokens`` is the step's budget and
``--page`` the size of a cache page."""
from __future__ import annotations

import argparse
import json
import random
import sys
import time


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompts", default=None, help="JSON file: a list of token-id lists or strings")
    ap.add_argument("--synthetic", type=int, default=4, help="without --prompts: this many random prompts")
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--max-tokens", type=int, default=64)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--dtype", default="auto", choices=("auto", "bfloat16", "float32"))
    ap.add_argument("--page", type=int, default=0, help="cache page size (0: 64 for a ragged family, 256 otherwise)")
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--max-model-len", type=int, default=8192)
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--seed", type=int, default=1234)
    a = ap.parse_args(argv)
    from .. import SamplingParams
    from ..llm import LLM
    from ..modeling import family_of, read_model_config
    hf = read_model_config(a.model)
    page = a.page or (64 if family_of(hf) == "ragged" else 256)
    if a.prompts:
        prompts = json.loads(open(a.prompts).read())
    else:
        rng = random.Random(a.seed)
        prompts = [[rng.randrange(hf.vocab_size) for _ in range(a.prompt_len)] for _ in range(a.synthetic)]
    tok = None if any(isinstance(p, str) for p in prompts) else "none"
    llm = LLM(a.model, tokenizer_path=tok, dtype=a.dtype, kvcache_block_size=page, max_num_seqs=a.max_num_seqs, max_model_len=a.max_model_len,
              max_num_batched_tokens=max(a.max_num_batched_tokens, a.max_model_len))
    sp = SamplingParams(temperature=a.temperature, max_tokens=a.max_tokens, ignore_eos=hf.eos_token_id < 0)
    t0 = time.perf_counter()
    out = llm.generate(prompts, sp, use_tqdm=False)
    dt = time.perf_counter() - t0
    for p, o in zip(prompts, out):
        print(json.dumps({"prompt_tokens": len(p), "token_ids": o["token_ids"], "text": o["text"]}))
    n = sum(len(o["token_ids"]) for o in out)
    print(json.dumps({"requests": len(out), "new_tokens": n, "seconds": round(dt, 3), "tokens_per_s": round(n / max(dt, 1e-9), 1)}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
