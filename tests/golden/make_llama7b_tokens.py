#!/usr/bin/env python3
"""Writes tests/golden/llama7b_q4_0_tokens.json: the greedy continuation of the random-init
7B-shape Q4_0 model (prompt 128, 256 new tokens, fp16 KV cache) as computed by the CPU checker
in oracle/, with the top-2 logit margin of every step.

The model is litenn_amd.synth.llama_7b_q4_0 with the seed below, the prompt is
synth.prompt_tokens of the same seed; a GPU test rebuilds both from the seed and compares the
device's tokens with this file.  Takes tens of minutes on 8 cores (every token streams 3.7 GB of
quantised weights through the checker); progress goes to stderr and the partial state is kept
in the output file so an interrupted run resumes.

Usage: python tests/golden/make_llama7b_tokens.py [--prompt 128] [--new 256] [--seed 4]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

OUT = os.path.join(HERE, "llama7b_q4_0_tokens.json")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--new", type=int, default=256)
    ap.add_argument("--seed", type=int, default=4)
    ap.add_argument("--threads", type=int, default=os.cpu_count() or 1)
    args = ap.parse_args()

    from litenn_amd import synth
    from oracle import oracle as orc
    from llama_util import oracle_model

    orc.build()
    orc.set_threads(args.threads)
    cfg = synth.llama_7b_q4_0(context_length=args.prompt + args.new)
    prompt = synth.prompt_tokens(cfg, args.prompt, args.seed)
    t0 = time.time()
    model = oracle_model(orc, cfg, args.seed, kv_f16=True)
    print(f"model built in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)

    # The prompt goes in one token at a time: every row of the checker's result is independent
    # of how many rows are evaluated together, and single rows keep its working set in cache.
    t1 = time.time()
    for i, tok in enumerate(prompt[:-1]):
        model.eval([int(tok)], all_logits=False)
        if i % 16 == 15:
            print(f"prompt {i + 1}/{args.prompt} ({time.time() - t1:.0f} s)", file=sys.stderr, flush=True)
    tokens: list[int] = []
    margins: list[float] = []
    feed = [int(prompt[-1])]
    for step in range(args.new):
        t1 = time.time()
        logits = model.eval(feed, all_logits=False)
        best = int(np.argmax(logits))  # first maximal index, like the runtime's arg-max
        rest = logits.copy()
        rest[best] = -np.inf
        tokens.append(best)
        margins.append(float(logits[best] - rest.max()))
        feed = [best]
        print(f"step {step}: token {best} margin {margins[-1]:.4g} ({time.time() - t1:.1f} s)", file=sys.stderr,
              flush=True)
        if step % 16 == 15 or step == args.new - 1:
            with open(OUT, "w") as f:
                json.dump({
                    "model": cfg.name, "seed": args.seed, "context_length": cfg.context_length, "kv_cache": "f16",
                    "prompt_length": args.prompt, "prompt_head": prompt[:8].tolist(), "new_tokens": len(tokens),
                    "complete": len(tokens) == args.new, "tokens": tokens, "margins": margins,
                    "source": "oracle/litenn_oracle.c via tests/golden/make_llama7b_tokens.py",
                }, f)
    return 0


if __name__ == "__main__":
    sys.exit(main())
