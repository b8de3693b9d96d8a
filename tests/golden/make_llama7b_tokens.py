#!/usr/bin/env python3
"""Writes tests/golden/llama7b_q4_0_tokens.json: the greedy continuation of the random-init
7B-shape Q4_0 model (prompt 128, 256 new tokens, fp16 KV cache) as computed by the CPU checker
in oracle/, with, for every step, the top-2 logit margin, the largest logit magnitude and the
logits at eight fixed vocabulary indices.

The model is litenn_amd.synth.llama_7b_q4_0 with the model seed below, the prompt is
synth.prompt_tokens of the prompt seed; a GPU test rebuilds both from the seeds and compares the
device's tokens, margins and probe logits with this file.  The prompt seed was chosen among 700 by
running the device's own decoder: the one whose continuation has at least 64 distinct tokens and the
widest smallest margin (with a vocabulary of 32000 the median margin of a step is 4 % of the largest
logit and the smallest of 256 steps is typically 1e-4 of it, where rounding differences between two
correct implementations could pick the other token).  The checker then has the last word: this
script asserts on ITS tokens and margins, and refuses to write a fixture that repeats itself or has
a step closer than 1e-3 of the largest logit.

Takes about a quarter of an hour on 8 cores (every token streams 3.7 GB of quantised weights
through the checker); progress goes to stderr and the partial state is kept in the output file:
an interrupted run feeds the tokens it already has back through the checker, checks that they
come out again and carries on.

Usage: python tests/golden/make_llama7b_tokens.py [--prompt 128] [--new 256] [--seed 4] [--prompt-seed 618]
       [--out FILE] [--checkpoint FILE.npz]
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
PROBES = [0, 1, 4099, 8191, 12345, 20000, 27182, 31999]  # vocabulary indices whose logits are kept
MIN_DISTINCT = 32
MIN_REL_MARGIN = 1e-3


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--new", type=int, default=256)
    ap.add_argument("--seed", type=int, default=4)
    ap.add_argument("--prompt-seed", type=int, default=618)
    ap.add_argument("--threads", type=int, default=os.cpu_count() or 1)
    ap.add_argument("--out", default=OUT)
    ap.add_argument("--checkpoint", default=None,
                    help="file (.npz) that keeps the checker's cache between runs; without it a resumed run "
                         "feeds the saved tokens through the checker again")
    args = ap.parse_args()

    from litenn_amd import synth
    from oracle import oracle as orc
    from llama_util import oracle_model

    orc.build()
    orc.set_threads(args.threads)
    cfg = synth.llama_7b_q4_0(context_length=args.prompt + args.new)
    prompt = synth.prompt_tokens(cfg, args.prompt, args.prompt_seed)
    head = {"model": cfg.name, "seed": args.seed, "prompt_seed": args.prompt_seed,
            "context_length": cfg.context_length, "kv_cache": "f16", "prompt_length": args.prompt,
            "prompt_head": prompt[:8].tolist(), "probe_indices": PROBES}
    done = {"tokens": [], "margins": [], "logit_absmax": [], "probes": []}
    if os.path.exists(args.out):
        try:
            with open(args.out) as f:
                old = json.load(f)
            if all(old.get(k) == v for k, v in head.items()) and not old.get("complete"):
                done = {k: old[k] for k in done}
                print(f"resuming after {len(done['tokens'])} tokens", file=sys.stderr, flush=True)
        except (OSError, ValueError, KeyError):
            pass
    t0 = time.time()
    model = oracle_model(orc, cfg, args.seed, kv_f16=True)
    print(f"model built in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)

    def save_state(n_prompt_done):
        """Cache rows and position beside the lists, so that a run that is cut off carries on from
        its last save instead of feeding everything through the checker again."""
        if not args.checkpoint:
            return
        past = model.past
        kv = [model.get_kv(layer) for layer in range(cfg.block_count)]
        tmp = args.checkpoint + ".tmp.npz"
        np.savez(tmp, k=np.stack([k for k, _ in kv]), v=np.stack([v for _, v in kv]), past=past,
                 n_prompt_done=n_prompt_done, n_tokens=len(tokens), head=json.dumps(head, sort_keys=True))
        os.replace(tmp, args.checkpoint)

    def save_lists(complete):
        tmp = args.out + ".tmp"
        with open(tmp, "w") as f:
            json.dump({**head, "new_tokens": len(tokens), "complete": complete, "tokens": tokens,
                       "margins": margins, "logit_absmax": absmax, "probes": probes,
                       "source": "oracle/litenn_oracle.c via tests/golden/make_llama7b_tokens.py"}, f)
        os.replace(tmp, args.out)

    known = list(done["tokens"])
    tokens, margins, absmax, probes = [], [], [], []
    prompt_done = 0
    if args.checkpoint and os.path.exists(args.checkpoint):
        with np.load(args.checkpoint) as ck:
            n_saved = int(ck["n_tokens"])
            if str(ck["head"]) == json.dumps(head, sort_keys=True) and n_saved <= len(known):
                for layer in range(cfg.block_count):
                    model.set_kv(layer, ck["k"][layer], ck["v"][layer])
                model.set_past(int(ck["past"]))
                prompt_done = int(ck["n_prompt_done"])
                tokens, margins = known[:n_saved], list(done["margins"][:n_saved])
                absmax, probes = list(done["logit_absmax"][:n_saved]), list(done["probes"][:n_saved])
                print(f"cache restored at position {model.past}: {prompt_done} prompt tokens, {n_saved} steps",
                      file=sys.stderr, flush=True)

    # The prompt goes in one token at a time: every row of the checker's result is independent
    # of how many rows are evaluated together, and single rows keep its working set in cache.
    t1 = time.time()
    for i in range(prompt_done, args.prompt - 1):
        model.eval([int(prompt[i])], all_logits=False)
        if i % 16 == 15:
            print(f"prompt {i + 1}/{args.prompt} ({time.time() - t1:.0f} s)", file=sys.stderr, flush=True)
            save_state(i + 1)
    feed = [int(prompt[-1])] if not tokens else [tokens[-1]]
    for step in range(len(tokens), args.new):
        t1 = time.time()
        logits = model.eval(feed, all_logits=False)
        best = int(np.argmax(logits))  # first maximal index, like the runtime's arg-max
        rest = logits.copy()
        rest[best] = -np.inf
        if step < len(known) and known[step] != best:
            print(f"step {step}: the saved token {known[step]} does not come out again ({best})", file=sys.stderr)
            return 1
        tokens.append(best)
        margins.append(float(logits[best] - rest.max()))
        absmax.append(float(np.abs(logits).max()))
        probes.append([float(logits[i]) for i in PROBES])
        feed = [best]
        print(f"step {step}: token {best} margin {margins[-1]:.4g} of {absmax[-1]:.4g} ({time.time() - t1:.1f} s)",
              file=sys.stderr, flush=True)
        if (step % 8 == 7 and step >= len(known)) or step == args.new - 1:
            complete = len(tokens) == args.new
            if complete:
                rel = np.array(margins) / np.array(absmax)
                distinct = len(set(tokens))
                print(f"{distinct} distinct tokens, smallest margin {rel.min():.3e} of the largest logit",
                      file=sys.stderr, flush=True)
                assert distinct >= MIN_DISTINCT, f"only {distinct} distinct tokens: the continuation repeats itself"
                assert rel.min() >= MIN_REL_MARGIN, f"a step is decided by {rel.min():.2e} of the largest logit"
            save_lists(complete)
            save_state(args.prompt - 1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
