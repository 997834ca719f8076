"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled.  The replay drives the engine's own model, step function,
cache manager and kernels; it only translates trace lines into step entries.
One JSON object per line on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: for each request its next tokens and the places among them whose
logits are wanted; all entries of a step run as one batch.  ``end``: requests
that are finished after the step; their pages and slot go back to the pools.
For a step with wanted places the logits are written to ``<out>/<step>.f32``
(little-endian float32, [wanted, vocab], in the order of the entries and of
``want``).  After every step a line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch


def page_rounded_tokens(max_tokens: int, page_size: int) -> int:
    """Pages for ``max_tokens`` tokens when each live request's count is rounded up to the
    larger of 64 and the page size."""
    unit = max(64, page_size)
    rounded = -(-max_tokens // unit) * unit
    return -(-rounded // page_size)


def run(argv=None, stdin=None, stdout=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--kvcache-block-size", type=int, default=16, help="tokens in a cache page")
    ap.add_argument("--max-num-seqs", type=int, default=8, help="most live requests")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--poison-cache", action="store_true",
                    help="fill the cache pool with NaN before the first step: a read of a slot that no step wrote shows in the logits")
    args = ap.parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout

    from ..kernels import ops
    from .batch import StepEntry
    from .runner import ModelRunner, load_model

    os.makedirs(args.out, exist_ok=True)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    ops.hip()       # builds the kernel library at the first call, and fails here if there is no GPU
    model = load_model(args.model, args.dtype, args.device)
    num_pages = page_rounded_tokens(args.max_tokens, args.kvcache_block_size)
    runner = ModelRunner(model, args.dtype, args.device, args.kvcache_block_size, num_pages, args.max_num_seqs,
                         max_num_batched_tokens=1 << 30)
    if args.poison_cache:
        runner.storage.fill(float("nan"))
    live = {}
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for ent in rec.get("entries", []):
            rid = ent["id"]
            tokens = [int(t) for t in ent["tokens"]]
            if not tokens:
                continue
            rc = live.get(rid)
            if rc is None:
                rc = live[rid] = runner.manager.admit(rid)
            runner.manager.reserve(rc, len(tokens))
            entries.append(StepEntry(rc, tokens, [int(w) for w in ent.get("want", [])]))
        logits = runner.step(entries) if entries else None        # a line may only end requests
        if logits is not None and logits.shape[0] > 0:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, "%s.f32.tmp" % step)
            data.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, "%s.f32" % step))
        for rid in rec.get("end", []):
            rc = live.pop(rid, None)
            if rc is not None:
                runner.manager.release(rc)
        stdout.write("done %s\n" % step)
        stdout.flush()
    return 0
