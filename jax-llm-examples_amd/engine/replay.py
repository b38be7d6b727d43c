"""Trace replay: feeds given token ids through the model step by step and writes
logits.  It samples nothing and has no forward pass, cache or loader of its
own: it drives :class:`~.runner.ModelRunner`, the same step function, cache
manager and kernels that generation uses.

Input (standard input, one JSON object per line)::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits
at the wanted places, in the order of the entries and of ``want``, as
little-endian float32 ``[wanted, vocab]``.  After every step a line
``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch

from ..cache.manager import CacheManager
from .batch import StepEntry
from .loading import get_ops, load_model, parse_dtype
from .runner import ModelRunner

def make_runner(model_dir: str, dtype, max_tokens: int, device: str = "cuda:0", page_size: int = 16,
                max_requests: int = 8, reference_ops: bool = False, poison: bool = False,
                decode_graphs=None) -> ModelRunner:
    """``max_tokens``: the most tokens live requests hold at any time, each request's count rounded
    up to a multiple of 64; every group's pool is made for that many (plus a page per request, for
    counts that are rounded to pages here), so pages are used again.  ``max_requests``: requests
    that may be live at once."""
    dtype = parse_dtype(dtype)
    ops = get_ops(device, reference_ops=reference_ops)
    model = load_model(model_dir, dtype, device)
    rounded = -(-max_tokens // 64) * 64
    num_pages = -(-rounded // page_size) + max_requests
    cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=num_pages,
                         max_requests=max_requests, dtype=dtype, device=device, poison=poison)
    return ModelRunner(model, cache, ops, decode_graphs=decode_graphs)


def replay(runner: ModelRunner, lines, out_dir: str, out=sys.stdout) -> None:
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", ())) for e in rec.get("entries", ())]
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                arr = logits.detach().to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", ()):
            runner.finish(rid)
        print(f"done {step}", file=out, flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-requests", type=int, default=8, help="requests that may be live at once")
    ap.add_argument("--poison", action="store_true",
                    help="fill the page pools with NaN, and every page again when it is given back: a page that is "
                         "read without having been written by its present holder then shows in the logits")
    ap.add_argument("--no-decode-graphs", action="store_true",
                    help="run steps of single tokens launch by launch instead of replaying recorded HIP graphs")
    args = ap.parse_args(argv)
    runner = make_runner(args.model, args.dtype, args.max_tokens, args.device, args.page_size, args.max_requests,
                         poison=args.poison, decode_graphs=False if args.no_decode_graphs else None)
    replay(runner, sys.stdin, args.out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
