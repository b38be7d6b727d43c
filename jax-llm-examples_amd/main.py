"""Command line: from a model folder to generated token ids.

The reference's ``llama4/main.py`` has no options (fixed checkpoint path, three
prompts, 32 decode steps, ``main.py:44-74``); its serving mains name theirs
``--ckpt-path``, ``--max-seq-len``, ``--decode-batch-size`` and ``--max-decode-length``
(``serving/main_serving_gemma4.py:164-170``), and its samplers ``sample_temp`` and
``sample_topk``.  Those names are kept.  Prompts are token ids (no tokenizer here).

    python -m jax_llm_examples_amd.main --ckpt-path DIR --prompt-ids 1,2,3 --max-decode-length 32
    python -m jax_llm_examples_amd.main --random-weights tiny --write-model DIR --seed 0
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import torch


def _parse_prompts(args, vocab: int) -> list:
    prompts = []
    for s in args.prompt_ids or []:
        prompts.append([int(t) for t in s.replace(" ", "").split(",") if t])
    if args.prompt_file:
        with open(args.prompt_file) as f:
            for line in f:
                line = line.strip()
                if line:
                    prompts.append(json.loads(line) if line.startswith("[") else [int(t) for t in line.split(",")])
    if args.random_prompts:
        g = torch.Generator().manual_seed(args.seed)
        for _ in range(args.random_prompts):
            prompts.append(torch.randint(0, vocab, (args.prompt_len,), generator=g).tolist())
    if not prompts:
        raise SystemExit("no prompts: give --prompt-ids, --prompt-file or --random-prompts")
    return prompts


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="jax_llm_examples_amd.main", description=__doc__.split("\n\n")[0])
    ap.add_argument("--ckpt-path", help="model folder: config.json and model.safetensors")
    ap.add_argument("--random-weights", metavar="CONFIG",
                    help="no checkpoint: draw seeded random weights for this config.json file or preset name")
    ap.add_argument("--write-model", metavar="DIR", help="with --random-weights: write the model folder here and exit")
    ap.add_argument("--num-layers", type=int, help="with a preset: keep only the first layers")
    ap.add_argument("--seed", type=int, default=0, help="seed of random weights and random prompts")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may be repeated")
    ap.add_argument("--prompt-file", help="one prompt per line: comma-separated ids or a JSON list")
    ap.add_argument("--random-prompts", type=int, default=0, help="this many prompts of random token ids")
    ap.add_argument("--prompt-len", type=int, default=32)
    ap.add_argument("--max-decode-length", type=int, default=32, help="tokens to generate per prompt")
    ap.add_argument("--max-seq-len", type=int, default=4096, help="longest prompt + generation the cache is sized for")
    ap.add_argument("--decode-batch-size", type=int, default=16, help="requests running at once")
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048, help="token budget of one step")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--cache-tokens", type=int, help="tokens the page pools hold (default: batch size x max-seq-len)")
    ap.add_argument("--num-pages", type=int, help="the same in pages of --page-size tokens")
    ap.add_argument("--kv-memory-fraction", type=float,
                    help="size the page pools to this part of the device memory that is free after the weights")
    ap.add_argument("--no-decode-graphs", action="store_true",
                    help="run steps of single tokens launch by launch instead of replaying recorded HIP graphs")
    ap.add_argument("--profile", metavar="DIR",
                    help="trace the generation with the PyTorch profiler: a kernel table on stderr, a trace file in DIR")
    ap.add_argument("--sample-temp", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--sample-topk", type=int, default=0, help="sample among the k most likely tokens (0 = all)")
    ap.add_argument("--sample-seed", type=int, default=0)
    ap.add_argument("--eos-tokens", default="", help="comma-separated token ids that end a generation")
    args = ap.parse_args(argv)

    from .config.presets import PRESETS, preset
    from .config.registry import architecture_name, get_architecture
    from .engine import Engine, load_model, random_model
    from .sampling import SamplingParams
    from .weights import write_random_model

    if args.random_weights:
        if args.random_weights in PRESETS:
            top = preset(args.random_weights, args.num_layers)
        else:
            with open(args.random_weights) as f:
                top = json.load(f)
        arch = get_architecture(architecture_name(top))
        cfg = arch.parse_config(top)
        if args.write_model:
            dt = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
            write_random_model(arch, cfg, args.write_model, args.seed, dt, architecture=architecture_name(top))
            print(f"wrote {args.write_model}")
            return 0
        model = random_model(arch, cfg, args.seed, args.dtype, args.device)
    elif args.ckpt_path:
        model = load_model(args.ckpt_path, args.dtype, args.device)
    else:
        raise SystemExit("give --ckpt-path or --random-weights")

    prompts = _parse_prompts(args, model.plan.vocab_size)
    limit = getattr(getattr(model, "config", None), "max_position_embeddings", None)
    max_seq_len = args.max_seq_len if limit is None else min(args.max_seq_len, limit)
    sizing = {}
    if args.kv_memory_fraction is not None:
        sizing["kv_memory_fraction"] = args.kv_memory_fraction
    else:
        sizing["cache_tokens"] = (args.cache_tokens or (args.num_pages or 0) * args.page_size
                                  or args.decode_batch_size * max_seq_len)
    engine = Engine(model, page_size=args.page_size, decode_batch_size=args.decode_batch_size,
                    max_num_batched_tokens=args.max_num_batched_tokens, max_seq_len=max_seq_len,
                    decode_graphs=False if args.no_decode_graphs else None, **sizing)
    eos = tuple(int(t) for t in args.eos_tokens.split(",") if t)
    params = [SamplingParams(sample_temp=args.sample_temp, sample_topk=args.sample_topk,
                             seed=args.sample_seed + i, max_decode_length=args.max_decode_length, eos_tokens=eos)
              for i in range(len(prompts))]
    t0 = time.time()
    if args.profile:
        import os

        from torch.profiler import ProfilerActivity, profile

        os.makedirs(args.profile, exist_ok=True)
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            outs = engine.generate(prompts, params)
            if model.device.type == "cuda":
                torch.cuda.synchronize()
        prof.export_chrome_trace(os.path.join(args.profile, "generate_trace.json"))
        print(prof.key_averages().table(sort_by="cuda_time_total", row_limit=25), file=sys.stderr)
    else:
        outs = engine.generate(prompts, params)
        if model.device.type == "cuda":
            torch.cuda.synchronize()
    dt = time.time() - t0
    for i, o in enumerate(outs):
        print(json.dumps({"prompt": i, "tokens": o}))
    n = sum(len(o) for o in outs)
    print(f"generated {n} tokens in {dt:.2f} s ({n / dt:.1f} tok/s), {engine.scheduler.stats['steps']} steps, "
          f"{engine.scheduler.stats['preemptions']} preemptions", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
