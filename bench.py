"""Decode and prefill throughput of the Llama 4 Scout layer sizes with random weights on
one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

prints one JSON line: ``value`` = decoded tokens per second at batch 8 and context 4,096
(a "step" is one decode step of the whole batch, sampling included), plus the prefill of
2,048 tokens, the decode step's HBM roofline fraction and, under ``points``, decode at other
batch sizes and context lengths (``decode_b<batch>[_c<context>]``: tokens a second, with
``..._hbm_frac``: the step's bytes / its time / 8 TB/s) and longer prefills
(``prefill_<tokens>``: tokens a second, ``..._frac`` of the dtype's MFMA peak).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0  # MI355X: HBM3E 8 TB/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}  # dense MFMA


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration's 48")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64,16,32,128@2048,8@16384,8@32768",
                    help="other decode steps to report: batch or batch@context, comma-separated")
    ap.add_argument("--prefill-points", default="8192", help="other prefill lengths to report")
    ap.add_argument("--point-steps", type=int, default=12)
    ap.add_argument("--serve", default="", help="requests through the scheduler, e.g. 64x512+128@64 (requests x prompt "
                    "+ output tokens @ decode batch), comma-separated: tokens a second end to end")
    ap.add_argument("--preset", default="llama4-scout")
    ap.add_argument("--no-prefill", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus > 1 is not supported")
        return 2

    import torch

    from jax_llm_examples_amd.cache import CacheManager
    from jax_llm_examples_amd.config.presets import PRESETS, preset
    from jax_llm_examples_amd.config.registry import architecture_name, get_architecture
    from jax_llm_examples_amd.engine import ModelRunner, StepEntry, get_ops, random_model
    from jax_llm_examples_amd.engine.accounting import StepWatcher, decode_step_bytes, prefill_flops
    from jax_llm_examples_amd.sampling import Sampler, SamplingParams

    dev = "cuda:0"
    full_layers = PRESETS[args.preset]["num_hidden_layers"]
    layers = args.layers or full_layers
    top = preset(args.preset, layers)
    arch = get_architecture(architecture_name(top))
    cfg = arch.parse_config(top)
    t0 = time.time()
    model = random_model(arch, cfg, seed=0, dtype=args.dtype, device=dev)
    torch.cuda.synchronize()
    print(f"[bench] {layers}-layer model with random weights on the GPU after {time.time() - t0:.0f} s "
          f"({model.num_parameters() / 1e9:.1f} B parameters)", file=sys.stderr, flush=True)

    page = 16
    points_at = []  # (batch, context)
    for spec in args.points.split(","):
        if spec:
            b, _, c = spec.partition("@")
            points_at.append((int(b), int(c) if c else args.context))
    prefill_points = [] if args.no_prefill else [int(t) for t in args.prefill_points.split(",") if t]
    batches = [args.batch] + [b for b, _ in points_at]
    need_tokens = (max([args.batch * (args.context + page)] + [b * (c + page) for b, c in points_at])
                   + max([args.prefill_tokens] + prefill_points) + 4 * page)
    ops = get_ops(dev)
    cache = CacheManager(model.cache_needs(), page_size=page, num_pages=-(-need_tokens // page),
                         max_requests=max(batches) + 1, dtype=model.dtype, device=dev)
    for g in cache.groups:  # stand-in keys and values for contexts that are not computed
        for t in g.tensors.values():
            step = max(1, (1 << 28) // max(1, t[0].numel()))
            for o in range(0, t.shape[0], step):
                t[o: o + step].normal_(0.0, 0.5)
    runner = ModelRunner(model, cache, ops)
    sampler = Sampler(ops, dev)
    gen = torch.Generator().manual_seed(0)
    V = model.plan.vocab_size
    greedy = SamplingParams()
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"

    # ------------------------------------------------------------------ prefill of 2,048 tokens
    def run_prefill(T: int, tries: int):
        times = []
        for it in range(tries):
            toks = torch.randint(0, V, (T,), generator=gen).tolist()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            logits = runner.step([StepEntry(f"p{T}_{it}", toks, [T - 1])])
            sampler(logits, [greedy], [0])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t1)
            runner.finish(f"p{T}_{it}")
            print(f"[bench] prefill of {T} tokens: {times[-1] * 1e3:.1f} ms", file=sys.stderr, flush=True)
        sec = min(times[1:])
        return sec, prefill_flops(model, T) / sec / PEAK_FLOPS[dkey]

    prefill = None
    if not args.no_prefill:
        T = args.prefill_tokens
        sec, frac = run_prefill(T, 3)
        prefill = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 2), "frac": round(frac, 4)}

    # ------------------------------------------------------------------ decode
    def decode(batch: int, steps: int, warmup: int, context: int):
        ctx0 = context - (steps + warmup)
        ids = [f"d{batch}_{context}_{i}" for i in range(batch)]
        for rid in ids:  # contexts stand in: pages are taken, their contents are the random fill
            cache.add_request(rid)
            cache.reserve(rid, ctx0)
            cache.commit(rid)
        last = torch.randint(0, V, (batch,), generator=gen).tolist()
        params, ctr = [greedy] * batch, [0] * batch

        def one(tap=None):
            nonlocal last
            logits = runner.step([StepEntry(r, [t], [0]) for r, t in zip(ids, last)], tap=tap)
            last = sampler(logits, params, ctr)

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t1) / steps
        # three more steps, watched: which experts their tokens choose (a watched step runs launch by launch);
        # the step's bytes are the mean over them (the count of distinct experts wanders from step to step)
        totals, weights_b, kv_b, counts = [], [], [], []
        for _ in range(3):
            watcher = StepWatcher()
            one(tap=watcher)
            counts += [int(torch.unique(seen["routing"][0]).numel()) for b in model.blocks
                       for seen in [watcher.seen.get(id(b.feed_forward))] if seen and "routing" in seen]
            nb = decode_step_bytes(model, cache, [cache.num_tokens(r) for r in ids], watcher)
            totals.append(nb["total"])
            weights_b.append(nb["weights"])
            kv_b.append(nb["kv"])
        nbytes = {"total": sum(totals) / 3, "weights": sum(weights_b) / 3, "kv": sum(kv_b) / 3}
        distinct = {i: c for i, c in enumerate(counts)}
        for rid in ids:
            runner.finish(rid)
        print(f"[bench] decode batch {batch} at context {context}: {sec * 1e3:.2f} ms/step, {batch / sec:.1f} tok/s, "
              f"{nbytes['total'] / 1e9:.1f} GB/step -> {nbytes['total'] / sec / 1e9:.0f} GB/s", file=sys.stderr,
              flush=True)
        return sec, nbytes, (sum(distinct.values()) / max(1, len(distinct)))

    sec, nbytes, mean_experts = decode(args.batch, args.steps, args.warmup, args.context)
    points = {}
    for b, c in points_at:
        s_, nb, _ = decode(b, args.point_steps, 2, c)
        key = f"decode_b{b}" + (f"_c{c}" if c != args.context else "")
        points[key] = round(b / s_, 1)
        points[key + "_hbm_frac"] = round(nb["total"] / s_ / 1e9 / PEAK_HBM_GBS, 4)
    for T in prefill_points:
        s_, frac = run_prefill(T, 2)
        points[f"prefill_{T}"] = round(T / s_, 1)
        points[f"prefill_{T}_frac"] = round(frac, 4)

    # ------------------------------------------------------------------ whole requests through the scheduler
    for spec in [v for v in args.serve.split(",") if v]:
        from jax_llm_examples_amd.engine.engine import Engine
        reqs_s, _, rest = spec.partition("x")
        plen_s, _, rest = rest.partition("+")
        olen_s, _, dbs_s = rest.partition("@")
        nreq, plen, olen = int(reqs_s), int(plen_s), int(olen_s)
        dbs = int(dbs_s) if dbs_s else min(nreq, 64)
        eng = Engine(model, cache_tokens=dbs * (plen + olen + 4 * page), decode_batch_size=dbs, page_size=page,
                     max_num_batched_tokens=2048, max_seq_len=plen + olen + 8)
        prompts = [torch.randint(0, V, (plen,), generator=gen).tolist() for _ in range(nreq)]
        # (every other request samples with a temperature; none ends early)
        sp = [SamplingParams(max_decode_length=olen, sample_temp=0.0 if i % 2 == 0 else 0.8, seed=i, ignore_eos=True)
              for i in range(nreq)]
        eng.generate(prompts[:dbs], [SamplingParams(max_decode_length=4, ignore_eos=True)] * min(nreq, dbs))  # records
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        outs = eng.generate(prompts, sp)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t1
        made = sum(len(o) for o in outs)
        print(f"[bench] {nreq} requests of {plen} + {olen} tokens, at most {dbs} decoding together: {dt:.2f} s, "
              f"{made / dt:.0f} generated tok/s, {(made + nreq * plen) / dt:.0f} processed tok/s", file=sys.stderr,
              flush=True)
        points[f"serve_{nreq}x{plen}+{olen}_b{dbs}"] = round(made / dt, 1)
        del eng
        torch.cuda.empty_cache()

    achieved = nbytes["total"] / sec / 1e9
    out = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} "
                  f"(Llama 4 {args.preset.split('-')[-1].capitalize()} layer sizes, random weights)",
        "value": round(args.batch / sec, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey,
        "data": "synthetic: random token ids, seeded random weights, decode contexts filled with random keys/values",
        "config": {
            "model": args.preset, "num_layers": layers, "num_layers_full": full_layers,
            "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "num_experts": cfg.num_local_experts,
            "experts_per_tok": cfg.num_experts_per_tok, "expert_intermediate": cfg.intermediate_size,
            "mlp_intermediate": cfg.intermediate_size_mlp, "vocab_size": cfg.vocab_size,
            "attention_chunk": cfg.attention_chunk_size, "global_batch": args.batch, "seq_len": args.context,
            "prefill_tokens": args.prefill_tokens, "page_size": page, "parallelism": "single-gpu",
            "mean_distinct_experts": round(mean_experts, 2),
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
