#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at OPT-6.7B size with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model 6.7b|350m|1.3b|2.7b|13b|30b|66b] [--mix]

One JSON line: `value` is decoded tokens per second at batch 8 and a 2,048-token context
(a "step" is one decode step of the whole engine: schedule, model, sampling);
`prefill` is one 2,048-token prompt in one step; `roofline` sets the bytes a decode step has
to read (every weight once, and the cache of the live requests) against its time; `points`
holds decoding at batch 1 and 64 (tokens a second, milliseconds a step, share of the memory roofline) and the
whole way of batch 8 from 512-token prompts to the 2,048-token context (mean tokens a second, its share of the
roofline at the mean context, and the percentiles of the time between two steps). The measuring follows the reference's own benchmark
(generation_demo.py:107-187: warm-up runs, then timed ones; random token ids as prompts,
:492-494). Weights and prompts are synthetic and seeded; there are no published numbers of
the reference to compare with, so `vs_baseline` is null.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# OPT-6.7B: the measurement of record
MODEL = dict(architectures=["OPTForCausalLM"], model_type="opt", vocab_size=50272, hidden_size=4096,
             num_hidden_layers=32, num_attention_heads=32, ffn_dim=16384, max_position_embeddings=2048,
             word_embed_proj_dim=4096, do_layer_norm_before=True, activation_function="relu", enable_bias=True,
             layer_norm_elementwise_affine=True, init_std=0.02, torch_dtype="bfloat16")
# More members of the family, for `--model` (the default run and its JSON line stay OPT-6.7B)
OTHER_MODELS = {
    "350m": dict(hidden_size=1024, num_hidden_layers=24, num_attention_heads=16, ffn_dim=4096, word_embed_proj_dim=512,
                 do_layer_norm_before=False),
    "1.3b": dict(hidden_size=2048, num_hidden_layers=24, num_attention_heads=32, ffn_dim=8192, word_embed_proj_dim=2048),
    "2.7b": dict(hidden_size=2560, num_hidden_layers=32, num_attention_heads=32, ffn_dim=10240, word_embed_proj_dim=2560),
    "13b": dict(hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, ffn_dim=20480, word_embed_proj_dim=5120),
    "30b": dict(hidden_size=7168, num_hidden_layers=48, num_attention_heads=56, ffn_dim=28672, word_embed_proj_dim=7168),
    "66b": dict(hidden_size=9216, num_hidden_layers=64, num_attention_heads=72, ffn_dim=36864, word_embed_proj_dim=9216),
}
CONTEXT = 2048
PREFILL_TOKENS = 2048
PEAK_HBM_GBS = 8000.0                      # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def prefill_flops(cfg, tokens):
    """Multiply-adds times two of one whole prompt: the matrix products of every layer, causal
    attention (half of the square), and the head for the last token."""
    h, f, l = cfg["hidden_size"], cfg["ffn_dim"], cfg["num_hidden_layers"]
    linear = 2 * tokens * l * (4 * h * h + 2 * h * f)
    attention = l * 2 * 2 * h * tokens * (tokens + 1) / 2
    head = 2 * cfg["vocab_size"] * cfg["word_embed_proj_dim"]
    return linear + attention + head


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--prefill-only", action="store_true", help="measure the prompt step alone (for profiles)")
    ap.add_argument("--model", default="6.7b", choices=["6.7b"] + sorted(OTHER_MODELS),
                    help="layer sizes: OPT-6.7B (the measurement of record) or another member of the family")
    ap.add_argument("--do-sample", action="store_true",
                    help="decode with temperature 0.8, top-k 50 and top-p 0.95 instead of greedily")
    ap.add_argument("--mix", action="store_true",
                    help="instead: 64 requests with prompts of 16 to 1,024 tokens and 256 new tokens each, all "
                         "queued at once (a continuous-batching workload); prints its own line")
    ap.add_argument("--own-products", action="store_true",
                    help="every matrix product on our own kernels (none goes to the vendor library)")
    ap.add_argument("--tune-all", action="store_true",
                    help="time the vendor library's candidates for the many-rows products too")
    ap.add_argument("--big-batch", type=int, default=64, help="the larger batch of `points` (cut to what fits the device at the full context)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import runner_from_random
    from transformers_neuronx_amd.sampling import SamplingParams

    if args.own_products:
        from transformers_neuronx_amd.kernels.hip import HipOps
        HipOps.library_rows = 0
    if args.tune_all:
        from transformers_neuronx_amd.kernels.hip import HipOps
        HipOps.library_tune = 2
    raw = dict(MODEL)
    raw.update(OTHER_MODELS.get(args.model, {}))
    layers_full = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = OPTConfig.from_dict(raw)
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    item = 2 if dtype == torch.bfloat16 else 4
    kv_bytes_per_token = 2 * cfg.num_hidden_layers * cfg.hidden_size * item
    # the larger batch of `points` is cut to what the device holds beside the weights at the full context
    weights = item * (cfg.num_hidden_layers * (4 * cfg.hidden_size ** 2 + 2 * cfg.hidden_size * cfg.ffn_dim)
                      + (cfg.vocab_size + cfg.max_position_embeddings) * cfg.hidden_size)
    # (the random weights are drawn apart and fused afterwards: a quarter of them is held twice meanwhile, and
    # what that leaves free again is in pieces too small for the cache's blocks)
    room = int(0.95 * torch.cuda.mem_get_info()[1]) - int(1.27 * weights) - (4 << 30)
    fits = max(1, room // (kv_bytes_per_token * CONTEXT))
    if args.big_batch > fits and not (args.no_points or args.prefill_only):
        print(f"[bench] {args.big_batch} requests of {CONTEXT} tokens do not fit beside {weights / 1e9:.0f} GB of "
              f"weights; the larger batch is {fits}", file=sys.stderr, flush=True)
        args.big_batch = fits
    if args.batch > fits:
        print(f"bench.py: {args.batch} requests of {CONTEXT} tokens do not fit beside {weights / 1e9:.0f} GB of weights "
              f"on this device ({fits} do)")
        return 2
    max_batch = args.batch if args.no_points or args.prefill_only else max(args.batch, args.big_batch)
    ecfg = EngineConfig(dtype=dtype, page_size=64, max_tokens=max_batch * CONTEXT, max_num_seqs=max_batch,
                        max_num_batched_tokens=max(2048, PREFILL_TOKENS), max_model_len=CONTEXT,
                        prompts_first=True)
    t0 = time.time()
    runner = runner_from_random(cfg, seed=0, cfg=ecfg)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s "
          f"({runner.model.weight_bytes / 1e9:.2f} GB of weights"
          + (f", {runner.ops.copy_bytes / 1e9:.1f} GB of them a second time in tile order" if getattr(runner.ops, "copy_bytes", None) is not None else "")
          + ")", file=sys.stderr, flush=True)
    engine = LLMEngine(runner, ecfg)
    gen = torch.Generator().manual_seed(1)

    def decode(batch, steps, warmup, prompt_len=None, latencies=None):
        """Tokens per second, seconds per step and bytes per step of `steps` decode steps that end at
        the full context (or begin after prompts of `prompt_len` tokens)."""
        engine.reset()
        if prompt_len is None:
            prompt_len = CONTEXT - (steps + warmup) - 1
        for i in range(batch):
            params = SamplingParams(max_new_tokens=steps + warmup + 1, do_sample=args.do_sample, temperature=0.8,
                                    top_k=50, top_p=0.95, seed=i, ignore_eos=True)
            engine.add_request(torch.randint(3, cfg.vocab_size, (prompt_len,), generator=gen).tolist(), params)
        while any(not r.decoding for r in engine.requests.values()):
            engine.step()                 # prompts first: nothing decodes until every prompt is in
        assert all(len(r.output) == 1 for r in engine.requests.values())
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        start = time.perf_counter()
        lens = made = 0
        last = start
        for _ in range(steps):
            lens += sum(r.num_computed for r in engine.requests.values())
            made += len(engine.step())
            if latencies is not None:        # host time between two steps: the device sets the pace
                now = time.perf_counter()
                latencies.append(now - last)
                last = now
        torch.cuda.synchronize()
        sec = (time.perf_counter() - start) / steps
        assert made == batch * steps, f"{made} tokens in {steps} steps of batch {batch}"
        read = runner.model.weight_bytes + lens / steps * kv_bytes_per_token
        return made / (sec * steps), sec, read

    def prefill(tokens):
        engine.reset()
        params = SamplingParams(max_new_tokens=1, do_sample=False, ignore_eos=True)
        times = []
        for i in range(6):
            engine.add_request(torch.randint(3, cfg.vocab_size, (tokens,), generator=gen).tolist(), params)
            torch.cuda.synchronize()
            start = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - start)
        return sorted(times[1:])[2]       # the median of five, after one warm-up

    if args.mix:
        # every request is there at the start; the scheduler mixes portions of prompts with decoding. The
        # workload runs twice with other tokens and the second run is timed: the first loads the vendor
        # library and lets it choose its algorithms, which a server does once in its life
        params = SamplingParams(max_new_tokens=256, do_sample=False, ignore_eos=True)
        for timed in (False, True):
            engine.reset()
            lengths = torch.randint(16, 1025, (64,), generator=torch.Generator().manual_seed(2)).tolist()
            for n in lengths:
                engine.add_request(torch.randint(3, cfg.vocab_size, (n,), generator=gen).tolist(), params)
            preempted = engine.scheduler.num_preemptions
            torch.cuda.synchronize()
            start = time.perf_counter()
            first, made, steps = {}, 0, 0
            while engine.has_work:
                for o in engine.step():
                    first.setdefault(o.req_id, time.perf_counter() - start)
                    made += 1
                steps += 1
            torch.cuda.synchronize()
            sec = time.perf_counter() - start
            assert made == 64 * 256, made
        print(json.dumps({"metric": f"OPT-{args.model.upper()} continuous batching: 64 requests, prompts 16-1,024, "
                                    "256 new tokens each", "value": round(made / sec, 1), "unit": "generated tokens/s",
                          "seconds": round(sec, 3), "steps": steps, "prompt_tokens": sum(lengths),
                          "mean_time_to_first_token_ms": round(1e3 * sum(first.values()) / len(first), 2),
                          "preemptions": engine.scheduler.num_preemptions - preempted, "dtype": args.dtype,
                          "warmup": "the same workload once, untimed"}))
        return 0
    if args.prefill_only:
        sec_p = prefill(PREFILL_TOKENS)
        print(json.dumps({"prefill_ms": round(sec_p * 1e3, 3), "tokens": PREFILL_TOKENS,
                          "frac": round(prefill_flops(raw, PREFILL_TOKENS) / sec_p / PEAK_FLOPS[args.dtype], 4)}))
        return 0
    value, sec, read = decode(args.batch, args.steps, args.warmup)
    print(f"[bench] decode batch {args.batch}: {value:.1f} tok/s, {sec * 1e3:.2f} ms/step", file=sys.stderr, flush=True)
    achieved = read / sec / 1e9
    out = {
        "metric": f"OPT-{args.model.upper()} decode tok/s @ batch 1/8/{args.big_batch}; prefill tok/s @ 2,048 tokens",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random weights and token ids)"
                                      + (", sampled (temperature 0.8, top-k 50, top-p 0.95)" if args.do_sample else ""),
        "config": {"model": "OPT-" + args.model.upper(), "global_batch": args.batch, "seq_len": CONTEXT, "parallelism": "none",
                   "layers": cfg.num_hidden_layers, "layers_of_model": layers_full, "hidden_size": cfg.hidden_size,
                   "heads": cfg.num_attention_heads, "head_size": cfg.head_size, "ffn_dim": cfg.ffn_dim,
                   "vocab_size": cfg.vocab_size, "max_positions": cfg.max_position_embeddings,
                   "prompt_len": CONTEXT - args.steps - args.warmup - 1, "page_size": ecfg.page_size,
                   "activation": cfg.activation_function, "pre_norm": cfg.do_layer_norm_before,
                   "prefill_tokens": PREFILL_TOKENS},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if not args.no_points:
        sec_p = prefill(PREFILL_TOKENS)
        flops = prefill_flops(raw, PREFILL_TOKENS)
        out["prefill"] = {"value": round(PREFILL_TOKENS / sec_p, 1), "tokens": PREFILL_TOKENS,
                          "ms": round(sec_p * 1e3, 3), "frac": round(flops / sec_p / PEAK_FLOPS[args.dtype], 4)}
        print(f"[bench] prefill: {out['prefill']}", file=sys.stderr, flush=True)
        points = {}
        for b, k, w in ((1, min(args.steps, 64), args.warmup),
                        (args.big_batch, min(args.steps, 32), min(args.warmup, 4))):
            v, s, rd = decode(b, k, w)
            points[f"decode_b{b}"] = round(v, 2)
            points[f"decode_b{b}_ms"] = round(s * 1e3, 4)
            points[f"decode_b{b}_hbm_frac"] = round(rd / s / 1e9 / PEAK_HBM_GBS, 4)
            print(f"[bench] decode batch {b}: {v:.1f} tok/s, {s * 1e3:.2f} ms/step", file=sys.stderr, flush=True)
        # the whole way from 512-token prompts to the full context, as the reference's benchmark generates whole
        # sequences (generation_demo.py:159-187) and reports the percentiles of their latency
        lat = []
        first = 512
        k = CONTEXT - first - 1 - 4
        v, s, rd = decode(args.batch, k, 4, prompt_len=first, latencies=lat)
        lat.sort()
        points["decode_512_to_2048"] = round(v, 2)
        points["decode_512_to_2048_ms"] = round(s * 1e3, 4)
        points["decode_512_to_2048_hbm_frac"] = round(rd / s / 1e9 / PEAK_HBM_GBS, 4)
        for q in (0, 50, 90, 95, 99, 100):
            points[f"step_latency_p{q}_ms"] = round(lat[min(len(lat) - 1, int(len(lat) * q / 100))] * 1e3, 4)
        print(f"[bench] decode batch {args.batch}, 512 -> 2,048: {v:.1f} tok/s, {s * 1e3:.2f} ms/step",
              file=sys.stderr, flush=True)
        out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
