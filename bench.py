#!/usr/bin/env python3
"""Decode and prefill throughput of the engine with random weights; by default at OPT-6.7B's sizes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model NAME | FOLDER | CONFIG.json] [--mix] ...

One JSON line: `value` is decoded tokens per second at batch 8 and a 2,048-token context
(a "step" is one decode step of the whole engine: schedule, model, sampling);
`prefill` is one 2,048-token prompt in one step; `roofline` sets the bytes a decode step has
to read (every weight once, and the cache of the live requests) against its time; `points`
holds decoding at batch 1 and 64 (tokens a second, milliseconds a step, share of the memory roofline), the
whole way of batch 8 from 512-token prompts to the 2,048-token context (mean tokens a second, its share of the
roofline at the mean context, and the percentiles of the time between two steps), a continuous-batching mix at
OPT-350m's sizes and, where the device has room, decoding and a prompt at OPT-66B's; `ceilings` is what this
device reaches at best, measured here (a kernel that only reads memory, a loop of matrix instructions on
registers), and `roofline` / `prefill` give their shares of these beside the shares of the published peaks;
`check` compares the bfloat16 engine with a float32 engine on the same weights at full depth, by the
reference's own yardstick (generation_demo.py:437-443). The measuring follows the reference's own benchmark
(generation_demo.py:107-187: warm-up runs, then timed ones; random token ids as prompts,
:492-494). Weights and prompts are synthetic and seeded; there are no published numbers of
the reference to compare with, so `vs_baseline` is null.

The model is any registered architecture's: `--model` takes a name of the table below (config.json contents of
the OPT family), a model folder or a config.json file. Bytes and flops come from what the model's parts
declare, not from formulas of one architecture.
"""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# config.json contents by name: the measurement of record is OPT-6.7B
_OPT = dict(architectures=["OPTForCausalLM"], model_type="opt", vocab_size=50272, max_position_embeddings=2048,
            do_layer_norm_before=True, activation_function="relu", enable_bias=True,
            layer_norm_elementwise_affine=True, init_std=0.02, torch_dtype="bfloat16")
PRESETS = {
    "6.7b": dict(_OPT, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32, ffn_dim=16384, word_embed_proj_dim=4096),
    "350m": dict(_OPT, hidden_size=1024, num_hidden_layers=24, num_attention_heads=16, ffn_dim=4096, word_embed_proj_dim=512,
                 do_layer_norm_before=False),
    "1.3b": dict(_OPT, hidden_size=2048, num_hidden_layers=24, num_attention_heads=32, ffn_dim=8192, word_embed_proj_dim=2048),
    "2.7b": dict(_OPT, hidden_size=2560, num_hidden_layers=32, num_attention_heads=32, ffn_dim=10240, word_embed_proj_dim=2560),
    "13b": dict(_OPT, hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, ffn_dim=20480, word_embed_proj_dim=5120),
    "30b": dict(_OPT, hidden_size=7168, num_hidden_layers=48, num_attention_heads=56, ffn_dim=28672, word_embed_proj_dim=7168),
    "66b": dict(_OPT, hidden_size=9216, num_hidden_layers=64, num_attention_heads=72, ffn_dim=36864, word_embed_proj_dim=9216),
}
PREFILL_TOKENS = 2048
PEAK_HBM_GBS = 8000.0                      # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def log(text):
    print(f"[bench] {text}", file=sys.stderr, flush=True)


def raw_config(model: str) -> dict:
    """config.json contents for `--model`: a name of the table, a model folder or a config.json file."""
    if model in PRESETS:
        return dict(PRESETS[model], name="OPT-" + model.upper())
    path = os.path.join(model, "config.json") if os.path.isdir(model) else model
    with open(path) as fp:
        raw = json.load(fp)
    raw.setdefault("name", os.path.basename(os.path.dirname(os.path.abspath(path))))
    return raw


def keep_busy(ops, torch, seconds):
    """Reads memory for a while before anything is timed. Memory-bound steps measure some 4 % slow for two or
    three seconds after a lot of device memory has been given back, by a process that has just ended or by this
    one (an engine closed and another built): seen with one and the same program started twice in a row, and
    with engines of OPT-6.7B's sizes built one after the other in one process, each as fast as the first once
    the device had been kept reading for four seconds (4.37 against 4.58 ms a step). The cause is not
    established (the memory given back may be being cleared meanwhile; a kernel that only reads one buffer does
    not feel it). The headline is measured on the first engine of the process, after this."""
    buf = torch.empty(1 << 30, dtype=torch.uint8, device=ops.device)
    out = torch.zeros(ops.compute_units * 32, dtype=torch.float32, device=ops.device)
    end = time.time() + seconds
    while time.time() < end:
        for _ in range(20):
            ops.call("probe", "tnx_probe_stream_read", buf.data_ptr(), buf.numel(), out.data_ptr(),
                     ops.compute_units * 32, ops.stream())
        torch.cuda.synchronize(ops.device)
    del buf, out
    torch.cuda.empty_cache()


def measured_ceilings(ops, torch):
    """What a kernel of ours reaches on this device at best: GB/s of a kernel that only reads 8 GB of memory,
    TFLOP/s of a loop of bfloat16 matrix instructions whose operands stay in registers."""
    dev = ops.device
    buf = torch.empty(8 << 30, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).fill_(1)
    units = ops.compute_units
    out = torch.zeros(units * 16 * 256, dtype=torch.float32, device=dev)

    def timed(fn, repeats):
        fn()
        torch.cuda.synchronize(dev)
        best = float("inf")
        for _ in range(repeats):
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            fn()
            end.record()
            end.synchronize()
            best = min(best, start.elapsed_time(end) * 1e-3)
        return best

    read = timed(lambda: ops.call("probe", "tnx_probe_stream_read", buf.data_ptr(), buf.numel(), out.data_ptr(),
                                  units * 32, ops.stream()), 5)
    iterations, blocks = 20000, units * 8
    loop = timed(lambda: ops.call("probe", "tnx_probe_mfma_loop", blocks, iterations, out.data_ptr(), ops.stream()), 3)
    del buf, out
    torch.cuda.empty_cache()
    return {"hbm_read_gbs_measured": round(8 * (1 << 30) / read / 1e9, 1),
            "mfma_tflops_measured": round(blocks * 4 * iterations * 4 * 2 * 32 * 32 * 16 / loop / 1e12, 1)}


class Bench:
    """One model on the device and the measurements over it."""

    def __init__(self, raw, dtype_name, max_batch, context, layers=None, layers_key="num_hidden_layers", storage=None,
                 max_tokens=None, step_tokens=PREFILL_TOKENS):
        import torch
        from transformers_neuronx_amd.config import EngineConfig
        from transformers_neuronx_amd.config.registry import resolve
        from transformers_neuronx_amd.engine.engine import LLMEngine
        from transformers_neuronx_amd.engine.factory import runner_from_random
        self.torch = torch
        raw = {k: v for k, v in raw.items() if k != "name"}
        self.layers_full = raw.get(layers_key)
        if layers:
            raw[layers_key] = layers
        self.cfg = resolve(raw).config_class.from_dict(raw)
        self.dtype_name = dtype_name
        self.dtype = torch.bfloat16 if dtype_name == "bf16" else torch.float32
        self.context = context
        self.ecfg = EngineConfig(dtype=self.dtype, page_size=64, max_tokens=max_tokens or max_batch * context,
                                 max_num_seqs=max_batch, max_num_batched_tokens=max(2048, step_tokens),
                                 max_model_len=context, prompts_first=True)
        t0 = time.time()
        self.runner = runner_from_random(self.cfg, seed=0, cfg=self.ecfg, storage=storage)
        torch.cuda.synchronize()
        self.model = self.runner.model
        copies = getattr(self.runner.ops, "copy_bytes", None)
        log(f"model ready in {time.time() - t0:.1f} s ({self.model.weight_bytes / 1e9:.2f} GB of weights"
            + (f", {copies / 1e9:.1f} GB of them a second time in tile order" if copies is not None else "") + ")")
        self.engine = LLMEngine(self.runner, self.ecfg)
        self.gen = torch.Generator().manual_seed(1)
        self.vocab = self.model.spec.vocab_size

    def close(self):
        self.engine = self.runner = self.model = None
        gc.collect()
        self.torch.cuda.empty_cache()

    def prompt(self, n):
        return self.torch.randint(3, self.vocab, (n,), generator=self.gen).tolist()

    def decode(self, batch, steps, warmup, prompt_len=None, latencies=None, do_sample=False):
        """Tokens per second, seconds per step and bytes per step of `steps` decode steps that end at
        the full context (or begin after prompts of `prompt_len` tokens)."""
        from transformers_neuronx_amd.sampling import SamplingParams
        torch, engine = self.torch, self.engine
        engine.reset()
        if prompt_len is None:
            prompt_len = self.context - (steps + warmup) - 1
        for i in range(batch):
            params = SamplingParams(max_new_tokens=steps + warmup + 1, do_sample=do_sample, temperature=0.8,
                                    top_k=50, top_p=0.95, seed=i, ignore_eos=True)
            engine.add_request(self.prompt(prompt_len), params)
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
        # every weight once, and of each live request the cache that its token reads (at the mean length)
        read = self.model.weight_bytes + batch * self.model.cache_bytes_read(lens / steps / batch, self.dtype)
        return made / (sec * steps), sec, read

    def prefill(self, tokens):
        """Seconds of one whole prompt in one step (the median of five, after one warm-up) and its flops."""
        from transformers_neuronx_amd.sampling import SamplingParams
        torch, engine = self.torch, self.engine
        engine.reset()
        params = SamplingParams(max_new_tokens=1, do_sample=False, ignore_eos=True)
        times = []
        for i in range(6):
            engine.add_request(self.prompt(tokens), params)
            torch.cuda.synchronize()
            start = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - start)
        return sorted(times[1:])[2], self.model.step_flops(tokens, (tokens + 1) / 2, 1)

    def kernel_rates(self, batch, tokens):
        """What the kernels of a decode step of `batch` requests at the full context, and of a prompt step of
        `tokens` tokens, reach: {"<step> <entry point> <sizes> us": microseconds a launch, "... GB/s" or
        "... TFLOP/s": the bytes the launch has to move, or its flops, over that time}, for the launches that say
        what they move (products, attention) and take a hundredth of their step or more. The steps run with
        events around every launch, unrecorded, so a launch stands alone; the kernels are the recorded step's."""
        from transformers_neuronx_amd.sampling import SamplingParams
        engine, out = self.engine, {}
        for step, count, length in ((f"decode_b{batch}", batch, self.context - 5), (f"prefill_{tokens}", 1, tokens)):
            engine.reset()
            new = 4 if step.startswith("decode") else 1
            for i in range(count):
                engine.add_request(self.prompt(length), SamplingParams(max_new_tokens=new, do_sample=False, ignore_eos=True))
            if step.startswith("decode"):
                while any(not r.decoding for r in engine.requests.values()):
                    engine.step()
                engine.profile(1)                                    # once unmeasured: what is made at first use
            else:
                engine.profile(1)
                engine.reset()
                engine.add_request(self.prompt(length), SamplingParams(max_new_tokens=1, do_sample=False, ignore_eos=True))
            table, _ = engine.profile(1, work=True)
            whole = sum(row[1] for row in table.values())
            for name, (calls, ms, nbytes, flops) in table.items():
                if nbytes and ms >= 0.01 * whole:
                    key = f"{step} {name.replace('tnx_', '')}"
                    out[key + " us"] = round(1e3 * ms / calls, 1)
                    if step.startswith("decode"):
                        out[key + " GB/s"] = round(nbytes / ms / 1e6)
                    else:
                        out[key + " TFLOP/s"] = round(flops / ms / 1e9, 1)
        engine.reset()
        return out

    def mix(self, requests=64, new_tokens=256):
        """Every request is there at the start; the scheduler mixes portions of prompts with decoding. The
        workload runs twice with other tokens and the second run is timed: the first loads the vendor
        library and lets it choose its algorithms, which a server does once in its life."""
        from transformers_neuronx_amd.sampling import SamplingParams
        torch, engine = self.torch, self.engine
        params = SamplingParams(max_new_tokens=new_tokens, do_sample=False, ignore_eos=True)
        for timed in (False, True):
            engine.reset()
            lengths = torch.randint(16, 1025, (requests,), generator=torch.Generator().manual_seed(2)).tolist()
            for n in lengths:
                engine.add_request(self.prompt(n), params)
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
            assert made == requests * new_tokens, made
        return {"tokens_per_s": round(made / sec, 1), "seconds": round(sec, 3), "steps": steps,
                "prompt_tokens": sum(lengths),
                "mean_time_to_first_token_ms": round(1e3 * sum(first.values()) / len(first), 2),
                "preemptions": engine.scheduler.num_preemptions - preempted}


def room_for(raw, args, context, torch):
    """How many requests of `context` tokens the device holds beside the model's weights, from what the model
    declares (nothing is loaded)."""
    from transformers_neuronx_amd.config.registry import resolve
    from transformers_neuronx_amd.engine.model import DecoderModel
    raw = {k: v for k, v in raw.items() if k != "name"}
    if args.layers:
        raw[args.layers_key] = args.layers
    arch = resolve(raw)
    model = DecoderModel(arch.build_spec(arch.config_class.from_dict(raw)))
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    item = 2 if args.dtype == "bf16" else 4
    weights = sum(item * int(torch.Size(d.shape).numel()) for d in model.param_decls() if d.tied_to is None)
    # (the random weights are drawn apart and fused afterwards: a quarter of them is held twice meanwhile, and
    # what that leaves free again is in pieces too small for the cache's blocks)
    per_request = model.cache_bytes_read(1, dtype) * context
    total = int(0.95 * torch.cuda.mem_get_info()[1]) - (4 << 30)
    # beside the weights and their tile-ordered copies, which decoding at small batches reads; where not even
    # eight requests fit beside both (the largest models), beside the weights alone
    beside_copies = int((total - 2.3 * weights) // per_request)
    return max(1, beside_copies if beside_copies >= 8 else int((total - 1.27 * weights) // per_request))


def flat_config(cfg, extra):
    """The sizes of a run in one flat dictionary of at most 20 keys: the run's own first, then the typed
    configuration's sizes (integers), then its options (strings and truth values) while there is room."""
    out = dict(extra)
    raw = cfg.to_dict()
    skip = ("_token_id", "torch_dtype", "model_type", "init_std", "architectures")
    fields = [(k, v) for k, v in raw.items() if not any(s in k for s in skip) and not isinstance(v, (list, dict))
              and v is not None]
    for wanted in ((int,), (str, bool)):
        for k, v in fields:
            if len(out) < 20 and k not in out and type(v) in wanted and not k.startswith("_"):
                out[k] = v
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=None,
                    help="the context length decoding ends at (default: the model's positions); a longer one than "
                         "the configuration names is written into it, random weights allow any")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--layers-key", default="num_hidden_layers", help="the config.json key that --layers sets")
    ap.add_argument("--positions-key", default="max_position_embeddings", help="the config.json key that --context raises")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip everything but the headline decode measurement")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the measurements at other models' sizes (the OPT-350m mix, OPT-66B) and the full-depth check")
    ap.add_argument("--prefill-only", action="store_true", help="measure the prompt step alone (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="the length of the prompt that is taken in one step (2,048; with --context up to that)")
    ap.add_argument("--model", default="6.7b",
                    help="a name of " + ", ".join(PRESETS) + " (OPT-6.7B is the measurement of record), a model "
                         "folder or a config.json file of any registered architecture; weights are random")
    ap.add_argument("--do-sample", action="store_true",
                    help="decode with temperature 0.8, top-k 50 and top-p 0.95 instead of greedily")
    ap.add_argument("--mix", action="store_true",
                    help="instead: 64 requests with prompts of 16 to 1,024 tokens and 256 new tokens each, all "
                         "queued at once (a continuous-batching workload); prints its own line")
    ap.add_argument("--own-products", action="store_true",
                    help="every matrix product on our own kernels (none goes to the vendor library)")
    ap.add_argument("--tune-all", action="store_true",
                    help="time the vendor library's candidates for the many-rows products too")
    ap.add_argument("--big-batch", type=int, default=None,
                    help="the larger batch of `points` (64; cut to what fits the device at the full context)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    from transformers_neuronx_amd.kernels.hip import HipOps
    if args.own_products:
        HipOps.library_rows = 0
    if args.tune_all:
        HipOps.library_tune = 2
    raw = raw_config(args.model)
    name = raw["name"]
    if args.context and args.context > raw.get(args.positions_key, 0):
        raw[args.positions_key] = args.context
    context = args.context or raw[args.positions_key]
    tokens = args.prefill_tokens
    peak_flops = PEAK_FLOPS[args.dtype]

    # the larger batch of `points` is cut to what the device holds beside the weights at the full context
    only = args.no_points or args.prefill_only or args.mix
    big = args.big_batch or 64
    if not only:
        fits = room_for(raw, args, context, torch)
        if big > fits:
            log(f"{big} requests of {context} tokens do not fit beside the weights; the larger batch is {fits}")
            big = fits
        if args.batch > fits:
            print(f"bench.py: {args.batch} requests of {context} tokens do not fit on this device ({fits} do)")
            return 2
    max_batch = args.batch if only else max(args.batch, big)
    if args.mix:
        max_batch = 64
    if tokens > context:
        print(f"bench.py: a prompt of {tokens} tokens is longer than the context of {context}")
        return 2
    bench = Bench(raw, args.dtype, max_batch, context, args.layers, args.layers_key, step_tokens=tokens)
    cfg = bench.cfg

    if args.mix:
        got = bench.mix()
        print(json.dumps(dict({"metric": f"{name} continuous batching: 64 requests, prompts 16-1,024, 256 new tokens each",
                               "value": got.pop("tokens_per_s"), "unit": "generated tokens/s"}, **got,
                              dtype=args.dtype, warmup="the same workload once, untimed")))
        return 0
    if args.prefill_only:
        sec_p, flops = bench.prefill(tokens)
        print(json.dumps({"prefill_ms": round(sec_p * 1e3, 3), "tokens": tokens,
                          "frac": round(flops / sec_p / peak_flops, 4)}))
        return 0

    keep_busy(bench.runner.ops, torch, 3.0)
    ceilings = measured_ceilings(bench.runner.ops, torch) if not args.no_points else None
    if ceilings:
        log(f"this device at best: {ceilings}")
    points = {}
    if not args.no_points:
        # the whole way from 512-token prompts to the full context, as the reference's benchmark generates whole
        # sequences (generation_demo.py:159-187) and reports the percentiles of their latency
        lat = []
        first = min(512, context // 4)
        k = context - first - 1 - 4
        v, s, rd = bench.decode(args.batch, k, 4, prompt_len=first, latencies=lat, do_sample=args.do_sample)
        lat.sort()
        tag = f"decode_{first}_to_{context}"
        points[tag] = round(v, 2)
        points[tag + "_ms"] = round(s * 1e3, 4)
        points[tag + "_hbm_frac"] = round(rd / s / 1e9 / PEAK_HBM_GBS, 4)
        for q in (0, 50, 90, 95, 99, 100):
            points[f"step_latency_p{q}_ms"] = round(lat[min(len(lat) - 1, int(len(lat) * q / 100))] * 1e3, 4)
        log(f"decode batch {args.batch}, {first} -> {context:,}: {v:.1f} tok/s, {s * 1e3:.2f} ms/step")
    value, sec, read = bench.decode(args.batch, args.steps, args.warmup, do_sample=args.do_sample)
    log(f"decode batch {args.batch}: {value:.1f} tok/s, {sec * 1e3:.2f} ms/step")
    achieved = read / sec / 1e9
    out = {
        "metric": f"{name} decode tok/s @ batch 1/8/{big}; prefill tok/s @ {tokens:,} tokens",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random weights and token ids)"
                                      + (", sampled (temperature 0.8, top-k 50, top-p 0.95)" if args.do_sample else ""),
        "config": flat_config(cfg, {"model": name, "global_batch": args.batch, "seq_len": context, "parallelism": "none",
                                    "layers_of_model": bench.layers_full, "page_size": bench.ecfg.page_size,
                                    "prompt_len": context - args.steps - args.warmup - 1, "prefill_tokens": tokens}),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if ceilings:
        out["ceilings"] = ceilings
        out["roofline"]["peak_measured"] = ceilings["hbm_read_gbs_measured"]
        out["roofline"]["frac_of_measured"] = round(achieved / ceilings["hbm_read_gbs_measured"], 4)
    if not args.no_points:
        sec_p, flops = bench.prefill(tokens)
        out["prefill"] = {"value": round(tokens / sec_p, 1), "tokens": tokens, "ms": round(sec_p * 1e3, 3),
                          "frac": round(flops / sec_p / peak_flops, 4)}
        if args.dtype == "bf16":
            out["prefill"]["peak_measured_tflops"] = ceilings["mfma_tflops_measured"]
            out["prefill"]["frac_of_measured"] = round(flops / sec_p / 1e12 / ceilings["mfma_tflops_measured"], 4)
        log(f"prefill: {out['prefill']}")
        for b, k, w in ((1, min(args.steps, 64), args.warmup), (big, min(args.steps, 32), min(args.warmup, 4))):
            v, s, rd = bench.decode(b, k, w, do_sample=args.do_sample)
            points[f"decode_b{b}"] = round(v, 2)
            points[f"decode_b{b}_ms"] = round(s * 1e3, 4)
            points[f"decode_b{b}_hbm_frac"] = round(rd / s / 1e9 / PEAK_HBM_GBS, 4)
            log(f"decode batch {b}: {v:.1f} tok/s, {s * 1e3:.2f} ms/step")
        out["points"] = points
        if args.dtype == "bf16":
            try:
                out["kernels"] = bench.kernel_rates(args.batch, tokens)
                log(f"kernels: {out['kernels']}")
            except Exception as e:                                   # noqa: BLE001 (never at the cost of the line)
                out["kernels"] = {"error": f"{type(e).__name__}: {e}"[:200]}
        if not args.no_extras and args.dtype == "bf16":
            extras(out, bench, raw, args, context)
    print(json.dumps(out))
    return 0


def extras(out, bench, raw, args, context):
    """What the line carries beyond its own model: the full-depth check against a float32 engine, and the other
    workloads the family is measured on. None of them may cost the line: what fails is named and left out."""
    import torch
    from transformers_neuronx_amd.testing import compare_precisions
    points = out["points"]
    try:
        # the float32 engine on the very weights of the bfloat16 one (drawn in bfloat16 from the same seed)
        wide = Bench(raw, "fp32", 1, context, args.layers, args.layers_key, storage=torch.bfloat16, max_tokens=384)
        report = compare_precisions(wide.engine, bench.engine, bench.prompt(300), 21)
        wide.close()
        out["check"] = {k: (round(v, 6) if isinstance(v, float) else v) for k, v in report.items()}
        out["check"]["what"] = ("bfloat16 engine against the float32 engine on the same weights, all layers: a 300-token "
                                "prompt and 20 decode steps; allclose is atol 1.0, rtol 1e-3")
        log(f"check: {out['check']}")
    except Exception as e:                                   # noqa: BLE001
        out["check"] = {"error": f"{type(e).__name__}: {e}"[:200]}
    bench.close()
    try:
        small = Bench(raw_config("350m"), "bf16", 64, 2048)
        got = small.mix()
        small.close()
        for k, v in got.items():
            points[f"mix_350m_{k}"] = v
        log(f"OPT-350m mix: {got}")
    except Exception as e:                                   # noqa: BLE001
        points["mix_350m_error"] = f"{type(e).__name__}: {e}"[:200]
    try:
        free = torch.cuda.mem_get_info()[0]
        if free < 262e9:
            points["opt66b_skipped"] = f"{free / 1e9:.0f} GB free"
            return
        # Twice: with the cache of 8 requests most matrices get their tile-ordered copy beside the 131 GB of
        # weights; then with the largest batch that fits at the full context (the family's is 32), where
        # hardly any does.
        def decode_points(large, batches):
            for b, k, w in batches:
                v, s, rd = large.decode(b, k, w)
                points[f"opt66b_decode_b{b}"] = round(v, 2)
                points[f"opt66b_decode_b{b}_ms"] = round(s * 1e3, 3)
                points[f"opt66b_decode_b{b}_hbm_frac"] = round(rd / s / 1e9 / PEAK_HBM_GBS, 4)
                log(f"OPT-66B decode batch {b}: {v:.1f} tok/s, {s * 1e3:.2f} ms/step")

        large = Bench(raw_config("66b"), "bf16", 8, 2048)
        decode_points(large, ((8, 16, 4), (1, 16, 4)))
        large.close()
        most = min(32, room_for(raw_config("66b"), argparse.Namespace(layers=None, layers_key="", dtype="bf16"), 2048, torch))
        large = Bench(raw_config("66b"), "bf16", most, 2048)
        decode_points(large, ((most, 12, 3),))
        sec_p, flops = large.prefill(PREFILL_TOKENS)
        points["opt66b_prefill_ms"] = round(sec_p * 1e3, 2)
        points["opt66b_prefill_frac"] = round(flops / sec_p / PEAK_FLOPS["bf16"], 4)
        log(f"OPT-66B prefill: {sec_p * 1e3:.1f} ms")
        large.close()
    except Exception as e:                                   # noqa: BLE001
        points["opt66b_error"] = f"{type(e).__name__}: {e}"[:200]


if __name__ == "__main__":
    sys.exit(main())
