"""Command line in the manner of the reference's `opt_demo` and `generation_demo`.

    opt_demo [--amp f32|bf16] save DIR --random --config CONFIG.json [--seed N]
    opt_demo [--amp f32|bf16] run DIR [--batch_size 4] [--n_positions 128] [--print_latency]
             [--prompt_len N | --prompt_ids 5,6,7] [--top_k 50] [--top_p 1.0] [--temperature 1.0]
             [--do_sample] [--max_new_tokens N] [--seed N] [--benchmark] [--profile] [--snapshot]
             [--dump_logits DIR [--dump_logits_limit N]]
    opt_demo analyze -d DIR [DIR ...] GOLDEN_DIR

Option names and meanings are the reference's where it has them: gpt_demo.py:37-66
(`--amp`, `save`, `--random`, `--config`, `run`, `--batch_size`, `--n_positions`,
`--print_latency`) and generation_demo.py:201-280 (`--prompt_len`: random token ids of
that length, :267, :492-494; `--top_k`, `--top_p`, `--temperature`, `--do_sample`,
`--max_new_tokens`, `--dump_logits`, `--dump_logits_limit`, `--benchmark`; `analyze -d`, :286-290). Without `--do_sample` `run` does what
the reference's `run` does: `model.sample(input_ids, sequence_length=n_positions)` with
top_k 50. There is no tokenizer here (no network to fetch one): prompts are token ids.
"""
import argparse
import json
import math
import os
import sys
import time

import torch


def _parser():
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--amp", default="f32", choices=["f32", "f16", "bf16"])
    sub = parser.add_subparsers(dest="which", required=True)
    save = sub.add_parser("save")
    save.add_argument("save", help="Directory to save the model")
    save.add_argument("--random", action="store_true",
                      help="Random weights flag. If true, config.json would be used to generate a model with "
                           "random weight")
    save.add_argument("--config", type=str, default="", help="Path to config.json file")
    save.add_argument("--seed", type=int, default=0)
    ana = sub.add_parser("analyze")
    ana.add_argument("-d", "--dirs", nargs="+", required=True, help="folders of dumped logits; the last is the golden one")
    run = sub.add_parser("run")
    run.add_argument("load")
    run.add_argument("--batch_size", type=int, default=4, help="Input batch size")
    run.add_argument("--n_positions", type=int, default=128, help="Input sequence length")
    run.add_argument("--tp_degree", type=int, default=1, help="must be 1: one GPU")
    run.add_argument("--print_latency", action="store_true", help="Print latency of each step")
    # gpt_demo.py:53, :55, :66 and generation_demo.py:245-262: taken where they mean something on one GPU
    run.add_argument("--unroll", type=int, default=None, help="accepted; nothing is unrolled here")
    run.add_argument("--context_length_estimate", type=int, default=None, help="accepted; prompts are not bucketed here")
    run.add_argument("--quantize", action="store_true", help="refused: weights stay in the dtype of --amp")
    run.add_argument("--continuous_batching", action="store_true",
                     help="accepted: requests are batched continuously whether it is given or not")
    run.add_argument("--various", action="store_true",
                     help="Generated batched sequence with different length if set; otherwise using same length")
    run.add_argument("--simple_sample_eos_token_override", type=int, default=None,
                     help="override eos token, set to -1 to always generate exactly as many tokens as asked for")
    run.add_argument("--prompt_len", type=int, default=None, help="random token ids of this length as the prompt")
    run.add_argument("--prompt_ids", type=str, default=None, help="comma-separated token ids of the prompt")
    run.add_argument("--do_sample", action="store_true")
    run.add_argument("--top_k", type=int, default=50)
    run.add_argument("--top_p", type=float, default=1.0)
    run.add_argument("--temperature", type=float, default=1.0)
    run.add_argument("--no_repeat_ngram_size", type=int, default=0)
    run.add_argument("--max_new_tokens", type=int, default=None)
    run.add_argument("--max_length", type=int, default=None)
    run.add_argument("--seed", type=int, default=15213)
    run.add_argument("--dump_logits", type=str, default=None,
                     help="folder for the logits that each generated token was chosen from: <step>.pt, [batch, vocab]")
    run.add_argument("--dump_logits_limit", type=int, default=1, help="how many steps to dump; -1 for all")
    run.add_argument("--benchmark", action="store_true",
                     help="2 warm-up generations, then 5 timed ones: latency percentiles of a whole sequence, "
                          "context encoding and output token latency, throughput")
    run.add_argument("--profile", action="store_true",
                     help="time every kernel of one prompt step and one decode step and print the table")
    run.add_argument("--snapshot", action="store_true",
                     help="write what every step reads and gives to tnx_snapshot_<amp>_b<batch_size>/iter<n> "
                          "(TNX_SNAPSHOT_STEPS='[3, 7]' keeps those steps only); "
                          "`python -m transformers_neuronx_amd.engine.snapshot` runs one of them again")
    run.add_argument("--page_size", type=int, default=64)
    return parser


def save(args):
    from .gen_random_pretrained import gen_random_pretrained
    if not args.random:
        raise SystemExit("save: only --random --config FILE is possible here (there is no network to fetch a model)")
    if not args.config or not os.path.exists(args.config):
        raise SystemExit("Please provide the config.json like: --config=./config.json")
    dtype = {"f32": "float32", "f16": "float16", "bf16": "bfloat16"}[args.amp]
    gen_random_pretrained(args.config, args.save, args.seed, dtype)
    print(f"saved {args.save}")


def run(args):
    from ..config.engine_config import GenerationConfig
    from .model import OPTForSampling
    if args.quantize:
        raise SystemExit("run: --quantize is not to be had here: weights stay in the dtype of --amp")
    torch.manual_seed(args.seed)
    if args.snapshot:
        # generation_demo.py:551-554 names the folder in the environment, where the runtime looks for it
        os.environ["TNX_SNAPSHOT_PATH"] = f"tnx_snapshot_{args.amp}_b{args.batch_size}"
        print(f"Set snapshot path {os.environ['TNX_SNAPSHOT_PATH']}")
    print("running OPTForSampling.from_pretrained")
    model = OPTForSampling.from_pretrained(args.load, batch_size=args.batch_size, amp=args.amp,
                                           tp_degree=args.tp_degree, n_positions=args.n_positions,
                                           unroll=args.unroll, context_length_estimate=args.context_length_estimate,
                                           page_size=args.page_size)
    print("running model.load")
    model.load()
    vocab = model.config.vocab_size
    if args.prompt_ids:
        row = [int(t) for t in args.prompt_ids.split(",")]
        input_ids = torch.tensor([row] * args.batch_size)
    else:
        n = args.prompt_len or 8
        input_ids = torch.randint(3, vocab, (args.batch_size, n))
    start_ids = None
    if args.various and args.batch_size > 1:
        # rows of different lengths, padded on the left up to `start_ids` (generation_demo.py:262; the padding
        # is the pad token and is dropped before the rows reach the engine)
        width = input_ids.shape[1]
        start_ids = torch.tensor([(b * max(1, width // args.batch_size)) % width for b in range(args.batch_size)])
        for b in range(args.batch_size):
            input_ids[b, :int(start_ids[b])] = getattr(model.config, "pad_token_id", 1)
    total = args.n_positions
    if args.max_new_tokens is not None:
        total = min(total, input_ids.shape[1] + args.max_new_tokens)
    if args.max_length is not None:
        total = min(total, args.max_length)
    gen = None
    if args.do_sample:
        gen = GenerationConfig(do_sample=True, top_k=args.top_k, top_p=args.top_p, temperature=args.temperature)
    if args.simple_sample_eos_token_override is not None:
        # the generation stops at this token (generation_demo.py:245); -1 is no token's id: it never stops early
        eos = args.simple_sample_eos_token_override
        gen = gen or GenerationConfig(do_sample=False, top_k=1)
        gen.eos_token_id = eos if eos >= 0 else None
    dumped = []
    if args.dump_logits:
        # generation_demo.py:694-702 writes the scores of the first `dump_logits_limit` generated tokens
        os.makedirs(args.dump_logits, exist_ok=True)

        def keep(requests, logits):
            if args.dump_logits_limit < 0 or len(dumped) < args.dump_logits_limit:
                order = sorted(range(len(requests)), key=lambda i: requests[i].req_id)
                dumped.append(logits[order].cpu())
        model.engine.logits_hook = keep
    if args.print_latency:
        model.engine.record_timings = True
    print("running model.sample")

    def generate():
        return model.sample(input_ids, sequence_length=total, start_ids=start_ids, top_k=args.top_k,
                            temperature=args.temperature, top_p=args.top_p, seed=args.seed, generation_config=gen,
                            no_repeat_ngram_size=args.no_repeat_ngram_size)
    out = generate()
    print("generated_sequence=", out)
    for i, logits in enumerate(dumped):
        torch.save(logits, os.path.join(args.dump_logits, f"{i}.pt"))
    if args.dump_logits:
        print(f"Dumped the logits of {len(dumped)} steps into {args.dump_logits}")
    if args.print_latency:
        for rec in model.engine.timings:
            print(f"Latency: {math.ceil(rec['seconds'] * 1000)} ms ({rec['tokens']} tokens)")
    if args.benchmark:
        model.engine.logits_hook = None
        print(json.dumps(benchmark(model, generate, args.batch_size, input_ids.shape[1], total)))
    if args.profile:
        from ..sampling.params import SamplingParams
        engine = model.engine
        engine.reset()
        for row in input_ids.tolist():
            engine.add_request(row, SamplingParams(max_new_tokens=3, do_sample=False, ignore_eos=True))
        for title in ("prompt step", "decode step"):
            table, _ = engine.profile(1, work=True)
            print(f"{title}: {sum(row[1] for row in table.values()):.3f} ms in kernels")
            for name, (calls, ms, nbytes, flops) in table.items():
                rates = f"  {nbytes / ms / 1e6:8.0f} GB/s {flops / ms / 1e9:8.1f} TFLOP/s" if nbytes and ms > 0 else ""
                print(f"  {name:48s} {calls:5d} launches {ms:9.3f} ms{rates}")
        engine.reset()


def percentile(values, percent):
    """The reference's percentile of a list (generation_demo.py:96-105): the element at `len * percent / 100`,
    rounded down unless its fraction is above one half, and never beyond the last."""
    ordered = sorted(values)
    pos = len(ordered) * percent / 100
    last = len(ordered) - 1
    low, high = min(math.floor(pos), last), min(math.ceil(pos), last)
    return ordered[high] if pos - low > 0.5 else ordered[low]


def benchmark(model, generate, batch_size, context_length, output_length, warmup=2, iterations=5):
    """The reference's benchmark report (generation_demo.py:107-187): `warmup` whole generations, then
    `iterations` timed ones; latency percentiles of a whole sequence, mean latency of the context encoding
    (the steps that take prompts in) and of an output token, and throughput."""
    engine = model.engine
    print(f"Warmup ({warmup} iterations) ...")
    for _ in range(warmup):
        generate()
    print(f"Benchmark loop ({iterations} iterations) ...")
    latencies, context = [], []
    engine.record_timings = True
    begin = time.time()
    for _ in range(iterations):
        engine.timings.clear()
        start = time.time()
        generate()
        latencies.append((time.time() - start) * 1000)
        context.append(1000 * sum(r["seconds"] for r in engine.timings if r["prefill_tokens"]))
    duration = time.time() - begin
    engine.record_timings = False
    new = output_length - context_length
    return {
        "sequence_length": output_length, "context_length": context_length, "output_length": output_length,
        "batch_size": batch_size, "iterations": iterations, "batches": len(latencies),
        "inferences": len(latencies) * batch_size, "total_duration_seconds": duration,
        "mean_context_encoding_latency": sum(context) / len(context),
        "e2e_output_token_throughput": len(latencies) * batch_size * new / duration,
        "mean_output_token_latency": (sum(latencies) - sum(context)) / len(latencies) / max(1, new),
        "sequence_latency_percentiles": {f"sequence_latency_p{q}": percentile(latencies, q)
                                         for q in (0, 50, 90, 95, 99, 100)},
    }


def analyze(args):
    """Logits dumped by two or more runs against the last one, the golden one, step by step: the
    reference's yardstick (generation_demo.py:404-443), `allclose(atol=1.0, rtol=1e-3)` and the same
    greedy token. Returns the number of steps that fail either."""
    def load(folder):
        names = sorted((f for f in os.listdir(folder) if f.endswith(".pt")), key=lambda f: int(f[:-3]))
        return [torch.load(os.path.join(folder, f), weights_only=True) for f in names]
    golden_dir, golden = args.dirs[-1], load(args.dirs[-1])
    failures = 0
    for folder in args.dirs[:-1]:
        cand = load(folder)
        print(f"{folder} vs {golden_dir} (golden): {len(cand)} vs {len(golden)} steps")
        for i, (a, b) in enumerate(zip(cand, golden)):
            close = torch.allclose(a, b, atol=1.0, rtol=0.001)
            same = torch.equal(a.argmax(-1), b.argmax(-1))
            if not close:
                print(f"  step {i}: logits differ by up to {float((a - b).abs().max()):.4f}")
            if not same:
                print(f"  step {i}: greedy tokens differ: {a.argmax(-1).tolist()} vs {b.argmax(-1).tolist()}")
            failures += (not close) or (not same)
            if not same:
                break                      # later steps follow different tokens
    print("all steps match" if not failures else f"{failures} steps do not match")
    return failures


def main(argv=None):
    args = _parser().parse_args(argv)
    if args.which == "save":
        save(args)
    elif args.which == "analyze":
        return 1 if analyze(args) else 0
    else:
        run(args)


if __name__ == "__main__":
    sys.exit(main())
