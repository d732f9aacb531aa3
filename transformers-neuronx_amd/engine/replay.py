"""Trace replay: given token ids go through the model step by step and the
logits at the wanted places are written out. Nothing is sampled. It drives the
model, step function, cache and kernels that generation uses.

Reference precedents: per-step logits dumps and their offline comparison
(generation_demo.py:694-702, :404-443); the loop that feeds a prompt's tail
token by token through the decode path (base.py:284-299).

Input: one JSON object a line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
`entries` are one batch; `end` lists the requests that are over after the step.
Output: `<out>/<step>.f32`, the wanted logits as little-endian float32
`[wanted, vocab]` in the order of the entries and of `want`; then a line
`done <step>` on standard output.
"""
import json
import os
import sys
from typing import Iterable, Optional, TextIO

import numpy as np
import torch

from ..config.engine_config import EngineConfig
from .batch import StepEntry
from .factory import runner_from_folder


def make_replay_runner(model_dir: str, dtype: str, max_tokens: int, page_size: int = 64, device: str = "cuda:0",
                       kernels: str = "hip", max_requests: int = 16):
    """The runner a replay uses: a page pool for `max_tokens` tokens (each
    request's count rounded up to whole pages by the caller)."""
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_num_seqs=max_requests,
                       device=device, kernels=kernels)
    return runner_from_folder(model_dir, cfg)


def replay(lines: Iterable[str], runner, out_dir: str, out: Optional[TextIO] = None) -> int:
    """Run the steps; returns how many ran."""
    os.makedirs(out_dir, exist_ok=True)
    out = out or sys.stdout
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], list(e["tokens"]), list(e.get("want", []))) for e in rec.get("entries", [])]
        logits = runner.step(entries) if entries else None
        if logits is not None:
            arr = logits.detach().to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(out_dir, f"{step}.f32"))
        else:
            runner.ops.synchronize()
        for req in rec.get("end", []):
            runner.finish(req)
        print(f"done {step}", file=out, flush=True)
        n += 1
    return n


def main(argv=None) -> int:
    """`trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N < steps.jsonl`"""
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="the most tokens live requests hold at a time (each request's count in whole pages)")
    ap.add_argument("--page-size", type=int, default=64, help="tokens per cache page (divides 64 or is a multiple)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if not os.environ.get("HOME") or not os.access(os.environ.get("HOME", "/"), os.W_OK):
        # libraries that want a writable home get a private temporary one
        import tempfile
        os.environ["HOME"] = tempfile.mkdtemp(prefix="trace_run_home_")
    print("[trace_run] loading the model ...", file=sys.stderr, flush=True)
    runner = make_replay_runner(args.model, args.dtype, args.max_tokens, args.page_size, args.device)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay(sys.stdin, runner, args.out)
    return 0
