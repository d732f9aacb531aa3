"""Snapshots of steps: what a step read and what it gave, written to a folder, so that the one step can be
run again alone, on another day or another build, and compared.

Reference: compiler.py:539-570 (`snapshot_enter`, `snapshot_exit`: a kernel's input and output tensors under
`<HLO_SNAPSHOT_PATH>/iter<n>/inputs` and `outputs`, for the iterations listed in `HLO_SNAPSHOT_STEPS` or for
all) and generation_demo.py:269 (`--snapshot`). There the unit is a compiled kernel; here it is a step of the
runner, whose inputs are the step's integers and the cache pages and state slots of its requests.

A snapshot `<folder>/iter<n>/` holds
    step.json            the entries (request, tokens, wanted places, tokens cached before the step, slot), the
                         page size, every group's block table for these requests, the dtype
    inputs.safetensors   `pages.<cache id>.<name>`: the pages these requests hold, as they were before the step,
                         in the order of `step.json`'s `pages` list of the cache's group;
                         `state.<cache id>.<name>`: the rows of the requests' slots; `kept_tokens` where a step
                         names a token by its slot
    outputs.safetensors  `logits` (if any were wanted) and every tensor the model taps, `tap.<name>`

`replay_snapshot(folder, runner)` gives the saved requests pages and slots of the runner's own cache, puts the
saved contents there, runs the step and returns how far its logits and taps lie from the saved ones.
"""
import json
import os
from typing import Dict, Iterable, List, Optional

import numpy as np
import torch
from safetensors.torch import load_file, save_file

from .. import debug
from .batch import StepEntry


def snapshots_from_environment() -> Optional["StepSnapshots"]:
    """`TNX_SNAPSHOT_PATH` (or the reference's `HLO_SNAPSHOT_PATH`) names the folder, `TNX_SNAPSHOT_STEPS`
    (`HLO_SNAPSHOT_STEPS`) a JSON list of the steps to keep; without it every step is kept."""
    folder = os.environ.get("TNX_SNAPSHOT_PATH") or os.environ.get("HLO_SNAPSHOT_PATH")
    if not folder:
        return None
    steps = os.environ.get("TNX_SNAPSHOT_STEPS") or os.environ.get("HLO_SNAPSHOT_STEPS")
    return StepSnapshots(folder, json.loads(steps) if steps else None)


class StepSnapshots:
    """Counts the steps of a runner and writes those asked for."""

    def __init__(self, folder: str, steps: Optional[Iterable[int]] = None):
        self.folder = folder
        self.steps = None if steps is None else set(int(s) for s in steps)
        self.iteration = 0

    def wanted(self) -> bool:
        return self.steps is None or self.iteration in self.steps

    def path(self) -> str:
        path = os.path.join(self.folder, f"iter{self.iteration}")
        os.makedirs(path, exist_ok=True)
        return path

    def enter(self, runner, entries: List[StepEntry]) -> None:
        """Before the step runs (its pages are there already): the integers and what the cache holds."""
        cache = runner.cache
        reqs = [e.req for e in entries]
        groups = {}
        for name, g in cache.groups.items():
            table = cache.block_table(reqs, name)
            groups[name] = {"window": g.window, "table": table.tolist(),
                            "pages": sorted(set(int(p) for p in table.reshape(-1) if p >= 0))}
        record = {
            "iteration": self.iteration,
            "dtype": str(cache.dtype).replace("torch.", ""),
            "page_size": cache.page_size,
            "entries": [{"id": repr(e.req), "tokens": [int(t) for t in e.tokens], "want": [int(w) for w in e.want],
                         "cached": cache.num_tokens(e.req), "slot": cache.slot_of(e.req)} for e in entries],
            "groups": groups,
        }
        tensors: Dict[str, torch.Tensor] = {}
        slots = torch.tensor([cache.slot_of(r) for r in reqs], dtype=torch.long, device=runner.model.device)
        for cid, lc in cache.caches.items():
            if not lc.writes:
                continue
            if lc.group is not None:
                held = torch.tensor(groups[lc.group]["pages"], dtype=torch.long, device=runner.model.device)
                for name, pages in lc.pages.items():
                    tensors[f"pages.{cid}.{name}"] = pages[held].contiguous().cpu()
            for name, state in lc.state.items():
                tensors[f"state.{cid}.{name}"] = state[slots].contiguous().cpu()
        if any(t < 0 for e in entries for t in e.tokens):
            tensors["kept_tokens"] = runner.kept_tokens.cpu()
        path = self.path()
        with open(os.path.join(path, "step.json"), "w") as f:
            json.dump(record, f)
        save_file(tensors, os.path.join(path, "inputs.safetensors"))

    def exit(self, logits: Optional[torch.Tensor], taps: Dict[str, torch.Tensor]) -> None:
        tensors = {f"tap.{name}": t.contiguous().cpu() for name, t in taps.items()}
        if logits is not None:
            tensors["logits"] = logits.detach().contiguous().cpu()
        save_file(tensors, os.path.join(self.path(), "outputs.safetensors"))


def replay_snapshot(folder: str, runner) -> Dict[str, float]:
    """Run the step of `folder` (an `iter<n>` folder) on `runner`, a runner of the same model with room for the
    step's requests and none of their names live. Returns {name: largest absolute difference} for `logits` and
    every tap, against what the snapshot holds."""
    with open(os.path.join(folder, "step.json")) as f:
        record = json.load(f)
    inputs = load_file(os.path.join(folder, "inputs.safetensors"))
    saved = load_file(os.path.join(folder, "outputs.safetensors"))
    cache, dev = runner.cache, runner.model.device
    if record["page_size"] != cache.page_size:
        raise ValueError(f"the snapshot's pages hold {record['page_size']} tokens, the runner's {cache.page_size}")
    if set(record["groups"]) != set(cache.groups):
        raise ValueError(f"the snapshot has the page groups {sorted(record['groups'])}, the runner "
                         f"{sorted(cache.groups)}: not the same model")
    names = [("snapshot", i) for i in range(len(record["entries"]))]
    entries = []
    try:
        for name, e in zip(names, record["entries"]):
            cache.add_request(name)
            # pages as the request held them: those of all its positions first, then the step's own
            cache.grow(name, e["cached"] + len(e["tokens"]))
            cache.advance(name, e["cached"])        # (a window lets go of the pages the saved request had let go of)
            entries.append(StepEntry(name, e["tokens"], e["want"]))
        for gname, g in record["groups"].items():
            mine = cache.block_table(names, gname)
            theirs = np.asarray(g["table"], dtype=np.int64).reshape(len(names), -1)
            where = {int(p): i for i, p in enumerate(g["pages"])}
            src, dst = [], []
            for row_mine, row_theirs in zip(mine, theirs):
                for b, p in enumerate(row_theirs):
                    if p >= 0:
                        if b >= len(row_mine) or row_mine[b] < 0:
                            raise ValueError(f"group {gname}: the runner holds no page where the snapshot has one")
                        src.append(where[int(p)])
                        dst.append(int(row_mine[b]))
            if not src:
                continue
            src_t, dst_t = torch.tensor(src, dtype=torch.long), torch.tensor(dst, dtype=torch.long, device=dev)
            for cid in cache.groups[gname].cache_ids:
                for pname, pages in cache.caches[cid].pages.items():
                    pages[dst_t] = inputs[f"pages.{cid}.{pname}"][src_t].to(device=dev, dtype=pages.dtype)
        slots = torch.tensor([cache.slot_of(n) for n in names], dtype=torch.long, device=dev)
        for cid, lc in cache.caches.items():
            if lc.writes:
                for sname, state in lc.state.items():
                    state[slots] = inputs[f"state.{cid}.{sname}"].to(device=dev, dtype=state.dtype)
        kept = "kept_tokens" in inputs
        if kept:
            # a token named by its slot: the saved slot's token goes where this runner's slot is
            old = inputs["kept_tokens"]
            for name, e in zip(names, record["entries"]):
                runner.kept_tokens[cache.slot_of(name)] = int(old[e["slot"]])
            for entry, name in zip(entries, names):
                entry.tokens = [t if t >= 0 else -1 - cache.slot_of(name) for t in entry.tokens]
        with debug.debug_context() as taps:
            logits = runner.step(entries, kept_allowed=kept)
            got = {f"tap.{k}": v for k, v in taps.items()}
        if logits is not None:
            got["logits"] = logits
        if set(got) != set(saved):
            raise ValueError(f"the step gives {sorted(set(got) ^ set(saved))} where the snapshot does not, or the "
                             f"other way round: not the same model")
        return {k: float((got[k].float().cpu() - saved[k].float()).abs().max()) if saved[k].numel() else 0.0
                for k in sorted(saved)}
    finally:
        for name in names:
            if cache.has(name):
                runner.finish(name)


def main(argv=None) -> int:
    """`python -m transformers_neuronx_amd.engine.snapshot --model DIR --snapshot DIR/iterN [--dtype ...]`"""
    import argparse
    from ..config.engine_config import EngineConfig
    from .factory import runner_from_folder
    ap = argparse.ArgumentParser(description="Run a saved step again and print how far it lies from what was saved.")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--snapshot", required=True, help="an iter<n> folder of a snapshot")
    ap.add_argument("--dtype", default=None, help="bfloat16 or float32 (default: the snapshot's)")
    ap.add_argument("--kernels", default="hip", choices=["hip", "reference"])
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    with open(os.path.join(args.snapshot, "step.json")) as f:
        record = json.load(f)
    tokens = sum(-(-(e["cached"] + len(e["tokens"])) // record["page_size"]) * record["page_size"]
                 for e in record["entries"])
    cfg = EngineConfig(dtype=args.dtype or record["dtype"], page_size=record["page_size"], max_tokens=tokens,
                       max_num_seqs=max(1, len(record["entries"])), device=args.device, kernels=args.kernels)
    runner = runner_from_folder(args.model, cfg)
    for name, diff in replay_snapshot(args.snapshot, runner).items():
        print(f"{name}: {diff:.3e}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
