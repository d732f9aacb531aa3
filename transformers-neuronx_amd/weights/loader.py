"""Weights from safetensors, by tensor name.

The checkpoint is opened lazily (one tensor at a time goes to the device; the
host never holds a second copy of the model). Every declared tensor is checked
before anything is computed: one `WeightsError` lists the missing names, the
unexpected names and the wrong shapes together.

Reference: module.py:434-460 (format priority; here `model.safetensors` and its
sharded index only), :75-80 (lazy `safe_open(...).get_tensor(key)`), :142-159
(ties), :161-176 with opt/model.py:207-208 (retry with the base model's names,
that is without the leading `model.`). The reference leaves a tensor that is in
no file uninitialised without a word (:129-140, :66-67); here that is an error.
"""
import json
import os
from typing import Dict, Iterable, List, Optional

import torch
from safetensors import safe_open

from ..parts.spec import ParamDecl

_ST_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}


class WeightsError(ValueError):
    """The checkpoint does not hold what the model declares."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=(), tied_differ=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        self.tied_differ = list(tied_differ)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, expected {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is {got}, expected a floating type")
        for name, other in self.tied_differ:
            lines.append(f"  tied tensors differ: {name} is in the checkpoint and is not equal to {other}, "
                         f"which the configuration ties it to")
        super().__init__("\n".join(lines))


class Checkpoint:
    """Names, shapes and dtypes of a folder's safetensors files; tensors on demand."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self._file_of: Dict[str, str] = {}
        if os.path.exists(single):
            files = [single]
        elif os.path.exists(index):
            with open(index) as fp:
                weight_map = json.load(fp)["weight_map"]
            files = sorted({os.path.join(folder, f) for f in weight_map.values()})
        else:
            raise FileNotFoundError(
                f"no model.safetensors or model.safetensors.index.json in {folder}")
        self._meta: Dict[str, tuple] = {}
        self._handles = {}
        for path in files:
            handle = safe_open(path, framework="pt", device="cpu")
            self._handles[path] = handle
            for key in handle.keys():
                sl = handle.get_slice(key)
                self._file_of[key] = path
                self._meta[key] = (tuple(sl.get_shape()), _ST_DTYPES.get(sl.get_dtype(), sl.get_dtype()))

    def names(self) -> List[str]:
        return list(self._meta)

    def shape(self, name):
        return self._meta[name][0]

    def dtype(self, name):
        return self._meta[name][1]

    def __contains__(self, name):
        return name in self._meta

    def tensor(self, name) -> torch.Tensor:
        return self._handles[self._file_of[name]].get_tensor(name)


class TensorDict:
    """The same interface over tensors held in memory (random weights without a folder)."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._t = dict(tensors)         # a map of its own: `release` empties this one, not the caller's

    def names(self):
        return list(self._t)

    def shape(self, name):
        return tuple(self._t[name].shape)

    def dtype(self, name):
        return self._t[name].dtype

    def __contains__(self, name):
        return name in self._t

    def tensor(self, name):
        return self._t[name]

    def release(self):
        """The model is loaded: tensors it made its own forms of (the fused QKV matrix) are not held any longer."""
        self._t.clear()


def _base_model_name(name: str, base_prefix: str) -> Optional[str]:
    """A checkpoint of the base model alone (without the head's wrapper) names its tensors without the
    wrapper's prefix; the architecture's spec says what that prefix is."""
    return name[len(base_prefix):] if base_prefix and name.startswith(base_prefix) else None


def _find(name: str, source, base_prefix: str) -> Optional[str]:
    for cand in (name, _base_model_name(name, base_prefix)):
        if cand is not None and cand in source:
            return cand
    return None


def resolve_names(decls: Iterable[ParamDecl], source, base_prefix: str = "") -> Dict[str, Optional[str]]:
    """Declared name -> name in the source (itself, its base-model form, or the
    tensor it is tied to); None when absent."""
    out = {}
    for d in decls:
        found = _find(d.name, source, base_prefix)
        if d.tied_to is not None:
            # A tied tensor is the tensor it is tied to; a copy in the file is compared with it, not used.
            found = _find(d.tied_to, source, base_prefix) or found
        out[d.name] = found
    return out


def check(decls: List[ParamDecl], source, base_prefix: str = "") -> Dict[str, Optional[str]]:
    """Raise one `WeightsError` for everything that is wrong; return the name map."""
    names = resolve_names(decls, source, base_prefix)
    missing = [n for n, src in names.items() if src is None]
    used = {src for src in names.values() if src is not None}
    declared = {d.name for d in decls} | {b for d in decls if (b := _base_model_name(d.name, base_prefix))}
    unexpected = [n for n in source.names() if n not in used and n not in declared]
    wrong_shape, wrong_dtype = [], []
    for d in decls:
        src = names[d.name]
        if src is None:
            continue
        if tuple(source.shape(src)) != tuple(d.shape):
            wrong_shape.append((src, source.shape(src), d.shape))
        dt = source.dtype(src)
        is_float = isinstance(dt, torch.dtype) and dt.is_floating_point
        if d.role == "index":
            if is_float:
                wrong_dtype.append((src, dt))
        elif not is_float:
            wrong_dtype.append((src, dt))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(missing, unexpected, wrong_shape, wrong_dtype)
    return names


def target_dtype(role: str, stored: torch.dtype, compute: torch.dtype, cast_float32: bool = False) -> torch.dtype:
    """The dtype a tensor is kept in on the device.

    float32 engine: every floating tensor in float32. bfloat16 engine: 16-bit
    tensors in bfloat16, a tensor stored in 32-bit stays in 32-bit unless
    `cast_float32` asks for its rounding (the reference's `amp='bf16'` rounds
    every weight, module.py:395-432); biases and norm parameters are widened to
    float32 (value-preserving), which is what the kernels read; integer tables in
    int32."""
    if role == "index":
        return torch.int32
    if compute == torch.float32 or role == "vector":
        return torch.float32
    if stored in (torch.float32, torch.float64) and not cast_float32:
        return torch.float32
    return torch.bfloat16


def load_tensors(decls: List[ParamDecl], source, compute: torch.dtype, device, base_prefix: str = "",
                 cast_float32: bool = False) -> Dict[str, torch.Tensor]:
    """Check, then read every declared tensor to `device` in its target dtype.
    Tensors that resolve to the same source tensor share one device buffer."""
    names = check(decls, source, base_prefix)
    by_source: Dict[tuple, torch.Tensor] = {}
    out = {}
    kept_wide, halves = [], []
    tied_differ = []
    for d in decls:
        src = names[d.name]
        stored = source.dtype(src)
        dt = target_dtype(d.role, stored, compute, cast_float32)
        if dt == torch.float32 and compute != torch.float32 and d.role in ("matrix", "table"):
            kept_wide.append(d.name)
        if stored == torch.float16 and dt == torch.bfloat16:
            halves.append(d.name)
        key = (src, dt)
        if key not in by_source:
            t = source.tensor(src)
            by_source[key] = t.to(device=device, dtype=dt).contiguous()
        out[d.name] = by_source[key]
        if d.tied_to is not None:
            own = _find(d.name, source, base_prefix)
            if own is not None and own != src:
                # the checkpoint holds a copy of its own of the tied tensor (the reference takes the
                # tie for granted, module.py:142-159): it must say the same, or the file is another model's
                a, b = source.tensor(own), source.tensor(src)
                if a.shape != b.shape or not torch.equal(a, b.to(a.dtype)):
                    tied_differ.append((own, src))
    if tied_differ:
        raise WeightsError([], [], [], [], tied_differ)
    import sys
    if halves:
        print(f"[transformers_neuronx_amd] {len(halves)} tensors are stored in float16 and are rounded to bfloat16, "
              f"the one 16-bit format of the kernels (3 bits of the fraction are lost; first: {halves[0]}); "
              f"dtype float32 keeps every bit", file=sys.stderr, flush=True)
    if kept_wide:
        print(f"[transformers_neuronx_amd] {len(kept_wide)} matrices are stored in 32-bit and stay so in this "
              f"{str(compute).replace('torch.', '')} engine (first: {kept_wide[0]}): their products run on the "
              f"float32 kernel, slower and at twice the memory; cast_float32_weights=True rounds them at load",
              file=sys.stderr, flush=True)
    return out
