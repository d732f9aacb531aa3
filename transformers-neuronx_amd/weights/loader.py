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

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, expected {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is {got}, expected a floating type")
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


def _base_model_name(name: str) -> Optional[str]:
    return name[len("model."):] if name.startswith("model.") else None


def resolve_names(decls: Iterable[ParamDecl], source) -> Dict[str, Optional[str]]:
    """Declared name -> name in the source (itself, its base-model form, or the
    tensor it is tied to); None when absent."""
    out = {}
    for d in decls:
        found = None
        for cand in (d.name, _base_model_name(d.name)):
            if cand is not None and cand in source:
                found = cand
                break
        if d.tied_to is not None:
            # A tied tensor is the tensor it is tied to; a copy in the file is not read.
            for cand in (d.tied_to, _base_model_name(d.tied_to)):
                if cand is not None and cand in source:
                    found = cand
                    break
        out[d.name] = found
    return out


def check(decls: List[ParamDecl], source) -> Dict[str, Optional[str]]:
    """Raise one `WeightsError` for everything that is wrong; return the name map."""
    names = resolve_names(decls, source)
    missing = [n for n, src in names.items() if src is None]
    used = {src for src in names.values() if src is not None}
    declared = {d.name for d in decls} | {b for d in decls if (b := _base_model_name(d.name))}
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


def target_dtype(role: str, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    """The dtype a tensor is kept in on the device.

    float32 engine: every floating tensor in float32. bfloat16 engine: 16-bit
    tensors in bfloat16, a tensor stored in 32-bit stays in 32-bit; biases and
    norm parameters are widened to float32 (value-preserving), which is what the
    kernels read; integer tables in int32."""
    if role == "index":
        return torch.int32
    if compute == torch.float32 or role == "vector":
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load_tensors(decls: List[ParamDecl], source, compute: torch.dtype, device) -> Dict[str, torch.Tensor]:
    """Check, then read every declared tensor to `device` in its target dtype.
    Tensors that resolve to the same source tensor share one device buffer."""
    names = check(decls, source)
    by_source: Dict[tuple, torch.Tensor] = {}
    out = {}
    for d in decls:
        src = names[d.name]
        dt = target_dtype(d.role, source.dtype(src), compute)
        key = (src, dt)
        if key not in by_source:
            t = source.tensor(src)
            by_source[key] = t.to(device=device, dtype=dt).contiguous()
        out[d.name] = by_source[key]
    return out
