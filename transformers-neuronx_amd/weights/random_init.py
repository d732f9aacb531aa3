"""Random weights from a configuration and a seed.

`write_random_model` makes a model folder (config.json, model.safetensors) that
the ordinary loader reads; `random_tensors` makes the same tensors in memory, on
any device, for models too large to write for a measurement.

Reference: opt/gen_random_pretrained.py:32-102 draws `init_std * randn` for
matrices and zeros for norm parameters and biases (:89), which leaves every
norm's output zero; here biases are drawn like matrices and norm weights around
one, so that no part is switched off.
"""
import json
import os
from typing import Dict, List

import torch
from safetensors.torch import save_file

from ..parts.spec import ParamDecl

_STORAGE = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def random_tensors(decls: List[ParamDecl], std: float, seed: int, matrix_dtype: torch.dtype,
                   device="cpu") -> Dict[str, torch.Tensor]:
    """Tensors in the order of `decls` from one generator seeded once. Matrices
    and tables are stored in `matrix_dtype`, vectors in float32. A tied tensor
    is not drawn: the loader takes the tensor it is tied to."""
    gen = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for d in decls:
        if d.tied_to is not None or d.name in out:
            continue
        if d.role == "index":
            raise ValueError(f"no random rule for integer table {d.name}")
        t = torch.randn(d.shape, generator=gen, device=device, dtype=torch.float32) * std
        if d.init == "around_one":
            t += 1.0
        out[d.name] = t if d.role == "vector" else t.to(matrix_dtype)
    return out


def write_random_model(config, folder: str, seed: int, dtype=None) -> str:
    """Write `folder/config.json` and `folder/model.safetensors` for a typed config.
    `dtype` (a torch dtype or its name) is the storage dtype of matrices and
    tables; it defaults to the config's `torch_dtype`."""
    from ..config.registry import resolve
    from ..engine.model import model_param_decls
    arch = resolve(config.to_dict())
    spec = arch.build_spec(config)
    if dtype is None:
        dtype = _STORAGE[config.torch_dtype]
    elif isinstance(dtype, str):
        dtype = _STORAGE[dtype]
    tensors = random_tensors(model_param_decls(spec), spec.init_std, seed, dtype)
    os.makedirs(folder, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {v: k for k, v in _STORAGE.items()}[dtype]
    with open(os.path.join(folder, "config.json"), "w") as fp:
        json.dump(raw, fp, indent=2)
    path = os.path.join(folder, "model.safetensors")
    save_file({k: v.contiguous() for k, v in tensors.items()}, path, metadata={"format": "pt"})
    os.chmod(path, 0o644)      # the writer leaves it readable by its owner alone; a model folder is for others too
    return folder
