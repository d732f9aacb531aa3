"""From a model folder and an `EngineConfig` to a runner with its cache."""
import os
from typing import Optional

import torch

from ..cache.manager import CacheManager
from ..config.engine_config import EngineConfig
from ..config.registry import read_config, resolve
from ..kernels import make_ops
from ..weights.loader import Checkpoint, TensorDict
from ..weights.random_init import random_tensors
from .model import DecoderModel
from .runner import ModelRunner


def _device_of(cfg: EngineConfig) -> torch.device:
    dev = torch.device(cfg.device)
    if cfg.kernels == "hip" and dev.type != "cuda":
        raise RuntimeError("the HIP kernels need a GPU device (cuda:N); "
                           "kernels='reference' is the only backend that runs elsewhere")
    return dev


def size_page_pool(cfg: EngineConfig, bytes_per_page: int, device: torch.device) -> int:
    """Pages per group: as told, or for `max_tokens`, or what free memory allows."""
    if cfg.num_pages is not None:
        return cfg.num_pages
    if cfg.max_tokens is not None:
        return max(1, -(-cfg.max_tokens // cfg.page_size))
    if device.type == "cuda" and bytes_per_page:
        free, _ = torch.cuda.mem_get_info(device)
        return max(1, int(free * cfg.memory_fraction) // bytes_per_page)
    return 256


def _cache_bytes(cfg: EngineConfig, bytes_per_page: int, total: int) -> int:
    """The cache's size as far as it is known before it is made (a quarter of the device's memory stands in
    for one sized from what is left)."""
    if cfg.num_pages is not None:
        return cfg.num_pages * bytes_per_page
    if cfg.max_tokens is not None:
        return -(-cfg.max_tokens // cfg.page_size) * bytes_per_page
    return total // 4


def _room_for_weight_copies(cfg: EngineConfig, model: DecoderModel, bytes_per_page: int, device):
    """Whether the matrices get a second, tile-ordered copy for the few-rows product (`weight_copies`): True
    when matrices twice over and the cache asked for fit 90 % of the device's memory, "later" when they do
    not (then as many as fit are made once the weights are loaded), or what the configuration says."""
    if cfg.weight_copies is not None and (not cfg.weight_copies or cfg.weight_copy_bytes is None):
        return bool(cfg.weight_copies)
    if device.type != "cuda" or cfg.dtype != torch.bfloat16:
        return False
    if cfg.weight_copy_bytes is not None:
        return "later"
    matrices = sum(2 * int(torch.Size(d.shape).numel()) for d in model.param_decls() if d.role in ("matrix", "table"))
    _, total = torch.cuda.mem_get_info(device)
    return True if 2.2 * matrices + _cache_bytes(cfg, bytes_per_page, total) <= 0.9 * total else "later"


def build_runner(model_config, source, cfg: EngineConfig) -> ModelRunner:
    """`model_config` a typed configuration, `source` a `Checkpoint` or `TensorDict`."""
    device = _device_of(cfg)
    arch = resolve(model_config.to_dict())
    model = DecoderModel(arch.build_spec(model_config))
    ops = make_ops(cfg.kernels, cfg.dtype, device)
    needs = model.cache_needs()
    pad = cfg.page_pad_bytes if device.type == "cuda" else 0
    bytes_per_page = CacheManager.bytes_per_page(needs, cfg.page_size, cfg.dtype, pad)
    if hasattr(ops, "decode_copies"):
        ops.decode_copies = _room_for_weight_copies(cfg, model, bytes_per_page, device)
    later = getattr(ops, "decode_copies", None) == "later"
    model.load(source, ops, cfg.dtype, device, cast_float32=cfg.cast_float32_weights, finish=not later)
    if hasattr(source, "release"):
        source.release()        # before the cache is sized and made: what the source held is free again,
        if device.type == "cuda":  # and goes back to the device, so that the cache's large blocks find room
            torch.cuda.empty_cache()
    if later:
        # the copies that fit beside the weights and the cache, with a twentieth of the device and 4 GB to spare
        free, total = torch.cuda.mem_get_info(device)
        room = free - _cache_bytes(cfg, bytes_per_page, total) - total // 20 - (4 << 30)
        if cfg.weight_copy_bytes is not None:
            room = min(room, cfg.weight_copy_bytes)
        ops.copy_bytes = ops.finish_weights(max(0, room))
        model.finish_load()
        torch.cuda.empty_cache()
    num_pages = size_page_pool(cfg, bytes_per_page, device)
    cache = CacheManager(needs, cfg.page_size, num_pages, cfg.max_num_seqs, cfg.dtype, device, page_pad_bytes=pad)
    return ModelRunner(model, cache, ops, use_graphs=cfg.use_graphs)


def runner_from_folder(folder: str, cfg: EngineConfig) -> ModelRunner:
    _, model_config = read_config(folder)
    return build_runner(model_config, Checkpoint(folder), cfg)


def runner_from_random(model_config, seed: int, cfg: EngineConfig, storage: Optional[torch.dtype] = None) -> ModelRunner:
    """Random weights drawn on the device, without a folder (for models too large
    to write for a measurement). `storage` is the precision the matrices are drawn in (the engine's own
    if not given): a float32 engine on bfloat16-drawn matrices has the very weights of a bfloat16 engine
    with the same seed."""
    device = _device_of(cfg)
    arch = resolve(model_config.to_dict())
    spec = arch.build_spec(model_config)
    decls = DecoderModel(spec).param_decls()
    if storage is None:
        storage = torch.float32 if cfg.dtype == torch.float32 else torch.bfloat16
    source = TensorDict(random_tensors(decls, spec.init_std, seed, storage, device))
    return build_runner(model_config, source, cfg)       # the source alone holds the tensors, and lets go of them
