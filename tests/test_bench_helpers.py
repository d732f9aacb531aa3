"""The measurement's accounting: bytes and flops come from what the parts declare, and for OPT they are the
closed forms one writes down by hand; the record's `config` stays flat and within 20 keys."""
import json
import subprocess
import sys

import torch

from conftest import ROOT, TINY_A, TINY_B


def _model(raw):
    from transformers_neuronx_amd.config.registry import resolve
    from transformers_neuronx_amd.engine.model import DecoderModel
    arch = resolve(raw)
    cfg = arch.config_class.from_dict(raw)
    return cfg, DecoderModel(arch.build_spec(cfg))


def test_flops_and_cache_bytes_from_the_declarations():
    for raw in (TINY_A, TINY_B):
        cfg, model = _model(raw)
        h, f, l, v, e = cfg.hidden_size, cfg.ffn_dim, cfg.num_hidden_layers, cfg.vocab_size, cfg.word_embed_proj_dim
        tokens = 37
        # a whole prompt: every token meets the four attention matrices and the two of the feed-forward, attends to
        # (tokens + 1) / 2 keys on average (scores and weighted values), one row goes through the head
        projection = 2 * h * e if e != h else 0                 # into the model's width, and out of it again
        want = (tokens * (l * (2 * (4 * h * h + 2 * h * f) + 4 * h * (tokens + 1) / 2) + projection)
                + 2 * v * e + projection)
        assert model.step_flops(tokens, (tokens + 1) / 2, 1) == want
        # a decoded token reads the keys and values of every layer
        assert model.cache_bytes_read(100, torch.bfloat16) == 100 * 2 * l * h * 2
        assert model.cache_bytes_read(100, torch.float32, page_size=16) == 100 * 2 * l * h * 4


def test_windowed_layers_read_their_window_only():
    import toy_parts  # noqa: F401  (registers the toy parts)
    from transformers_neuronx_amd.engine.model import DecoderModel
    model = DecoderModel(toy_parts.toy_spec(window=24))
    # past the window another cached token costs only what the layers without a window read
    early = model.cache_bytes_read(24, torch.float32) - model.cache_bytes_read(23, torch.float32)
    late = model.cache_bytes_read(1000, torch.float32) - model.cache_bytes_read(999, torch.float32)
    assert 0 <= late < early


def test_the_record_is_flat_and_small(tmp_path):
    sys.path.insert(0, ROOT)
    import bench
    cfg, _ = _model({k: v for k, v in bench.raw_config("6.7b").items() if k != "name"})
    flat = bench.flat_config(cfg, {"model": "m", "global_batch": 8, "seq_len": 2048, "parallelism": "none",
                                   "layers_of_model": 32, "page_size": 64, "prompt_len": 1975, "prefill_tokens": 2048})
    assert len(flat) <= 20 and all(not isinstance(v, (list, dict)) for v in flat.values())
    for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "ffn_dim",
                "max_position_embeddings", "word_embed_proj_dim", "do_layer_norm_before", "activation_function"):
        assert key in flat
    # a config.json of any registered architecture, by file or by folder
    path = tmp_path / "config.json"
    path.write_text(json.dumps(TINY_B))
    assert bench.raw_config(str(path))["hidden_size"] == 96 and bench.raw_config(str(tmp_path))["vocab_size"] == 1000


def test_more_than_one_gpu_is_refused_in_one_line():
    done = subprocess.run([sys.executable, f"{ROOT}/bench.py", "--gpus", "2"], capture_output=True, text=True)
    assert done.returncode == 2 and len(done.stdout.strip().splitlines()) == 1
