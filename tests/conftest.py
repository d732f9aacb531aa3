import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations that differ in every size and option.
TINY_A = dict(
    architectures=["OPTForCausalLM"], model_type="opt",
    vocab_size=512, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, ffn_dim=256,
    max_position_embeddings=128, word_embed_proj_dim=64, do_layer_norm_before=True,
    activation_function="relu", enable_bias=True, layer_norm_elementwise_affine=True,
    layer_norm_eps=1e-5, init_std=0.02)
TINY_B = dict(
    architectures=["OPTForCausalLM"], model_type="opt",
    vocab_size=1000, hidden_size=96, num_hidden_layers=3, num_attention_heads=3, ffn_dim=320,
    max_position_embeddings=256, word_embed_proj_dim=48, do_layer_norm_before=False,
    activation_function="gelu", enable_bias=False, layer_norm_elementwise_affine=False,
    layer_norm_eps=3e-4, init_std=0.05)
# A third one whose sizes reach the paths that need them: head size 64, widths that are multiples of 128
# (the tile-ordered weight copies of the few-rows product), a vocabulary that is a multiple of 16.
TINY_C = dict(
    architectures=["OPTForCausalLM"], model_type="opt",
    vocab_size=640, hidden_size=128, num_hidden_layers=2, num_attention_heads=2, ffn_dim=256,
    max_position_embeddings=192, word_embed_proj_dim=128, do_layer_norm_before=True,
    activation_function="gelu_new", enable_bias=True, layer_norm_elementwise_affine=True,
    layer_norm_eps=1e-6, init_std=0.04)
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """{name: (folder, raw config, float32 tensors by name)} of the two tiny models, float32 on disk."""
    from safetensors.torch import load_file
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights import write_random_model
    out = {}
    for name, (raw, seed) in TINY.items():
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(OPTConfig.from_dict(raw), folder, seed, dtype="float32")
        with open(os.path.join(folder, "config.json")) as fp:
            cfg = json.load(fp)
        out[name] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return out


@pytest.fixture(scope="session")
def tiny_folders_bf16(tmp_path_factory):
    """The same models with matrices stored in bfloat16 (norm parameters and biases in float32)."""
    from safetensors.torch import load_file
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights import write_random_model
    out = {}
    for name, (raw, seed) in TINY.items():
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}_bf16"))
        write_random_model(OPTConfig.from_dict(raw), folder, seed, dtype="bfloat16")
        with open(os.path.join(folder, "config.json")) as fp:
            cfg = json.load(fp)
        out[name] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return out
