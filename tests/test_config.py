"""Configuration and registry."""
import json

import pytest

from conftest import TINY_A, TINY_B
from transformers_neuronx_amd.config import (ConfigError, EngineConfig, NeuronConfig, ContinuousBatchingConfig,
                                             known_architectures, parse_dtype, read_config, resolve)
from transformers_neuronx_amd.opt.config import OPTConfig


def test_reads_every_key():
    a = OPTConfig.from_dict(TINY_A)
    assert (a.vocab_size, a.hidden_size, a.num_hidden_layers, a.num_attention_heads) == (512, 64, 2, 4)
    assert (a.ffn_dim, a.max_position_embeddings, a.word_embed_proj_dim, a.head_size) == (256, 128, 64, 16)
    assert a.do_layer_norm_before and a.enable_bias and a.layer_norm_elementwise_affine
    b = OPTConfig.from_dict(TINY_B)
    assert (b.word_embed_proj_dim, b.head_size, b.activation_function) == (48, 32, "gelu")
    assert not b.do_layer_norm_before and not b.enable_bias and not b.layer_norm_elementwise_affine
    assert b.layer_norm_eps == 3e-4 and b.init_std == 0.05


def test_defaults_follow_the_family():
    raw = {k: TINY_A[k] for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                  "ffn_dim", "max_position_embeddings")}
    c = OPTConfig.from_dict(raw)
    assert c.word_embed_proj_dim == c.hidden_size
    assert c.do_layer_norm_before and c.enable_bias and c.activation_function == "relu"
    assert c.layer_norm_eps == 1e-5 and c.eos_token_id == 2 and c.pad_token_id == 1


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "ffn_dim", "max_position_embeddings"])
def test_missing_key_is_named(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        OPTConfig.from_dict(raw)


@pytest.mark.parametrize("key,value,word", [
    ("hidden_size", 66, "multiple"), ("activation_function", "swish", "activation_function"),
    ("vocab_size", 0, "positive"), ("num_hidden_layers", "2", "integer"), ("enable_bias", 1, "true or false"),
    ("layer_norm_eps", 0.0, "positive"), ("ffn_dim", 2.5, "integer")])
def test_bad_values_are_refused(key, value, word):
    raw = dict(TINY_A)
    raw[key] = value
    with pytest.raises(ConfigError, match=word):
        OPTConfig.from_dict(raw)


def test_unknown_keys_are_ignored_and_round_trip(tmp_path):
    raw = dict(TINY_B, dropout=0.1, layerdrop=0.0, _name_or_path="x")
    c = OPTConfig.from_dict(raw)
    c.save(str(tmp_path))
    arch, again = read_config(str(tmp_path))
    assert again == c and arch.name == "OPTForCausalLM"
    assert json.load(open(tmp_path / "config.json"))["architectures"] == ["OPTForCausalLM"]


def test_registry():
    assert "OPTForCausalLM" in known_architectures()
    assert resolve({"architectures": ["OPTForCausalLM"]}).config_class is OPTConfig
    assert resolve({"model_type": "opt"}).name == "OPTForCausalLM"
    with pytest.raises(ConfigError, match="known architectures"):
        resolve({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    from transformers_neuronx_amd.opt.model import OPTForSampling
    assert resolve({"model_type": "opt"}).user_class() is OPTForSampling


def test_engine_config():
    assert parse_dtype("bf16") == parse_dtype("bfloat16") and parse_dtype("f32") == parse_dtype("float32")
    with pytest.raises(ValueError):
        parse_dtype("int8")
    with pytest.raises(ValueError, match="page_size"):
        EngineConfig(page_size=24)
    with pytest.raises(ValueError, match="kernels"):
        EngineConfig(kernels="cpu")
    cb = ContinuousBatchingConfig(batch_size_for_shared_caches=4, max_model_len=128)
    assert cb.max_num_seqs == 4
    cb.init_cache_engine(block_size=32, num_blocks=10)
    assert NeuronConfig(continuous_batching=cb).continuous_batching.num_blocks == 10
    with pytest.raises(ValueError, match="float32"):
        NeuronConfig(cast_logits_dtype="bfloat16")
    # the reference's other keywords (config.py:206-363): layouts and fusions are taken and change nothing,
    # what would change the result and has no counterpart is refused, a name it does not have is an error
    nc = NeuronConfig(attention_layout="BSH", fuse_qkv=True, weight_tiling=True, compilation_worker_count=4,
                      sequence_parallel_norm=True, output_all_logits=True)
    assert nc.fuse_qkv and nc.attention_layout == "BSH" and nc.output_all_logits and nc.quant is None
    for bad in (dict(quant=object()), dict(log_softmax_scores=True), dict(group_query_attention="shard-over-heads"),
                dict(is_eagle_draft=True), dict(has_pre_attention_norm=False)):
        with pytest.raises(ValueError, match="no counterpart"):
            NeuronConfig(**bad)
    with pytest.raises(TypeError, match="unknown"):
        NeuronConfig(no_such_switch=1)


def test_sequence_length_guard():
    from transformers_neuronx_amd.opt.model import OPTForSampling
    with pytest.raises(ValueError, match="position embedding"):
        OPTForSampling(OPTConfig.from_dict(TINY_A), n_positions=129, amp="f32")
    with pytest.raises(ValueError, match="one GPU"):
        OPTForSampling(OPTConfig.from_dict(TINY_A), n_positions=64, amp="f32", tp_degree=2)


def test_auto_model_picks_the_class_the_folder_names(tmp_path):
    """modeling_auto.py:30-47: the class comes from config.json; an unknown model is an AssertionError."""
    import json
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM, OPTForSampling
    from conftest import TINY_A
    good = tmp_path / "good"
    good.mkdir()
    (good / "config.json").write_text(json.dumps(TINY_A))
    model = NeuronAutoModelForCausalLM.from_pretrained(str(good), batch_size=2, amp="f32", n_positions=64,
                                                       kernels="reference", device="cpu")
    assert isinstance(model, OPTForSampling) and model.config.hidden_size == 64
    by_type = dict(TINY_A, architectures=["SomethingElse"])
    (good / "config.json").write_text(json.dumps(by_type))
    assert isinstance(NeuronAutoModelForCausalLM.from_pretrained(str(good), amp="f32", n_positions=64), OPTForSampling)
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text(json.dumps(dict(TINY_A, architectures=["LlamaForCausalLM"], model_type="llama")))
    with pytest.raises(AssertionError, match="not supported"):
        NeuronAutoModelForCausalLM.from_pretrained(str(bad))


def test_console_scripts_of_the_package_resolve():
    """pyproject.toml names the reference's console scripts for this architecture and the trace replay."""
    import importlib
    import os
    try:
        import tomllib
    except ImportError:
        tomllib = pytest.importorskip("tomli")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "pyproject.toml"), encoding="utf-8") as fp:
        project = tomllib.loads(fp.read())
    scripts = project["project"]["scripts"]
    assert set(scripts) == {"opt_demo", "opt_gen_random_pretrained", "trace_run"}
    for target in scripts.values():
        module, _, name = target.partition(":")
        assert callable(getattr(importlib.import_module(module), name))
    for package in project["tool"]["setuptools"]["packages"]:
        folder = package.replace("transformers_neuronx_amd", "transformers-neuronx_amd").replace(".", "/")
        assert os.path.isfile(os.path.join(root, folder, "__init__.py")), package
