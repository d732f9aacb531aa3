"""`NeuronAutoModelForCausalLM.from_pretrained(folder, ...)`: the model class is the one the folder's
config.json names (reference: modeling_auto.py:30-47, which keys its table on `model_type` and asserts
on one it does not know). The table is the registry of `config/registry.py`."""
from .config.registry import ConfigError, read_config


class NeuronAutoModelForCausalLM:

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path, *model_args, **kwargs):
        try:
            arch, _ = read_config(pretrained_model_name_or_path)
        except ConfigError as e:
            raise AssertionError(f"{e} (not supported by this engine)") from None
        return arch.user_class().from_pretrained(pretrained_model_name_or_path, *model_args, **kwargs)
