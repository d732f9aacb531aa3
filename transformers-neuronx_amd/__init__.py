"""An inference engine for OPT-family decoders on one AMD MI355X."""
__version__ = "0.1.0"

from .config import ContinuousBatchingConfig, EngineConfig, GenerationConfig, NeuronConfig  # noqa: F401
from .sampling import SamplingParams  # noqa: F401


def __getattr__(name):
    # the model classes pull in torch-heavy modules: loaded when first asked for
    if name in ("OPTForSampling", "OPTForGreedySearch"):
        from .opt import model
        return getattr(model, name)
    if name == "NeuronAutoModelForCausalLM":
        from .modeling_auto import NeuronAutoModelForCausalLM
        return NeuronAutoModelForCausalLM
    if name == "testing":
        import importlib
        return importlib.import_module(".testing", __name__)
    if name == "LLMEngine":
        from .engine.engine import LLMEngine
        return LLMEngine
    raise AttributeError(name)
