"""`OPTForSampling`: the user-facing class of the OPT architecture, in the reference's manner
(opt/model.py:34-193). Everything it does is the architecture-free `CausalLMForSampling`."""
from ..causal_lm import CausalLMForSampling
from .spec import ARCHITECTURE


class OPTForSampling(CausalLMForSampling):
    architecture = ARCHITECTURE


class OPTForGreedySearch(OPTForSampling):
    """Greedy token selection on the device (reference: opt/model.py:534-570)."""

    def sample(self, input_ids, sequence_length, start_ids=None, **_):
        return super().sample(input_ids, sequence_length, start_ids=start_ids, top_k=1)
