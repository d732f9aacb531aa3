from .loops import sample_greedy, simple_sample  # noqa: F401
from .params import SamplingParams  # noqa: F401
from .sampler import Sampler  # noqa: F401
