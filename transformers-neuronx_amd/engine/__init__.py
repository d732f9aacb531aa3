from .batch import GroupView, StepContext, StepEntry, build_context
from .model import DecoderModel, model_param_decls
from .runner import ModelRunner
