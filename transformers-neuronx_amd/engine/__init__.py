from .batch import GroupView, PackedStep, StepContext, StepEntry, build_context, context_from, pack_step
from .model import DecoderModel, model_param_decls
from .runner import ModelRunner
