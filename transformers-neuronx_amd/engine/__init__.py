from .batch import (GroupView, PackedStep, StepContext, StepEntry, build_context, context_from, pack_step,
                    register_step_planner, unregister_step_planner)
from .model import DecoderModel, model_param_decls
from .runner import ModelRunner
