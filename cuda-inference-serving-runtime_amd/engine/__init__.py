from .context import StepContext, StepArray, Batch, GroupView, Workspace
from .runner import ModelRunner, StepEntry
from .loading import load_model, write_random_model, random_model, parse_dtype, build_from_config_dict
