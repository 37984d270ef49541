"""MI355X-native Llama inference engine (import name: ``runtime``)."""
from . import models as _models  # registers the architectures
from .config import (ConfigError, LlamaConfig, register_architecture, registered_architectures, preset, preset_names)
from .weights import WeightError, TensorSpec
from .cache import CacheManager, KVNeed, StateNeed, OutOfPages
from .parts import register_part, make_part
from .models import Model, ScheduleEntry
from .engine import ModelRunner, StepEntry, load_model, write_random_model
