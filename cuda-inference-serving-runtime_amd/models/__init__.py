from .model import Model, ScheduleEntry
from .llama import build_llama
