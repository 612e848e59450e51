from .engine import Engine, StepEntry, StepError
from .model import Model, declared_tensors
