from .engine import DeviceToken, Engine, StepEntry, StepError
from .model import Model, declared_tensors
