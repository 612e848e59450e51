"""imparo_amd: a small, whole LFM2 inference engine for one MI355X."""
from .config import (Lfm2Config, ModelPlan, LayerPlan, LayerCall, PartSpec, register_architecture,
                     plan_from_config, ConfigError)
from .parts import register_part
from .weights import write_random_model, WeightsError

__all__ = ["Lfm2Config", "ModelPlan", "LayerPlan", "LayerCall", "PartSpec", "register_architecture",
           "plan_from_config", "ConfigError", "register_part", "write_random_model", "WeightsError",
           "Engine", "StepEntry", "generate"]


def __getattr__(name):
    if name in ("Engine", "StepEntry", "StepError"):
        from . import engine
        return getattr(engine, name)
    if name in ("generate", "SamplingParams", "Scheduler", "Request"):
        from .engine import scheduler
        return getattr(scheduler, name)
    raise AttributeError(name)
