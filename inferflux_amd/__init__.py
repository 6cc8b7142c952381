"""An inference engine for the Qwen2.5 dense decoder on one AMD Instinct MI355X.

    from inferflux_amd import Engine, SamplingParams
    engine = Engine.load("model_dir", dtype="bfloat16")
    out = engine.generate([[1, 2, 3]], SamplingParams(temperature=0, max_tokens=16))
"""
from .sampling.params import SamplingParams

__all__ = ["Engine", "SamplingParams", "SchedulerConfig"]


def __getattr__(name):
    if name == "Engine":
        from .engine.engine import Engine
        return Engine
    if name == "SchedulerConfig":
        from .engine.scheduler import SchedulerConfig
        return SchedulerConfig
    raise AttributeError(name)
