from .engine import Engine, EngineOptions, StepEntry, StepError
