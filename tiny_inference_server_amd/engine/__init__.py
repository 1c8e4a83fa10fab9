from .engine import Engine, StepOutput, resolve_dtype
