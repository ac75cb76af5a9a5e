from .step import Engine, StepError, require_gpu, resolve_dtype
