from .step import Engine, StepError, require_gpu, resolve_dtype
from .generate import GenerationResult, Generator, plan_batches
from .probe import StepProbe
