from .engine import Engine, GenerateChunk, GenerationResult, parse_dtype  # noqa: F401
from .runner import CacheExhausted, ModelRunner, StepEntry  # noqa: F401
from .scheduler import Request, Scheduled, Scheduler  # noqa: F401
