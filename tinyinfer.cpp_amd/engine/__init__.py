from .engine import Engine, StepEntry, EngineError, token_from_feedback
from .context import StepContext
from ..ops.kernels import required_libraries
