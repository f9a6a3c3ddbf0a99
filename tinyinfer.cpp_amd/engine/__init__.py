from .engine import Engine, StepEntry, EngineError
from .context import StepContext
from ..ops.kernels import required_libraries
