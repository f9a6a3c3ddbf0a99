from .engine import Engine, StepEntry, StepContext, EngineError, required_libraries
