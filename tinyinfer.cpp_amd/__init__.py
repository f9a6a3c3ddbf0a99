"""tinyinfer for AMD MI355X: a small, whole inference engine for the Qwen3 dense
decoder.  Configuration, weights, parts, cache and scheduler are plain Python;
everything that touches a token's numbers is a hand-written HIP kernel."""
from .config.base import ConfigError, read_config_json
from .config.qwen3 import Qwen3Config
from .registry import register_architecture, registered_architectures, config_and_spec
from .parts.registry import register_part, build_part
from . import parts as _parts          # noqa: F401  registers the built-in parts
from . import models as _models        # noqa: F401  registers the built-in architecture
from .models import Model, ModelSpec, LayerSpec, PartSpec
from .engine import Engine, StepEntry
from .engine.scheduler import Scheduler, Request
from .sampling import SamplingParams
from .api import LLM, generate_ids, GenerationStats

__all__ = ["ConfigError", "read_config_json", "Qwen3Config", "register_architecture",
           "registered_architectures", "config_and_spec", "register_part", "build_part",
           "Model", "ModelSpec", "LayerSpec", "PartSpec", "Engine", "StepEntry", "Scheduler", "Request",
           "SamplingParams", "LLM", "generate_ids", "GenerationStats"]
