"""tinyinfer for AMD MI355X: a small, whole inference engine for the Qwen3 dense
decoder.  Configuration, weights, parts, cache manager, step function, scheduler
and sampler are a C++ library (include/inference.h) over hand-written HIP kernels
(csrc/); this package binds it, and lets parts and architectures be defined in
Python beside the built-in ones."""
from .config.base import ConfigError, read_config_json
from .config.qwen3 import Qwen3Config
from .registry import register_architecture, registered_architectures, config_and_spec
from .parts.registry import register_part, build_part
from . import parts as _parts          # noqa: F401  registers the built-in parts
from .models import Model, ModelSpec, LayerSpec, PartSpec
from .engine import Engine, StepEntry, token_from_feedback
from .engine.scheduler import Scheduler, Request
from .sampling import SamplingParams
from .api import LLM, generate_ids, GenerationStats
from .weights import write_model_folder
from .native import load_plugin

__all__ = ["ConfigError", "read_config_json", "Qwen3Config", "register_architecture",
           "registered_architectures", "config_and_spec", "register_part", "build_part",
           "Model", "ModelSpec", "LayerSpec", "PartSpec", "Engine", "StepEntry", "token_from_feedback", "Scheduler", "Request",
           "SamplingParams", "LLM", "generate_ids", "GenerationStats", "write_model_folder", "load_plugin"]
