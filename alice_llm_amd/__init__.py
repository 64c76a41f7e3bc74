"""alice-llm_amd: a small Gemma 2 library for one MI355X: configuration and registry, safetensors
weights, layers built from parts, a paged cache with slots, one step function, a generation loop
with sampling, and hand-written HIP kernels for gfx950 in bfloat16 and in true 32-bit."""
from .config import (ConfigError, Gemma2Config, config_from_dict, load_config, register_architecture,
                     registered_architectures)
from .config.presets import preset, preset_names
from .parts import Precision
from .weights.loader import UnexpectedTensorsWarning, WeightError, init_random, load_weights, write_random_model
from .weights.safetensors_io import WeightFileError
from .cache import Cache, CacheError
from .api import Model, load, sample, GenerationResult
from .engine.step import Engine
from .engine.generate import Generator, plan_prompt_steps, run_prompt_steps
from .sampling import Sampler
