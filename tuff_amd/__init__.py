"""tuff_amd: a small, whole inference engine for one MI355X (gfx950).

From a model folder (config.json + model.safetensors) to the next token: typed configuration and
architecture registry, weights by name, layers put together from parts, a paged cache with
per-request state slots, one step function over mixed batches, a scheduler, sampling, and
hand-written HIP kernels beneath all of it.
"""
__version__ = "0.1.0"

from .config.base import ConfigError, ModelConfig  # noqa: F401
from .models.registry import (architectures, build_model, config_from_dict,  # noqa: F401
                              load_config, register_architecture)
