"""An OPT inference engine for one MI355X: typed configuration, safetensors
weights, layers assembled from parts, a paged cache manager, one step function,
a continuous-batching scheduler, sampling, and hand-written HIP kernels."""

__version__ = "0.1.0"

from .config import OptHyperParam, CacheParam, ConfigError  # noqa: F401
