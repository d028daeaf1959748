from .base_sampler import SamplerOutput  # noqa: F401
from .sampler import CacheConfig, Sampler  # noqa: F401
