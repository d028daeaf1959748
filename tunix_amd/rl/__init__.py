from . import common  # noqa: F401
from .rollout import HipRollout, RolloutConfig, RolloutOutput  # noqa: F401
