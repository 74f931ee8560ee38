from tritonix_amd.utils.spaces import Choice, Range, PowerOfTwo, SpaceConfig, ConfigSpace, ConfigParam
from tritonix_amd.utils.pruners import MonotonicCascadeTrie, CoordinateUnimodalFunction, CoordinateMonotonicFunction

__all__ = ["Choice", "Range", "PowerOfTwo", "SpaceConfig", "ConfigSpace", "ConfigParam",
           "MonotonicCascadeTrie", "CoordinateUnimodalFunction", "CoordinateMonotonicFunction"]
