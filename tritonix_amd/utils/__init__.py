"""Tuning-space helpers: parameter domains (``spaces``) and the two search-space pruners (``pruners``)."""
from tritonix_amd.utils import pruners, spaces
from tritonix_amd.utils.pruners import *  # noqa: F401,F403
from tritonix_amd.utils.spaces import *  # noqa: F401,F403

__all__ = list(spaces.__all__) + list(pruners.__all__)
