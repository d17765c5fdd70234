"""Drop-in module name for the reference's core/norm_dist.py: re-exports `sortnet_amd.functional`."""
from .functional import *  # noqa: F401,F403
from .functional import __all__  # noqa: F401
