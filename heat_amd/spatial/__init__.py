"""Distance functions (subset of heat/spatial)."""
from . import distance
from .distance import *  # noqa: F401,F403
