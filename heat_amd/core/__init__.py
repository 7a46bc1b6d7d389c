"""Array runtime subset needed by the k-means path."""
from .types import *  # noqa: F401,F403
from .communication import *  # noqa: F401,F403
from .devices import *  # noqa: F401,F403
from .dndarray import *  # noqa: F401,F403
from .factories import *  # noqa: F401,F403
from .base import *  # noqa: F401,F403
from .io import *  # noqa: F401,F403
from . import types, communication, devices, dndarray, factories, base, io  # noqa: F401
