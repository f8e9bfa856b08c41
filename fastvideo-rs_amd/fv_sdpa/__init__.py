"""Python mirror of the MI355X SDPA path (ctypes over libfv_sdpa_hip.so).

torch is used only for device memory and streams.
"""
from ._lib import FvDeclined, FvError, LIB_PATH, build, lib  # noqa: F401
from .ops import *  # noqa: F401,F403
from .vsa import *  # noqa: F401,F403
from .sdpa import *  # noqa: F401,F403
from .prep import *  # noqa: F401,F403
from .kv_cache import *  # noqa: F401,F403
