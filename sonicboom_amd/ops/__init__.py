"""HIP kernels of the engine, called through ctypes (see ``kernels.py``)."""
from .library import KernelLibraryError, loaded_paths  # noqa: F401
from .kernels import *  # noqa: F401,F403
from .kernels import PAGE, MAX_CANDIDATES, ATTENTION_ROW_TILE, TALL_ROW_TILE  # noqa: F401
