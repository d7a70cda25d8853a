"""MI355X-native (gfx950) flash-decode: split-KV GQA paged decode + LSE-weighted combine.

The directory name is not a Python identifier; import it as
``importlib.import_module("triton-distributed_amd")`` with the repository root on
``sys.path``, or through the ``triton_dist_amd`` alias module next to it.
"""
from . import kernels, layers, utils  # noqa: F401
from ._lib import LIB_PATH, load_library  # noqa: F401
from .kernels import *  # noqa: F401,F403
from .layers import SpGQAFlashDecodeAttention  # noqa: F401

__version__ = "0.1.0"
