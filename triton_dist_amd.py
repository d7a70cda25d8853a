"""Importable alias of the ``triton-distributed_amd`` package directory.

    import triton_dist_amd
    from triton_dist_amd.kernels import gqa_fwd_batch_decode
    from triton_dist_amd.layers import SpGQAFlashDecodeAttention
"""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
_pkg = importlib.import_module("triton-distributed_amd")
sys.modules[__name__] = _pkg
for _name, _mod in list(sys.modules.items()):
    if _name.startswith("triton-distributed_amd."):
        sys.modules[__name__ + _name[len("triton-distributed_amd"):]] = _mod
