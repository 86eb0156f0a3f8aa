"""Import alias: ``import flash_attention_triton_amd`` loads the package kept in the directory
``flash-attention-triton_amd/`` (whose name is not a Python identifier)."""

import importlib
import pathlib
import sys

_root = str(pathlib.Path(__file__).resolve().parent)
if _root not in sys.path:
    sys.path.insert(0, _root)

_pkg = importlib.import_module("flash-attention-triton_amd")
sys.modules[__name__] = _pkg
