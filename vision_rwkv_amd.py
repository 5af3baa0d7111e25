"""Import alias: the package directory is named ``vision-rwkv_amd`` (not a Python identifier),
so ``import vision_rwkv_amd`` loads it from there under this name."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vision-rwkv_amd")
_spec = importlib.util.spec_from_file_location(
    "vision_rwkv_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_mod = importlib.util.module_from_spec(_spec)
sys.modules["vision_rwkv_amd"] = _mod
_spec.loader.exec_module(_mod)
