"""Loads the product's Python binding (the package directory name has a hyphen)."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load():
    if "cann_hccl_amd" in sys.modules:
        return sys.modules["cann_hccl_amd"]
    path = os.path.join(ROOT, "cann-hccl_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("cann_hccl_amd", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["cann_hccl_amd"] = mod
    spec.loader.exec_module(mod)
    return mod
