"""MI355X-native hybrid activation compression behind the HyC-LoRA operator API.

The directory name is not a Python identifier; import it with
    importlib.import_module("hyc-lora_amd")
from the repository root (or with the repository root on sys.path).
"""
from . import _abi  # noqa: F401

__all__ = ["_abi", "kernels", "operators"]


def __getattr__(name):
    import importlib
    if name in ("kernels", "operators"):
        return importlib.import_module(__name__ + "." + name)
    raise AttributeError(name)
