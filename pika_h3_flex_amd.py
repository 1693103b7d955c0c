"""Import shim: the package directory is named ``pika-h3-flex_amd`` (not a Python identifier), so
``import pika_h3_flex_amd`` loads it from there under this importable name."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pika-h3-flex_amd")
_spec = importlib.util.spec_from_file_location(
    "pika_h3_flex_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_mod = importlib.util.module_from_spec(_spec)
sys.modules["pika_h3_flex_amd"] = _mod
_spec.loader.exec_module(_mod)
