"""Import shim: makes ``import qwen_engine_amd`` load the package whose folder is
``qwen-engine_amd/`` (a hyphen is not valid in a Python module name)."""
import importlib.util
import pathlib
import sys

_dir = pathlib.Path(__file__).resolve().parent / "qwen-engine_amd"
_spec = importlib.util.spec_from_file_location(
    __name__, _dir / "__init__.py", submodule_search_locations=[str(_dir)]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
