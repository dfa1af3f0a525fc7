"""Import alias: the package lives in the folder ``llm-rs_amd`` (a hyphen is no
identifier), so ``import llm_rs_amd`` loads that folder under this name."""
import importlib.util
import pathlib
import sys

_root = pathlib.Path(__file__).resolve().parent.parent / "llm-rs_amd"
_spec = importlib.util.spec_from_file_location(
    __name__, _root / "__init__.py", submodule_search_locations=[str(_root)])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
