"""Import name for the package folder ``qwen25vl-lite_amd``.

The folder's name carries a hyphen, which Python's ``import`` statement cannot spell.
Importing this module loads that folder as the package ``qwen25vl_lite_amd`` (one module
tree, one set of registries) and puts it in ``sys.modules`` under this name, so
``import qwen25vl_lite_amd`` and ``from qwen25vl_lite_amd.config import ...`` both work.
"""
import importlib.util
import os
import sys

_name = "qwen25vl_lite_amd"
_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qwen25vl-lite_amd")
_spec = importlib.util.spec_from_file_location(
    _name, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[_name] = _module
_spec.loader.exec_module(_module)

if __name__ == "__main__":          # ``python -m qwen25vl_lite_amd ...`` is the command line
    from qwen25vl_lite_amd.cli import main
    raise SystemExit(main())
