"""Import name of the package whose sources live in the folder ``gpt-fast_amd/``.

A folder name with a hyphen cannot be imported, so this module loads that folder as
the package ``gpt_fast_amd`` and puts it in its own place in ``sys.modules``;
``import gpt_fast_amd`` and ``from gpt_fast_amd.config import ...`` then work as for
any package.
"""
import importlib.util
import os
import sys

_folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpt-fast_amd")
_spec = importlib.util.spec_from_file_location(
    "gpt_fast_amd", os.path.join(_folder, "__init__.py"),
    submodule_search_locations=[_folder])
_package = importlib.util.module_from_spec(_spec)
sys.modules["gpt_fast_amd"] = _package
_spec.loader.exec_module(_package)

if __name__ == "__main__":          # python -m gpt_fast_amd ...  /  python gpt_fast_amd.py ...
    from gpt_fast_amd.engine.cli import cli
    sys.exit(cli())
