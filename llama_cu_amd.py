"""Import shim for the package that lives in the folder ``llama.cu_amd``.

The folder's name holds a dot, so ``import`` cannot name it.  This module loads
the folder as the package ``llama_cu_amd`` and puts it in its own place in
``sys.modules``: ``import llama_cu_amd`` and ``from llama_cu_amd.cache import X``
then work as for any package.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "llama.cu_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)
