"""Put this file's parent directory on PYTHONPATH to make `import grouped_gemm` resolve to the
gfx950 implementation (what moe/grouped_gemm_util.py:3-6 of the reference imports)."""
import importlib.util
import os
import sys

_PKG = "hetu_galvatron_amd"
if _PKG not in sys.modules:
    _root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    _spec = importlib.util.spec_from_file_location(
        _PKG, os.path.join(_root, "__init__.py"), submodule_search_locations=[_root])
    _mod = importlib.util.module_from_spec(_spec)
    sys.modules[_PKG] = _mod
    _spec.loader.exec_module(_mod)

from hetu_galvatron_amd.grouped_gemm import backend, ops  # noqa: E402,F401
