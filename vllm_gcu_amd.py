"""Import shim: the package directory is named ``vllm-gcu_amd`` (not a valid
Python identifier), so this module makes it importable as ``vllm_gcu_amd`` by
pointing its ``__path__`` at that directory and running its ``__init__``."""
import os as _os

_pkg_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "vllm-gcu_amd")
__path__ = [_pkg_dir]
with open(_os.path.join(_pkg_dir, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_pkg_dir, "__init__.py"), "exec"))
del _f
