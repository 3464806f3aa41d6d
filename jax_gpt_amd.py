"""Import shim: the package directory is named `jax-gpt_amd`, which Python cannot
import by name; this module loads it under the importable name `jax_gpt_amd`."""
import importlib.util as _ilu
import os as _os
import sys as _sys

_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "jax-gpt_amd")
_spec = _ilu.spec_from_file_location("jax_gpt_amd", _os.path.join(_dir, "__init__.py"),
                                     submodule_search_locations=[_dir])
_mod = _ilu.module_from_spec(_spec)
_sys.modules["jax_gpt_amd"] = _mod
_spec.loader.exec_module(_mod)
