"""Import name of the package that lives in the folder ``jax-llm-examples_amd/``.

The folder's name has a hyphen and so cannot be written in an ``import``
statement.  This module turns itself into that package: it takes the folder as
its ``__path__`` and runs the folder's ``__init__.py`` in its own namespace, so
``import jax_llm_examples_amd.config`` finds ``jax-llm-examples_amd/config``.
"""
import os as _os

_pkg_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "jax-llm-examples_amd")
__path__ = [_pkg_dir]
__package__ = __name__
if __spec__ is not None:
    __spec__.submodule_search_locations = __path__
with open(_os.path.join(_pkg_dir, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_pkg_dir, "__init__.py"), "exec"))
del _f
