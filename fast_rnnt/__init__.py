"""``import fast_rnnt`` for code written against k2-fsa/fast_rnnt: the same package
name, the same public functions and the same submodule names, all resolving to the
MI355X build (:mod:`fast_rnnt_amd`).  Nothing is defined here; the objects ARE the
ones of fast_rnnt_amd, so state
such as the boundary-row cache is shared whichever name a caller imports
(``fast_rnnt.rnnt_loss`` the attribute is the function, as in the reference; the
submodule of that name is reached by ``import fast_rnnt.rnnt_loss``).

Reference counterparts: fast_rnnt/python/fast_rnnt/__init__.py:1-15 (export list),
setup.py:100-103 and CMakeLists.txt:50 (``__version__`` = "1.2", which this build
extends with a local version label).
"""
import importlib as _importlib
import sys as _sys

import fast_rnnt_amd as _impl

# `import fast_rnnt.rnnt_loss` / `from fast_rnnt.mutual_information import ...`
# (as in the reference, the attribute fast_rnnt.rnnt_loss itself is the function)
for _name in ("mutual_information", "rnnt_loss"):
    _sys.modules[__name__ + "." + _name] = _importlib.import_module("fast_rnnt_amd." + _name)

__all__ = [name for name in vars(_impl) if not name.startswith("_")
           and callable(getattr(_impl, name))]
globals().update({name: getattr(_impl, name) for name in __all__})

__version__ = _impl.__version__
