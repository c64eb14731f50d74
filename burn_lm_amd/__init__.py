"""Import name of the package whose sources live in ``burn-lm_amd/`` (a hyphen cannot appear in
an import statement).  This module points its search path there and runs that package's
``__init__``; ``import burn_lm_amd.engine`` then finds ``burn-lm_amd/engine``."""
import os as _os

_src = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "burn-lm_amd")
__path__ = [_src]
with open(_os.path.join(_src, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_src, "__init__.py"), "exec"))
del _f
