"""Import name of the package whose sources live in the folder `alice-llm_amd/` (a hyphen cannot be
imported): this module points its search path there and runs that folder's __init__."""
import os as _os

_real = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "alice-llm_amd")
__path__[:] = [_real]
with open(_os.path.join(_real, "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(_real, "__init__.py"), "exec"))
del _f
