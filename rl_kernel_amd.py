"""Import shim: exposes the directory ``rl-kernel_amd/`` (not a valid Python identifier) as the
package ``rl_kernel_amd``.  Sub-modules resolve through ``__path__``."""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "rl-kernel_amd")]
with open(_os.path.join(__path__[0], "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(__path__[0], "__init__.py"), "exec"))
del _f, _os
