"""`import pam` for code written against epfml/pam: the same names, served by pam_amd.

The training forks and the hook layer of the reference import the package as `pam` and read
`pam.Linear`, `pam.Conv2d`, `pam.LayerNorm`, `pam.mean ... pam.pow`, `pam.pam_experimental.*`
(shared/modules/factories.py:13, 128-265; pam/__init__.py:8-10).  With this repository's root on
PYTHONPATH they get the MI355X implementation.  The submodules `pam.pam_ops`, `pam.cuda_bindings`,
`pam.pam_opt`, `pam.pam_experimental` and `pam.utils` are the pam_amd modules of the same names.
There is no `pam.native`: the CPU emulation is not part of this package.
"""
import sys as _sys

import pam_amd as _impl
from pam_amd import *                                   # noqa: F401,F403
from pam_amd import cuda_bindings, pam_experimental, pam_ops, pam_opt, utils   # noqa: F401

for _name in ("cuda_bindings", "pam_experimental", "pam_ops", "pam_opt", "utils"):
    _sys.modules[__name__ + "." + _name] = getattr(_impl, _name) if hasattr(_impl, _name) else __import__("pam_amd." + _name, fromlist=[_name])
del _name
