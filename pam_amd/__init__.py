"""MI355X-native piecewise-affine arithmetic (PAM): the GPU hot path of epfml/pam.

    import pam_amd as pam
    y = pam.matmul(a, b, approx_bwd=True)

The names of the reference's `pam` package that live on this path are re-exported here
(pam/__init__.py:8-10).
"""
from .pam_ops import *          # noqa: F401,F403
from .composites import *       # noqa: F401,F403
from .pam_opt import *          # noqa: F401,F403
from . import pam_experimental  # noqa: F401
from . import cuda_bindings     # noqa: F401
from . import pam_ops           # noqa: F401
from . import composites        # noqa: F401
