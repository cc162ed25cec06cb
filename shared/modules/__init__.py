"""The hook layer under the reference's import path: `from shared.modules import factories`."""
from . import factories  # noqa: F401
