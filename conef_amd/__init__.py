"""MI355X-native ConEF gradient compression: DDP communication hooks and count-sketch error
compressors backed by hand-written gfx950 HIP kernels (conef_amd/csrc) through a C-ABI library."""
from . import _lib  # noqa: F401
from ._pools import release  # noqa: F401  (drops the shared plans, staging, workspaces and side streams)

__all__ = ["_lib", "release"]
