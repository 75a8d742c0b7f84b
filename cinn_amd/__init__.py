"""cinn_amd: an MI355X (gfx950) GPU backend for the CINN tensor compiler.

``cinn_amd.frontend`` mirrors ``cinn.frontend`` (NetBuilder, Computation), ``cinn_amd.common`` mirrors
``cinn.common`` (types, targets) and ``cinn_amd.runtime`` exposes the C-ABI runtime
(``cinn_call_*`` intrinsics, hiprtc, code objects, device memory)."""
from . import _lib  # noqa: F401
from . import common, frontend, runtime  # noqa: F401

__all__ = ["common", "frontend", "runtime"]
