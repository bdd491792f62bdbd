"""MI355X-native AdamW step with deterministic gradient norm and clip.

The directory name is not an importable identifier; load the package with
`__graft_entry__.load_package()` (module name `rl_cu_amd`).
"""
from . import binding, layout  # noqa: F401

__all__ = ["binding", "layout", "host", "build"]
