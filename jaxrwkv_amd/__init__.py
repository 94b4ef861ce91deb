"""MI355X-native WKV recurrence (RWKV-7 / RWKV-6 / RWKV-4) behind the reference's ``inner_loop`` interface."""
from . import _lib  # noqa: F401  (loads nothing until first use)

__all__ = ["_lib"]
