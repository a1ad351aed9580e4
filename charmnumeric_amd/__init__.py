"""MI355X-native executor back end for charmnumeric's per-partition array execution path."""
from . import _lib  # noqa: F401  (fails loudly when libcnhip.so has not been built)

__all__ = ["_lib"]
