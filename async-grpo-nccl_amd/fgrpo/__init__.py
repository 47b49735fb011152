"""Host side of the MI355X fused logprob + GRPO path (ctypes over libfgrpo.so)."""
from . import _lib  # noqa: F401
from .build import build, LIB_PATH  # noqa: F401
