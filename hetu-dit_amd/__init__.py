"""MI355X-native one-GPU DiT denoise-step hot path (drop-in for Hetu-DiT's
transformer-block / attention-processor layer).  All computation runs in
hand-written gfx950 HIP kernels behind the C ABI in ``include/hdit.h``."""
from . import _lib, ops  # noqa: F401
from ._lib import HditError, LIB_PATH  # noqa: F401

__all__ = ["ops", "HditError", "LIB_PATH"]
