"""rocal_amd: MI355X-native augmentation hot path for rocAL (C ABI in include/rocal_mi355x.h)."""
from . import _lib, ops  # noqa: F401

__all__ = ["ops", "_lib"]
