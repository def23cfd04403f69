"""Abstract base class of calibrators, under the reference's module path (calib/calibrator.py)."""

from .max import _Calibrator

__all__ = ["_Calibrator"]
