"""Calibrators."""

from .max import MaxCalibrator, _Calibrator
from .mse import MseCalibrator

__all__ = ["MaxCalibrator", "MseCalibrator"]
