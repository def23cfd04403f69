"""Calibrators."""

from .max import MaxCalibrator, _Calibrator

__all__ = ["MaxCalibrator"]
