"""Input-range calibration."""
from .calibration import calibrate_input_ranges, InputRangeCalibrationType

__all__ = ["calibrate_input_ranges", "InputRangeCalibrationType"]
