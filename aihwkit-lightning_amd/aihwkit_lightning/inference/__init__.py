"""Post-training tools."""
from .calibration.calibration import calibrate_input_ranges, InputRangeCalibrationType

__all__ = ["calibrate_input_ranges", "InputRangeCalibrationType"]
