"""DAC / ADC / output-noise settings of one analog tile (reference ``io.py:22-60``)."""
from dataclasses import dataclass
from .helpers import _PrintableMixin


@dataclass
class IOParameters(_PrintableMixin):
    """Peripheral behaviour of a tile. Resolutions > 1 mean "number of steps",
    values in (0, 1) mean "1 / number of steps", values <= 0 switch the converter off."""

    inp_res: float = -1
    out_noise: float = 0.0
    out_noise_per_channel: bool = False
    out_bound: float = 0.0
    out_res: float = -1
