"""Writes ``calib_cases.npz`` by RUNNING THE REFERENCE's ``calibrate_input_ranges`` on the CPU.

    PYTHONPATH=/root/reference/src python tests/golden/make_golden_calib.py

For every case of ``calib_cases.py``: the calibrated ``input_range`` after the whole stream and,
for the moving strategies, after every batch. Only data is written.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from calib_cases import CALIB_CASES, RANDPERM_SEED, make_batches  # noqa: E402  pylint: disable=wrong-import-position
from golden_cases import DTYPES  # noqa: E402  pylint: disable=wrong-import-position

from aihwkit_lightning.inference.calibration.calibration import (  # noqa: E402  (the reference)
    InputRangeCalibrationType,
    calibrate_input_ranges,
)
from aihwkit_lightning.nn import AnalogConv2d, AnalogLinear  # noqa: E402
from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig  # noqa: E402


def run_case(case, store):
    dtype = DTYPES[case["dtype"]]
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = case["max_input_size"]
    cfg.pre_post.input_range.enable = False
    cfg.forward.inp_res = -1
    torch.manual_seed(7)
    if case["conv"]:
        layer = AnalogConv2d(3, case["N"], 3, padding=1, dtype=dtype, rpu_config=cfg)
    else:
        layer = AnalogLinear(case["K"], case["N"], dtype=dtype, rpu_config=cfg)
    layer.eval()
    batches = make_batches(case)
    trace = []

    def loader():
        for x in batches:
            if layer.input_range is not None:
                trace.append(layer.input_range.detach().float().clone())
            yield (x,), {}

    torch.manual_seed(RANDPERM_SEED)
    kwargs = {} if case["std_alpha"] is None else {"std_alpha": case["std_alpha"]}
    calibrate_input_ranges(layer, InputRangeCalibrationType(case["kind"]), loader(),
                           quantile=case["quantile"], max_samples=case["max_samples"],
                           verbose=False, **kwargs)
    store[f"{case['name']}/ir"] = layer.input_range.detach().float().numpy()
    if case["kind"] in ("MovingStd", "MovingQuantile"):
        # trace[i] is the range before batch i was seen (3.0 for i = 0)
        store[f"{case['name']}/trace"] = torch.stack(trace).numpy()


def main():
    store = {}
    for case in CALIB_CASES:
        run_case(case, store)
        print("done", case["name"], store[f"{case['name']}/ir"])
    path = os.path.join(HERE, "calib_cases.npz")
    np.savez_compressed(path, **store)
    print(f"wrote {path}: {os.path.getsize(path) / 1e3:.1f} kB, {len(store)} arrays")


if __name__ == "__main__":
    main()
