"""Calibration cases shared by the fixture writer (``make_golden_calib.py``) and the tests: a
single AnalogLinear (or AnalogConv2d) layer without input range, a fixed stream of batches (some
rows zeroed entirely: the reference drops those before taking statistics), one strategy."""
import torch

from golden_cases import DTYPES


def calib_case(name, kind, dtype="f32", K=40, N=6, max_input_size=16, batches=5, rows=12,
               quantile=0.99995, max_samples=1000, std_alpha=None, seed=0, conv=False):
    return dict(name=name, kind=kind, dtype=dtype, K=K, N=N, max_input_size=max_input_size,
                batches=batches, rows=rows, quantile=quantile, max_samples=max_samples,
                std_alpha=std_alpha, seed=seed, conv=conv)


CALIB_CASES = [
    calib_case("max_f32", "Max", seed=60),
    calib_case("max_bf16", "Max", dtype="bf16", seed=60),
    calib_case("moving_std_f32", "MovingStd", seed=61),
    calib_case("moving_std_bf16", "MovingStd", dtype="bf16", seed=61),
    calib_case("moving_std_alpha_f32", "MovingStd", std_alpha=2.5, batches=3, rows=33, seed=62),
    calib_case("moving_quantile_f32", "MovingQuantile", quantile=0.99, rows=40, seed=63),
    calib_case("moving_quantile_bf16", "MovingQuantile", dtype="bf16", quantile=0.9, rows=40, seed=63),
    calib_case("moving_quantile_default_f32", "MovingQuantile", rows=64, K=96, max_input_size=32,
               seed=64),
    calib_case("moving_quantile_one_f32", "MovingQuantile", quantile=1.0, seed=65),
    calib_case("cache_quantile_f32", "CacheQuantile", quantile=0.99, seed=66),
    calib_case("cache_quantile_subsampled_f32", "CacheQuantile", quantile=0.95, max_samples=25,
               batches=6, rows=10, seed=67),
    calib_case("cache_quantile_bf16", "CacheQuantile", dtype="bf16", quantile=0.99, seed=66),
    # convolution layer: statistics over the patches (3 channels, 3x3 kernel -> 27 patch entries)
    calib_case("conv_max_f32", "Max", K=27, N=4, max_input_size=10, batches=3, rows=2, seed=68,
               conv=True),
    calib_case("conv_moving_std_f32", "MovingStd", K=27, N=4, max_input_size=10, batches=3, rows=2,
               seed=69, conv=True),
]
CALIB_CASES_BY_NAME = {c["name"]: c for c in CALIB_CASES}
RANDPERM_SEED = 4321


def make_batches(c):
    """The stream of inputs: [rows, K] per batch (conv: [rows, 3, 7, 6] images). Every batch but
    the first has its rows 1 and 4 (if present) zeroed entirely."""
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(3000 + c["seed"])
    out = []
    for b in range(c["batches"]):
        if c["conv"]:
            x = torch.randn(c["rows"], 3, 7, 6, generator=gen) * (1.0 + 0.5 * b)
        else:
            x = torch.randn(c["rows"], c["K"], generator=gen) * (1.0 + 0.5 * b)
            if b > 0:
                x[1] = 0.0
                if c["rows"] > 4:
                    x[4] = 0.0
            x[0, :3] = x[2, :3]  # a few repeated values
        out.append(x.to(dtype))
    return out
