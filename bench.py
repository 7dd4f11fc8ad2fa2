"""Benchmark of the AnalogLinear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

Workload (the configuration the headline metric is quoted on): one AnalogLinear 4096 -> 4096,
bf16, 8192 tokens, 8 analog tiles of 512 inputs, learned input range (decay 0.01), 8-bit DAC and
ADC (out_bound 10), output noise 0.04, additive per-channel Gaussian weight noise 0.02, training
mode; one step = forward + straight-through backward (dX, dW, dBias, d input_range) on
synthetic N(0,1) inputs and N(0, 0.02^2) weights resident in HBM.

Prints ONE JSON line: whole-step throughput in algorithmic TFLOP/s (3 GEMMs x 2*M*N*K), the
roofline of the dominant kernel measured with HIP events on the launch stream, and the CPU
baseline (the torch-mode oracle on the host cores, on a token subsample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "aihwkit-lightning_amd"))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

M_TOKENS, K_IN, N_OUT, TILE = 8192, 4096, 4096, 512
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
# Bytes per launch that the L2s pull from / push to the fabric (HBM or Infinity Cache) are not
# measured by this run: they come from rocprofv3 FETCH_SIZE and WRITE_SIZE runs of
# `bench.py --kernels-only`, each scaled by what the same counter reads for the 256 MiB copy
# below. The table of the last such run is read from this file (and named in the line).
TRAFFIC_TABLE = os.path.join("profiles", "linear_fwd_bwd_4096x4096_8192tok_bf16_hbm_traffic.txt")
TRAFFIC_ROWS = {
    "linear_fwd": "ahl::k_fwd_pipe<",
    "linear_bwd_dx(+ir_grad)": "ahl::k_bwd_fast<ahl::BF16, 0",
    "linear_bwd_dw(+bias_grad)": "ahl::k_bwd_fast<ahl::BF16, 1",
}


def measured_traffic_bytes(kernel):
    """fetch + write bytes per launch of `kernel` from the committed counter table, or None."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_TABLE)) as handle:
            for line in handle:
                if line.startswith(TRAFFIC_ROWS[kernel]):
                    fetch, write = line.split()[-4:-2]
                    return int((float(fetch) + float(write)) * 2 ** 20)
    except (OSError, ValueError, KeyError):
        pass
    return None


def build_layer():
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.simulator.configs import (
        TorchInferenceRPUConfig, WeightClipType, WeightNoiseInjectionType,
    )

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = TILE
    cfg.forward.inp_res = 254
    cfg.forward.out_res = 254
    cfg.forward.out_bound = 10.0
    cfg.forward.out_noise = 0.04
    cfg.clip.type = WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
    cfg.clip.sigma = 2.5
    cfg.modifier.noise_type = WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL
    cfg.modifier.std_dev = 0.02
    ir = cfg.pre_post.input_range
    ir.enable, ir.dynamic, ir.learn_input_range = True, False, True
    ir.init_value, ir.init_from_data, ir.decay, ir.input_min_percentage = 3.0, 0, 0.01, 0.95
    gen = torch.Generator().manual_seed(2)
    layer = AnalogLinear(K_IN, N_OUT, bias=True, dtype=torch.bfloat16, rpu_config=cfg)
    layer.set_weights_and_biases(
        (0.02 * torch.randn(N_OUT, K_IN, generator=gen)).to(torch.bfloat16),
        torch.zeros(N_OUT, dtype=torch.bfloat16),
    )
    x = torch.randn(M_TOKENS, K_IN, generator=gen).to(torch.bfloat16)
    g = torch.randn(M_TOKENS, N_OUT, generator=gen).to(torch.bfloat16)
    return layer, x, g


def _analog_cfg(tile, noise=True, out_noise=0.04):
    from aihwkit_lightning.simulator.configs import (
        TorchInferenceRPUConfig, WeightClipType, WeightNoiseInjectionType,
    )

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = tile
    cfg.forward.inp_res = 254
    cfg.forward.out_res = 254
    cfg.forward.out_bound = 10.0
    cfg.forward.out_noise = out_noise if noise else 0.0
    cfg.clip.type = WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
    cfg.clip.sigma = 2.5
    if noise:
        cfg.modifier.noise_type = WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL
        cfg.modifier.std_dev = 0.02
    ir = cfg.pre_post.input_range
    ir.enable, ir.dynamic, ir.learn_input_range = True, False, True
    ir.init_value, ir.init_from_data, ir.decay, ir.input_min_percentage = 3.0, 0, 0.01, 0.95
    return cfg


# Workloads next to the headline one (`--workload NAME`, each prints its own line; the default
# run measures the headline workload only), same analog configuration. They exercise what the
# headline shape does not: a split whose tiles do not start on 256-column boundaries (padded tile
# layout of the operands) and a convolution (patch extraction, narrow weight gradient).
OTHER_WORKLOADS = {
    "linear_11008": "AnalogLinear 11008->4096 bf16, 8192 tokens, 22 tiles of 501/500, fwd+bwd",
    "conv2d_256": "AnalogConv2d 256->256 3x3 pad 1 bf16, 128 x 28 x 28 input, 4 tiles of 576, "
                  "fwd+bwd",
    "fwd_dynamic_4096": "AnalogLinear 4096->4096 bf16, 8192 tokens, 8 tiles x 512, dynamic per-token "
                        "per-tile input range, 8-bit DAC/ADC, out_noise 0.04, forward only",
    "mlp_3072_8192": "LLaMA-style MLP block, hidden 3072, intermediate 8192, SiLU gating, three "
                     "AnalogLinear layers, bf16, 4096 tokens, tiles of 512, learned input range, 8-bit "
                     "DAC/ADC, out_noise 0.067, fwd+bwd",
    "linear_4096_f16": "the headline layer and step in float16 (AnalogLinear 4096->4096, 8192 tokens, "
                       "8 tiles x 512, learned range, 8-bit DAC/ADC, both noises, fwd+bwd)",
    "lstm_1024": "AnalogRNN, 2 LSTM layers 1024->1024 bf16, 64 steps x 64 sequences, tiles of 512, "
                 "fwd+bwd through time",
    "lstm_1024_eval": "AnalogRNN, 2 LSTM layers 1024->1024 bf16, 64 steps x 64 sequences, tiles of "
                      "512, evaluation-mode forward replayed as one HIP graph",
}


def build_other(name):
    """(layer, x, grad_out, flops per step) of one of OTHER_WORKLOADS, on the device."""
    from aihwkit_lightning.nn import AnalogConv2d, AnalogLinear

    gen = torch.Generator().manual_seed(3)
    if name == "linear_11008":
        layer = AnalogLinear(11008, 4096, bias=True, dtype=torch.bfloat16, rpu_config=_analog_cfg(512))
        x = torch.randn(8192, 11008, generator=gen).to(torch.bfloat16)
        g = torch.randn(8192, 4096, generator=gen).to(torch.bfloat16)
        flops = 3 * 2.0 * 8192 * 11008 * 4096
    elif name == "conv2d_256":
        layer = AnalogConv2d(256, 256, 3, padding=1, bias=True, dtype=torch.bfloat16,
                             rpu_config=_analog_cfg(576))
        x = torch.randn(128, 256, 28, 28, generator=gen).to(torch.bfloat16)
        g = torch.randn(128, 256, 28, 28, generator=gen).to(torch.bfloat16)
        flops = 3 * 2.0 * (128 * 28 * 28) * (256 * 9) * 256
    elif name == "linear_4096_f16":
        layer = AnalogLinear(4096, 4096, bias=True, dtype=torch.float16, rpu_config=_analog_cfg(512))
        layer.set_weights_and_biases((0.02 * torch.randn(4096, 4096, generator=gen)).to(torch.float16),
                                     torch.zeros(4096, dtype=torch.float16))
        x = torch.randn(8192, 4096, generator=gen).to(torch.float16)
        g = torch.randn(8192, 4096, generator=gen).to(torch.float16)
        flops = 3 * 2.0 * 8192 * 4096 * 4096
    elif name == "fwd_dynamic_4096":
        cfg = _analog_cfg(512, noise=False)
        cfg.forward.out_noise = 0.04
        cfg.pre_post.input_range.dynamic = True
        layer = AnalogLinear(4096, 4096, bias=True, dtype=torch.bfloat16, rpu_config=cfg)
        x = torch.randn(8192, 4096, generator=gen).to(torch.bfloat16)
        g = None
        flops = 2.0 * 8192 * 4096 * 4096
    elif name == "mlp_3072_8192":
        class Mlp(torch.nn.Module):
            def __init__(self):
                super().__init__()
                def mk(k, n):   # learned range, 8-bit DAC/ADC, out_noise 0.067, no weight noise
                    cfg = _analog_cfg(512, noise=False)
                    cfg.forward.out_noise = 0.067
                    return AnalogLinear(k, n, bias=False, dtype=torch.bfloat16, rpu_config=cfg)

                self.gate, self.up, self.down = mk(3072, 8192), mk(3072, 8192), mk(8192, 3072)

            def forward(self, inp):
                return self.down(torch.nn.functional.silu(self.gate(inp)) * self.up(inp))

        layer = Mlp()
        for lin in (layer.gate, layer.up, layer.down):   # W ~ N(0, 0.02^2) like the other workloads
            lin.set_weights_and_biases(
                (0.02 * torch.randn(lin.out_features, lin.in_features, generator=gen)).to(torch.bfloat16), None)
        x = torch.randn(4096, 3072, generator=gen).to(torch.bfloat16)
        g = torch.randn(4096, 3072, generator=gen).to(torch.bfloat16)
        flops = 3 * 3 * 2.0 * 4096 * 3072 * 8192
    elif name in ("lstm_1024", "lstm_1024_eval"):
        from aihwkit_lightning.nn import AnalogLSTMCell, AnalogRNN

        class Outputs(torch.nn.Module):
            """The network's outputs without the states."""

            def __init__(self):
                super().__init__()
                self.net = AnalogRNN(AnalogLSTMCell, 1024, 1024, 2, dtype=torch.bfloat16,
                                     rpu_config=_analog_cfg(512, noise=name == "lstm_1024"))

            def forward(self, inp):
                return self.net(inp)[0]

        layer = Outputs()
        x = torch.randn(64, 64, 1024, generator=gen).to(torch.bfloat16)
        g = torch.randn(64, 64, 1024, generator=gen).to(torch.bfloat16)
        # two projections of 1024 -> 4096 per cell step, 64 steps, 2 layers
        flops = 2 * 64 * 2 * 2.0 * 64 * 1024 * 4096
        if name == "lstm_1024_eval":
            replay = layer.cuda().eval().net.graphed(x.cuda())
            return (lambda inp: replay(inp)[0]), x.cuda(), None, flops
        flops *= 3
    else:
        raise ValueError(name)
    with torch.no_grad():
        for param in layer.parameters():
            if param.dim() >= 2 and param.size(-1) > 16:
                param.mul_(0.02 / param.std())
    if g is None:  # forward only
        return layer.cuda().train(), x.cuda(), None, flops
    return layer.cuda().train(), x.cuda().requires_grad_(True), g.cuda(), flops


POST_TRAINING = ("post-training weight processing and calibration, fp32: 64 weight matrices "
                 "8192 x 3072 (N(0, 0.02) + 0.1 % outliers x 20, 6 tiles of 512 inputs) clipped at 3 "
                 "sigma per channel and quantised to 254 states per channel and tile; running "
                 "abs-max calibration over 256 batches of 2048 x 3072 Laplace(0, 1) activations")
# per matrix: one read for abs-max and sums, read + write for clip-and-quantise; per batch one read
POST_TRAINING_BYTES = 64 * 3 * 8192 * 3072 * 4 + 256 * 2048 * 3072 * 4


def _post_training_cfg():
    from aihwkit_lightning.simulator.configs import (TorchInferenceRPUConfig, WeightClipType,
                                                     WeightQuantizationType)
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 512
    cfg.clip.type = WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
    cfg.clip.sigma = 3.0
    cfg.modifier.quantization_type = WeightQuantizationType.DISCRETIZE_PER_CHANNEL
    cfg.modifier.res = 254
    return cfg


def time_post_training(with_cpu):
    """The reduction-bound configuration: `clip_weights` + `quantize_weights` of 64 layers through
    the layer methods, then the running abs-max of the MAX calibration over 256 activation
    batches (the kernel the calibration hook calls; 16 distinct batches, 403 MB, visited in turn).
    One timed pass over fresh matrices, wall clock around it."""
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.nn.modules.hip_utils import ops

    OPS = ops.direct(torch.empty(0, device="cuda"))   # what the calibration hook calls  # noqa: N806
    n, k, m, n_mat, n_batch = 8192, 3072, 2048, 64, 256
    gen = torch.Generator(device="cuda").manual_seed(4)

    def fresh(layer):
        with torch.no_grad():
            w = layer.weight
            w.normal_(0.0, 0.02, generator=gen)
            w.mul_(1.0 + 19.0 * (torch.rand(w.shape, device="cuda", generator=gen) < 1e-3))

    layers = [AnalogLinear(k, n, bias=False, device="cuda", rpu_config=_post_training_cfg())
              for _ in range(n_mat + 2)]
    for layer in layers:
        fresh(layer)
    lap = torch.distributions.Laplace(0.0, 1.0)
    batches = [lap.sample((m, k)).cuda() for _ in range(16)]
    in_sizes = layers[0].in_sizes
    for layer in layers[n_mat:]:  # warm-up on the two spare matrices
        layer.clip_weights()
        layer.quantize_weights()
    stat = torch.full((len(in_sizes),), float("-inf"), dtype=torch.float32, device="cuda")
    OPS.running_absmax(batches[0], in_sizes, stat)
    # sustained clocks before the timed pass (see PREHEAT_S): the calibration kernel on a scratch
    # statistic; the weight matrices stay untouched until they are timed
    scratch, turn = stat.clone(), [0]

    def heat():
        turn[0] += 1
        OPS.running_absmax(batches[turn[0] % 16], in_sizes, scratch)

    preheat(heat, PREHEAT_S / 2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for layer in layers[:n_mat]:
        layer.clip_weights()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for layer in layers[:n_mat]:
        layer.quantize_weights()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for i in range(n_batch):
        OPS.running_absmax(batches[i % 16], in_sizes, stat)
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    total = t3 - t0
    gbs = POST_TRAINING_BYTES / total / 1e9
    line = {
        "metric": "GB/s of algorithmic bytes, post-training weight processing + calibration",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": 1, "warmup": 0,
        "ms_per_step": round(total * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": POST_TRAINING, "ms": {"clip_weights x64": round((t1 - t0) * 1e3, 3),
                                                    "quantize_weights x64": round((t2 - t1) * 1e3, 3),
                                                    "running_absmax x256": round((t3 - t2) * 1e3, 3)}},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None},
    }
    if with_cpu:
        from oracle import torch_mode as om

        threads = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(threads)
        cgen = torch.Generator().manual_seed(4)
        mats = []
        for _ in range(16):
            w = 0.02 * torch.randn(n, k, generator=cgen)
            mats.append(w * (1.0 + 19.0 * (torch.rand(n, k, generator=cgen) < 1e-3)))
        cb = [lap.sample((m, k)) for _ in range(64)]
        t0 = time.perf_counter()
        for w in mats:
            om.quantize_weights(om.clip_weights(w, 3.0, True), in_sizes, "discretize_per_channel", 254.0)
        om.calibrate_max(cb, in_sizes)
        dt = (time.perf_counter() - t0) * 4.0
        line["cpu_baseline"] = {
            "value": POST_TRAINING_BYTES / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"16 of 64 matrices and 64 of 256 batches, time scaled by 4 ({dt:.1f} s for the "
                      "whole configuration)"}
    return line


# An idle MI355X runs the first tens of milliseconds of a burst of work below its sustained
# clocks: 20 steps timed right after 5 warm-up steps read 8-10 % longer than the same 20 steps
# after a few hundred (measured: 1.085 ms per step from idle, 0.990 ms from 100 steps on, flat up
# to 10 000 steps). Every timed region here therefore follows PREHEAT_S seconds of the very work
# it times, untimed; the headline line also carries the figure without it (`ms_per_step_cold_start`).
PREHEAT_S = 0.5


def preheat(fn, seconds=PREHEAT_S):
    """Run fn() back to back for `seconds` of wall clock, untimed (see PREHEAT_S); returns the
    number of calls made."""
    t0 = time.perf_counter()
    calls = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        calls += 10
        torch.cuda.synchronize()
    return calls


def time_other(name, steps, warmup, graph=False):
    """ms per fwd+bwd step and TFLOP/s of one of OTHER_WORKLOADS (wall clock around K steps)."""
    layer, x, g, flops = build_other(name)

    def step():
        if g is None:
            with torch.no_grad():
                layer(x)
            return
        x.grad = None
        layer.zero_grad(set_to_none=True)
        layer(x).backward(g)

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    preheat(step, PREHEAT_S / 2)
    ms = timed(step)
    res = {"workload": OTHER_WORKLOADS[name], "ms_per_step": round(ms, 4),
           "tflops": round(flops / (ms * 1e-3) / 1e12, 2)}
    if graph and g is not None:
        # the same step recorded into one HIP graph and replayed (no host between the launches)
        from aihwkit_lightning.nn.graphs import CapturedStep
        replay = CapturedStep(step)
        replay()
        preheat(replay, PREHEAT_S / 2)
        ms_graph = timed(replay)
        res["ms_per_step_graph_replay"] = round(ms_graph, 4)
        res["tflops_graph_replay"] = round(flops / (ms_graph * 1e-3) / 1e12, 2)
    return res


def time_reference_speed_test():
    """The workload of the reference's own speed script (its tests/test_speed.py:221-279): float16,
    512 rows, square layers of 128 ... 2048 inputs as one tile, input range + DAC, ADC (bound 12),
    output noise 0.02, additive weight noise, layer-wise clipping at 2 sigma; one step = forward,
    `out.sum().backward()`, `AnalogOptimizer(AdamW, lr=0).step()` (which clips the weights).
    Microseconds per step, eager and replayed from one HIP graph."""
    from aihwkit_lightning.nn import AnalogLinear
    from aihwkit_lightning.nn.graphs import CapturedStep
    from aihwkit_lightning.optim import AnalogOptimizer
    from aihwkit_lightning.simulator.configs import (
        TorchInferenceRPUConfig, WeightClipType, WeightNoiseInjectionType,
    )

    out = {}
    for size in (128, 256, 512, 1024, 2048):
        cfg = TorchInferenceRPUConfig()
        cfg.mapping.max_input_size = -1
        cfg.forward.inp_res, cfg.forward.out_res, cfg.forward.out_bound = 254, 254, 12
        cfg.forward.out_noise = 0.02
        ir = cfg.pre_post.input_range
        ir.enable, ir.learn_input_range, ir.init_from_data = True, True, 0
        cfg.clip.type, cfg.clip.sigma = WeightClipType.LAYER_GAUSSIAN, 2.0
        cfg.modifier.noise_type, cfg.modifier.std_dev = WeightNoiseInjectionType.ADD_NORMAL, 0.01
        layer = AnalogLinear(size, size, bias=True, rpu_config=cfg).to(device="cuda", dtype=torch.float16)
        optims = {"eager": AnalogOptimizer(torch.optim.AdamW, layer.analog_layers, layer.parameters(), lr=0.0),
                  # torch's optimizers record into a graph only in their capturable form
                  "graph": AnalogOptimizer(torch.optim.AdamW, layer.analog_layers, layer.parameters(), lr=0.0,
                                           capturable=True)}
        inp = torch.randn(512, size, device="cuda", dtype=torch.float16, requires_grad=True)
        which = ["eager"]

        def step():
            layer(inp).sum().backward()
            optims[which[0]].step()

        def timed(fn, reps=300):
            preheat(fn, 0.2)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / reps * 1e6

        eager = timed(step)
        which[0] = "graph"
        replay = CapturedStep(step)
        replay()
        # the same eager step with torch's own Linear and optimizer: what the host side of any
        # eager step costs on this box (autograd, AdamW's launches), with no analog work at all
        plain = torch.nn.Linear(size, size).to(device="cuda", dtype=torch.float16)
        plain_opt = torch.optim.AdamW(plain.parameters(), lr=0.0)

        def plain_step():
            plain(inp).sum().backward()
            plain_opt.step()

        out[str(size)] = {"us_eager": round(eager, 1), "us_graph_replay": round(timed(replay), 1),
                          "us_eager_torch_linear": round(timed(plain_step), 1)}
    return out


def event_time_ms(fn, reps):
    """Average duration of fn() over `reps` back-to-back calls, HIP events on the current stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    preheat(fn, 0.03)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def mfma_kernel_times(x, g, weight, bias, ir, in_sizes, dynamic, out_noise, weight_noise, reps):
    """ms per launch of the three MFMA kernels of one layer call (and of the two passes in front of
    them), through the same custom ops the layer uses, plus torch.matmul (the vendor library) on the
    same three products with the same operands -- what a plain product of each shape takes on this
    box, with none of the analog work. ``g`` None: forward only."""
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    noise_type = L.AHL_NOISE_ADD_NORMAL_PER_CHANNEL if weight_noise else L.AHL_NOISE_NONE
    prep = lambda: OPS.weight_prep(weight, in_sizes, L.AHL_QUANT_NONE, noise_type, 1.0, weight_noise,   # noqa: E731
                                   11, 1, True)
    wmax, tile_max, _, w_eff = prep()
    w_eff = weight if w_eff is None else w_eff
    icfg = [L.AHL_IR_DYNAMIC if dynamic else L.AHL_IR_STATIC, 0, 1, 1, 0, 12345, 0]
    fcfg = [254.0, 254.0, 10.0, out_noise, 0.01, 0.95]
    xq, ir_rows = OPS.dac(x, ir, in_sizes, icfg, fcfg)
    ir_used = ir_rows if dynamic else ir
    fwd = lambda: OPS.linear_fwd(None, xq, w_eff, bias, ir_used, wmax, tile_max, in_sizes, icfg, fcfg,   # noqa: E731
                                 g is not None)
    _, keep, flag = fwd()
    out = {"linear_fwd": event_time_ms(fwd, reps)}
    if g is not None:
        out["linear_bwd_dx(+ir_grad)"] = event_time_ms(
            lambda: OPS.linear_bwd_dx(g, keep, flag, w_eff, x, ir_used, in_sizes, icfg, fcfg), reps)
        out["linear_bwd_dw(+bias_grad)"] = event_time_ms(
            lambda: OPS.linear_bwd_dw(g, keep, flag, None, xq, ir_used, in_sizes, icfg, fcfg, bias is not None), reps)
    out["dac"] = event_time_ms(lambda: OPS.dac(x, ir, in_sizes, icfg, fcfg), reps)
    out["weight_prep"] = event_time_ms(prep, reps)
    vendor = {"fwd": event_time_ms(lambda: torch.matmul(xq, w_eff.t()), reps)}
    if g is not None:
        vendor["dx"] = event_time_ms(lambda: torch.matmul(g, w_eff), reps)
        vendor["dw"] = event_time_ms(lambda: torch.matmul(g.t(), xq), reps)
    return out, vendor


MFMA_KERNELS = ("linear_fwd", "linear_bwd_dx(+ir_grad)", "linear_bwd_dw(+bias_grad)")


def mfma_roofline(times, flops):
    """The roofline object of the slowest MFMA kernel among ``times`` ({name: ms per launch})."""
    dom = max((k for k in times if k.split(":")[-1] in MFMA_KERNELS), key=lambda k: times[k])
    achieved = flops[dom] / (times[dom] * 1e-3) / 1e12
    return {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "ms_per_launch": {k: round(v, 4) for k, v in times.items()}}


def kernel_rooflines(layer, x, g, reps):
    """Per-kernel timings of the headline layer, the vendor library's plain products beside them."""
    times, vendor = mfma_kernel_times(x, g, layer.weight.data, layer.bias.data, layer.input_range.detach(),
                                      layer.in_sizes, False, 0.04, 0.02, reps)
    # a plain device copy of known size (256 MiB read + 256 MiB written): the yardstick that
    # HBM byte counters of a profiler run of this command are scaled by
    src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=x.device)
    dst = torch.empty_like(src)
    times["copy_256MiB"] = event_time_ms(lambda: dst.copy_(src), reps)
    return times, vendor, 2.0 * M_TOKENS * K_IN * N_OUT


def other_config_roofline(name, reps=10):
    """The roofline of the slowest MFMA kernel of the dynamic-range forward / the MLP block."""
    gen = torch.Generator().manual_seed(3)
    bf = torch.bfloat16
    if name == "fwd_dynamic_4096":
        x = torch.randn(8192, 4096, generator=gen).to(bf).cuda()
        w = (0.02 * torch.randn(4096, 4096, generator=gen)).to(bf).cuda()
        times, vendor = mfma_kernel_times(x, None, w, torch.zeros(4096, dtype=bf, device="cuda"), None,
                                          [512] * 8, True, 0.04, 0.0, reps)
        roof = mfma_roofline(times, {"linear_fwd": 2.0 * 8192 * 4096 * 4096})
        roof["vendor_plain_ms"] = {k: round(v, 4) for k, v in vendor.items()}
        return roof
    assert name == "mlp_3072_8192"
    times, flops, vendors = {}, {}, {}
    for proj, k, n in (("gate/up", 3072, 8192), ("down", 8192, 3072)):
        x = torch.randn(4096, k, generator=gen).to(bf).cuda()
        g = torch.randn(4096, n, generator=gen).to(bf).cuda()
        w = (0.02 * torch.randn(n, k, generator=gen)).to(bf).cuda()
        ir = torch.full((k // 512,), 3.0, dtype=bf, device="cuda")
        t, vendor = mfma_kernel_times(x, g, w, None, ir, [512] * (k // 512), False, 0.067, 0.0, reps)
        for key, val in t.items():
            times[f"{proj}:{key}"] = val
            flops[f"{proj}:{key}"] = 2.0 * 4096 * k * n
        vendors[proj] = {key: round(val, 4) for key, val in vendor.items()}
        del x, g, w
    roof = mfma_roofline(times, flops)
    roof["vendor_plain_ms"] = vendors
    return roof


PEAK_HBM_GBS = 8000.0  # MI355X HBM3E


def hbm_kernel_rooflines(reps):
    """The memory-bound kernels of the path at the shapes of the clip / quantise / calibrate
    configuration: one 8192 x 3072 fp32 weight matrix (6 tiles of 512 inputs), activation batches
    of 2048 x 3072 fp32. GB/s = algorithmic bytes (each element read once, written where the
    operation writes) / launch time; fraction of the 8 TB/s HBM peak."""
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS
    from aihwkit_lightning.nn.modules.hip_utils import library as L

    gen = torch.Generator().manual_seed(4)
    n, k, m = 8192, 3072, 2048
    in_sizes = [512] * 6
    # 4 weight matrices (403 MB) and 16 activation batches (403 MB), visited in turn, so that
    # consecutive launches do not find their input in the 256 MB Infinity Cache
    w0 = (0.02 * torch.randn(n, k, generator=gen)).cuda()
    ws = [w0] + [w0.clone() for _ in range(3)]
    x0 = torch.randn(m, k, generator=gen).cuda()
    xs = [x0] + [x0.clone() for _ in range(15)]
    xbs = [x0.to(torch.bfloat16).repeat(4, 1) for _ in range(8)]  # 8192 x 3072 bf16 (50 MB each)
    cache = torch.zeros(6, dtype=torch.float32, device="cuda")
    irb = torch.full((6,), 3.0, device="cuda", dtype=torch.bfloat16)
    wb, xbytes = n * k * 4, m * k * 4
    icfg = [L.AHL_IR_STATIC, 0, 1, 0, 0, 0, 0]
    fcfg = [254.0, 254.0, 10.0, 0.0, 0.0, 0.95]
    geom = [64, 256, 1, 28, 28, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1]
    img0 = torch.randn(64, 256, 28, 28, generator=gen).to(torch.bfloat16).cuda()
    imgs = [img0] + [img0.clone() for _ in range(15)]
    patches = [OPS.im2col(img0, geom) for _ in range(2)]
    img_bytes, patch_bytes = img0.numel() * 2, patches[0].numel() * 2
    turn = [0]

    def nxt(lst):
        turn[0] += 1
        return lst[turn[0] % len(lst)]

    cases = {
        "sliced_absmax(W)": (lambda: OPS.sliced_absmax(nxt(ws), in_sizes, True), wb),
        "sliced_std(x)": (lambda: OPS.sliced_std(nxt(xs), in_sizes), xbytes),
        "running_absmax(x)": (lambda: OPS.running_absmax(nxt(xs), in_sizes, cache), xbytes),
        # sums and clamp from one read of W (a row stays in registers); writes only changed vectors
        "clip_weights(W, per channel)": (lambda: OPS.clip_weights(nxt(ws), 3.0, L.AHL_CLIP_PER_CHANNEL), wb),
        # abs-max and quantisation from one read, one write
        "quantize_weights(W)": (lambda: OPS.quantize_weights(
            nxt(ws), in_sizes, L.AHL_QUANT_DISCRETIZE_PER_CHANNEL, 254.0), 2 * wb),
        "dac(x bf16 8192x3072)": (lambda: OPS.dac(nxt(xbs), irb, in_sizes, icfg, fcfg),
                                  2 * xbs[0].numel() * 2),
        # calibration statistics: row filter + sums (2 reads); row filter + 4 digit histograms of
        # the radix selection (5 reads)
        "sliced_std_kept(x)": (lambda: OPS.sliced_std_kept(nxt(xs), in_sizes), 2 * xbytes),
        "sliced_quantile(x, 0.99995)": (lambda: OPS.sliced_quantile(nxt(xs), in_sizes, 0.99995),
                                        5 * xbytes),
        # patch extraction and fold of a 3x3 convolution, 64 x 256 x 28 x 28 bf16 (231 MB of patches)
        "im2col(3x3, 256 ch)": (lambda: OPS.im2col(nxt(imgs), geom), patch_bytes + img_bytes),
        "col2im(3x3, 256 ch)": (lambda: OPS.col2im(nxt(patches), geom), patch_bytes + img_bytes),
    }
    out = {}
    for name, (fn, nbytes) in cases.items():
        t = event_time_ms(fn, reps)
        gbs = nbytes / (t * 1e-3) / 1e9
        out[name] = {"us": round(t * 1e3, 1), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 3)}
    return out


def cpu_baseline(sample_tokens=M_TOKENS):
    """The torch-mode oracle (CPU restatement of the reference) on the host cores: the whole
    workload by default (about 7 s per forward + backward pass on 16 cores)."""
    from oracle import torch_mode as om

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    gen = torch.Generator().manual_seed(2)
    w = (0.02 * torch.randn(N_OUT, K_IN, generator=gen)).to(torch.bfloat16)
    x = torch.randn(sample_tokens, K_IN, generator=gen).to(torch.bfloat16)
    g = torch.randn(sample_tokens, N_OUT, generator=gen).to(torch.bfloat16)
    b = torch.zeros(N_OUT, dtype=torch.bfloat16)
    cfg = om.OracleCfg(max_input_size=TILE, inp_res=254, out_res=254, out_bound=10.0, out_noise=0.04,
                       bound_per_channel=True, ir_mode=om.IR_STATIC, ir_decay=0.01,
                       weight_noise=om.ADD_NORMAL_PER_CHANNEL, modifier_std=0.02)
    ir = torch.full((K_IN // TILE,), 3.0, dtype=torch.bfloat16)
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        out, saved = om.linear_forward(x, w, b, cfg, ir, True)
        om.linear_backward(g, saved)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    flops = 3 * 2.0 * sample_tokens * K_IN * N_OUT
    return {
        "value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{sample_tokens} of {M_TOKENS} tokens, same layer, fwd+bwd, best of 2 "
                  f"({best:.2f} s)",
    }


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--graph", action="store_true",
                        help="report the step replayed from one HIP graph instead of the eager step")
    parser.add_argument("--no-others", action="store_true",
                        help="headline workload only: skip the other configurations' short runs")
    parser.add_argument("--kernels-only", action="store_true",
                        help="only launch the individual kernels (for rocprofv3 runs)")
    parser.add_argument("--workload", default="linear", choices=["linear", "post_training", "reference_speed_test", *OTHER_WORKLOADS],
                        help="'linear' is the headline workload; the others print their own line")
    ns = parser.parse_args()
    if ns.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)

    if ns.workload == "reference_speed_test":
        res = time_reference_speed_test()
        print(json.dumps({
            "metric": "microseconds per forward + backward + optimizer step", "value": res["2048"]["us_eager"],
            "unit": "us", "n_gpus": 1, "steps": 300, "warmup": 0, "ms_per_step": res["2048"]["us_eager"] / 1e3,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "the reference's tests/test_speed.py fwd+bwd+step benchmark: float16, 512 rows, "
                                   "square AnalogLinear of 128 ... 2048 (value: 2048), all non-idealities on",
                       "us_per_step": res}}))
        return
    if ns.workload == "post_training":
        print(json.dumps(time_post_training(not ns.no_cpu)))
        return
    if ns.workload != "linear":
        torch.manual_seed(0)
        res = time_other(ns.workload, ns.steps, ns.warmup, ns.graph)
        print(json.dumps({
            "metric": "TFLOP/s of the workload's matrix products", "value": res["tflops"], "unit": "TFLOP/s", "n_gpus": 1,
            "steps": ns.steps, "warmup": ns.warmup, "ms_per_step": res["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f16" if ns.workload.endswith("_f16") else "bf16",
            "data": "synthetic", "config": {k: v for k, v in res.items() if k not in ("ms_per_step", "tflops")},
        }))
        return

    layer, x, g = build_layer()
    layer = layer.cuda().train()
    x = x.cuda().requires_grad_(True)
    g = g.cuda()
    torch.manual_seed(0)

    def step():
        x.grad = None
        layer.zero_grad(set_to_none=True)
        out = layer(x)
        out.backward(g)

    if ns.kernels_only:
        kernels, vendor, _ = kernel_rooflines(layer, x.detach(), g, max(ns.steps, 1))
        print(json.dumps({"ms_per_launch": kernels, "vendor_plain_ms": vendor}))
        return

    def timed(fn):
        for _ in range(ns.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(ns.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / ns.steps * 1e3

    # The eager step (Python between the launches) is the headline; next to it the same step
    # recorded once into a HIP graph and replayed (every replay draws new noise from the
    # device-resident Philox state). At this size the GPU is never waiting for the host, so the
    # two agree.
    from aihwkit_lightning.nn.graphs import CapturedStep
    ms_cold = timed(step)            # W + K steps on a GPU that was idle until now
    preheat_steps = preheat(step)
    ms_eager = timed(step)           # the same W + K steps at sustained clocks: the headline
    replay = CapturedStep(step)
    replay()                         # the recording itself (the GPU idles meanwhile)
    preheat(replay, PREHEAT_S / 2)
    ms_graph = timed(replay)
    ms_per_step = ms_graph if ns.graph else ms_eager
    step_flops = 3 * 2.0 * M_TOKENS * K_IN * N_OUT
    value = step_flops / (ms_per_step * 1e-3) / 1e12

    kernels, vendor, gemm_flops = kernel_rooflines(layer, x.detach(), g, max(ns.steps, 5))
    dom = max(MFMA_KERNELS, key=lambda k: kernels[k])
    achieved = gemm_flops / (kernels[dom] * 1e-3) / 1e12
    result = {
        "metric": "AnalogLinear fwd+bwd TFLOP/s (4096^2, 8192 tok, bf16) + % MFMA peak",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": ns.steps,
        "warmup": ns.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "AnalogLinear 4096->4096 bf16, 8192 tokens, 8 tiles x 512, learned input "
                        "range (decay 0.01), 8-bit DAC/ADC, out_noise 0.04, weight noise 0.02 per "
                        "channel, fwd+bwd",
            "frac_of_bf16_mfma_peak": round(value / PEAK_BF16_TFLOPS, 4),
            "step": "forward + backward replayed from one HIP graph" if ns.graph else "eager",
            "ms_per_step_eager": round(ms_eager, 4), "ms_per_step_graph_replay": round(ms_graph, 4),
            # timed regions follow PREHEAT_S seconds of the same work, untimed, so that they run at
            # sustained clocks; the same W + K steps on the GPU as the process found it (idle):
            "preheat_s": PREHEAT_S, "preheat_steps": preheat_steps,
            "ms_per_step_cold_start": round(ms_cold, 4),
            # torch.matmul (the vendor library) on the three products of this step, same operands:
            # what the plain products alone take on this box, no analog work (bench-only yardstick)
            "vendor_plain_ms": {k: round(v, 4) for k, v in vendor.items()},
        },
        "roofline": {
            "bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": measured_traffic_bytes(dom),
            "traffic_source": TRAFFIC_TABLE + " (rocprofv3 FETCH_SIZE and WRITE_SIZE runs of "
                              "`bench.py --kernels-only`, not this run)",
            "ms_per_launch": {k: round(v, 4) for k, v in kernels.items()},
        },
    }
    result["hbm_kernels"] = hbm_kernel_rooflines(max(ns.steps, 5))
    if not ns.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    # The other configurations of the benchmark set, a few steps each, after the headline's
    # timed region: the dynamic-range forward, the MLP block, the reduction-bound post-training
    # pass (with its own CPU baseline). `--workload NAME` prints each as a line of its own.
    if ns.no_others:
        print(json.dumps(result))
        return
    del layer, x, g
    torch.cuda.empty_cache()
    others = {}
    for name in ("fwd_dynamic_4096", "mlp_3072_8192", "linear_4096_f16", "linear_11008", "conv2d_256",
                 "lstm_1024"):
        res = time_other(name, 10, 3, graph=True) if name != "lstm_1024" else time_other(name, 4, 2, graph=True)
        res["frac_of_bf16_mfma_peak"] = round(res["tflops"] / PEAK_BF16_TFLOPS, 4)
        if name in ("fwd_dynamic_4096", "mlp_3072_8192"):
            torch.cuda.empty_cache()
            res["roofline"] = other_config_roofline(name)
        others[name] = res
        torch.cuda.empty_cache()
    post = time_post_training(not ns.no_cpu)
    others["post_training"] = {
        "workload": post["config"]["workload"], "ms": post["ms_per_step"], "parts_ms": post["config"]["ms"],
        "GB/s": post["value"], "frac_hbm": post["roofline"]["frac"],
        "cpu_baseline": post.get("cpu_baseline"),
    }
    # the workload of the reference's own speed script (float16, small layers, optimizer step)
    others["reference_speed_test"] = {
        "workload": "the reference's tests/test_speed.py fwd+bwd+step benchmark: float16, 512 rows, square "
                    "AnalogLinear of 128 ... 2048, all non-idealities on",
        "us_per_step": time_reference_speed_test(),
    }
    result["other_configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
