"""Host-side mirror of the reference API (no GPU): constructor, parameter / buffer names, shapes
and dtypes, tile split rule, state-dict metadata, layer iteration, optimizer wiring, conversion
from and to ``nn.Linear`` (reference ``nn/modules/linear.py``, ``nn/modules/base.py``,
``optim/analog_optimizer.py``)."""
import pytest
import torch

from aihwkit_lightning.nn import AnalogLinear
from aihwkit_lightning.nn.modules.container import AnalogSequential, AnalogWrapper
from aihwkit_lightning.nn.modules.linear import get_split_sizes
from aihwkit_lightning.optim import AnalogOptimizer
from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig, WeightClipType


def _cfg(max_input_size=128, ir=True, dynamic=False, clip=WeightClipType.NONE):
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = max_input_size
    cfg.pre_post.input_range.enable = ir
    cfg.pre_post.input_range.dynamic = dynamic
    cfg.clip.type = clip
    return cfg


@pytest.mark.parametrize("size,max_size,want", [
    (257, 128, [86, 86, 85]),      # nn/modules/linear.py:165-170: base + 1 for the first `extra`
    (512, 256, [256, 256]),
    (10, -1, [10]),
    (10, 0, [10]),
    (7, 16, [7]),
    (4096, 512, [512] * 8),
])
def test_tile_split_rule(size, max_size, want):
    assert get_split_sizes(size, max_size) == want
    assert sum(get_split_sizes(size, max_size)) == size


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_parameters_and_buffers_of_a_learned_range_layer(dtype):
    layer = AnalogLinear(257, 12, bias=True, dtype=dtype, rpu_config=_cfg())
    n_tiles = 3
    assert layer.in_sizes == [86, 86, 85]
    assert layer.upper_end_of_slices.tolist() == [86, 172, 257]
    assert layer.upper_end_of_slices.dtype == torch.int32
    assert isinstance(layer.input_range, torch.nn.Parameter) and layer.input_range.requires_grad
    assert layer.input_range.shape == (n_tiles,) and layer.input_range.dtype == dtype
    assert torch.all(layer.input_range == 3.0)                      # init_value default
    for name, val in (("input_range_update_idx", 0.0), ("x_min", -1e-5), ("x_max", 1e-5)):
        buf = getattr(layer, name)
        assert buf.shape == (n_tiles,) and buf.dtype == dtype
        assert torch.allclose(buf.float(), torch.full((n_tiles,), val), atol=1e-7)
    names = {n for n, _ in layer.named_parameters()}
    assert names == {"weight", "bias", "input_range"}
    assert {n for n, _ in layer.named_buffers()} == {"input_range_update_idx", "x_min", "x_max"}
    assert layer.learnable_weight_clip is None


def test_dynamic_or_disabled_range_has_no_range_state():
    for cfg in (_cfg(dynamic=True), _cfg(ir=False)):
        layer = AnalogLinear(64, 8, rpu_config=cfg)
        assert layer.input_range is None and layer.input_range_update_idx is None
        assert layer.x_min is None and layer.x_max is None


def test_learnable_clip_starts_at_the_per_tile_channel_abs_max():
    layer = AnalogLinear(20, 6, rpu_config=_cfg(max_input_size=10, clip=WeightClipType.LEARNABLE_PER_CHANNEL))
    clip = layer.learnable_weight_clip
    assert isinstance(clip, torch.nn.Parameter) and clip.shape == (2, 6)
    want = torch.stack([layer.weight[:, :10].abs().amax(1), layer.weight[:, 10:].abs().amax(1)])
    assert torch.equal(clip.data, want)


def test_state_dict_round_trip_carries_the_config():
    cfg = _cfg(max_input_size=16)
    cfg.forward.out_noise = 0.123
    src = AnalogLinear(32, 4, rpu_config=cfg)
    src.input_range.data.fill_(1.5)
    state = src.state_dict()
    assert set(state.keys()) == {"weight", "bias", "input_range", "input_range_update_idx", "x_min", "x_max"}
    dst = AnalogLinear(32, 4, rpu_config=_cfg(max_input_size=16))
    dst.load_state_dict(state)
    assert torch.equal(dst.input_range.data, src.input_range.data)
    assert dst.rpu_config.forward.out_noise == 0.123   # restored from the state-dict metadata
    assert dst.rpu_config is not src.rpu_config


def test_conversion_from_and_to_digital():
    lin = torch.nn.Linear(24, 5)
    analog = AnalogLinear.from_digital(lin, _cfg(max_input_size=8))
    assert torch.equal(analog.weight.data, lin.weight.data) and torch.equal(analog.bias.data, lin.bias.data)
    assert analog.in_sizes == [8, 8, 8]
    back = AnalogLinear.to_digital(analog)
    assert type(back) is torch.nn.Linear and torch.equal(back.weight.data, lin.weight.data)
    w, b = analog.get_weights_and_biases()
    assert torch.equal(w, lin.weight.data) and torch.equal(b, lin.bias.data)
    analog.set_weights_and_biases(torch.ones(5, 24), torch.zeros(5))
    assert float(analog.weight.detach().sum()) == 120.0 and float(analog.bias.detach().abs().sum()) == 0.0


def test_layer_iteration_skips_containers():
    a, b = AnalogLinear(8, 8, rpu_config=_cfg()), AnalogLinear(8, 4, rpu_config=_cfg())
    seq = AnalogSequential(a, torch.nn.ReLU(), b)
    assert list(seq.analog_layers()) == [a, b]
    assert [n for n, _ in seq.named_analog_layers()] == ["0", "2"]
    wrapped = AnalogWrapper(torch.nn.Sequential(a, b))
    assert list(wrapped.analog_layers()) == [a, b]
    assert isinstance(wrapped, torch.nn.Sequential)


def test_analog_optimizer_clips_after_every_step():
    calls = []

    class Probe(AnalogLinear):
        def clip_weights(self):            # the device call is not under test here
            calls.append(self)

    layer = Probe(8, 4, rpu_config=_cfg())
    opt = AnalogOptimizer(torch.optim.SGD, layer.analog_layers, layer.parameters(), lr=0.1)
    assert isinstance(opt, torch.optim.SGD) and isinstance(opt, AnalogOptimizer)
    layer.weight.grad = torch.ones_like(layer.weight)
    before = layer.weight.detach().clone()
    opt.step()
    assert calls == [layer]
    assert torch.allclose(layer.weight.detach(), before - 0.1)
    opt.step()
    assert len(calls) == 2
