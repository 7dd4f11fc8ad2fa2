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


# ------------------------------------------------------------------ convolutions and conversion
def test_conv_layers_tile_the_patch_dimension():
    """nn/modules/conv.py:167-189: in_features = C * prod(kernel), split like a linear layer;
    a 1-d layer stores a height-one 2-d kernel but saves the nn.Conv1d shape."""
    from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d, AnalogConv3d

    cfg = _cfg(max_input_size=10)
    c1 = AnalogConv1d(3, 4, 3, padding=1, rpu_config=cfg)
    assert c1.weight.shape == (4, 3, 1, 3) and c1.in_features == 9 and c1.in_sizes == [9]
    assert c1.state_dict()["weight"].shape == (4, 3, 3)
    assert c1.kernel_size == (1, 3) and c1.padding == (0, 1)
    c2 = AnalogConv2d(3, 5, (3, 2), stride=2, rpu_config=cfg)
    assert c2.in_features == 18 and c2.in_sizes == [9, 9] and c2.input_range.shape == (2,)
    assert c2.upper_end_of_slices.tolist() == [9, 18]
    c3 = AnalogConv3d(2, 5, (2, 3, 3), rpu_config=cfg)
    assert c3.in_features == 36 and c3.in_sizes == [9, 9, 9, 9] and c3.out_features == 5
    assert c2.geometry((2, 3, 9, 8)) == [2, 3, 1, 9, 8, 1, 3, 2, 1, 2, 2, 0, 0, 0, 1, 1, 1]
    with pytest.raises(ValueError):
        c2.geometry((2, 4, 9, 8))


def test_conv_layers_reject_what_the_reference_rejects():
    from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d, AnalogConv3d

    cfg = _cfg()
    with pytest.raises(ValueError):
        AnalogConv2d(4, 4, 3, groups=2, rpu_config=cfg)
    with pytest.raises(ValueError):
        AnalogConv2d(4, 4, 3, padding_mode="reflect", rpu_config=cfg)
    with pytest.raises(ValueError):
        AnalogConv1d(4, 4, 3, dilation=2, rpu_config=cfg)
    with pytest.raises(AssertionError):
        AnalogConv3d(4, 4, 3, dilation=2, rpu_config=cfg)
    with pytest.raises(AssertionError):
        AnalogConv2d(4, 4, 3)


def test_conv_output_size_in_the_library():
    """ahl_conv_out_size is host arithmetic: it runs without a GPU."""
    from aihwkit_lightning.exceptions import HipBackendError
    from aihwkit_lightning.nn.modules.hip_utils.ops import conv_out_size

    geom = [2, 3, 5, 9, 8, 2, 3, 3, 1, 2, 1, 1, 1, 0, 1, 1, 2]
    want = [(5 + 2 - 1 - 1) // 1 + 1, (9 + 2 - 2 - 1) // 2 + 1, (8 - 4 - 1) // 1 + 1]
    assert conv_out_size(geom) == want
    with pytest.raises(HipBackendError):  # kernel larger than the padded input
        conv_out_size([1, 1, 1, 2, 2, 1, 3, 3, 1, 1, 1, 0, 0, 0, 1, 1, 1])


class _Net(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = torch.nn.Conv1d(3, 3, 3, padding=1)
        self.conv2 = torch.nn.Conv2d(3, 10, 3)
        self.seq = torch.nn.Sequential(torch.nn.Linear(4, 5), torch.nn.ReLU(), torch.nn.Linear(5, 2))
        self.rnn = torch.nn.GRU(4, 4)


def test_convert_to_analog_and_back():
    """tests/test_conversion.py of the reference: default map, empty map, in place, exclusion,
    per-layer config hook, round trip of the weights."""
    from aihwkit_lightning.exceptions import ArgumentError
    from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d
    from aihwkit_lightning.nn.conversion import convert_to_analog, convert_to_digital

    model = _Net()
    analog = convert_to_analog(model, _cfg())
    assert isinstance(analog, AnalogWrapper)
    assert isinstance(analog.conv1, AnalogConv1d) and isinstance(analog.conv2, AnalogConv2d)
    assert isinstance(analog.seq, AnalogSequential) and isinstance(analog.seq[0], AnalogLinear)
    assert isinstance(analog.rnn, _rnn_classes()[0])
    assert isinstance(model.conv1, torch.nn.Conv1d), "without inplace the model is copied"
    assert len(list(analog.analog_layers())) == 6
    assert analog.conv1.rpu_config is not analog.conv2.rpu_config

    untouched = convert_to_analog(model, _cfg(), conversion_map={})
    assert isinstance(untouched.conv1, torch.nn.Conv1d) and isinstance(untouched, AnalogWrapper)
    partial = convert_to_analog(model, _cfg(), exclude_modules=["seq.0", "conv2"])
    assert isinstance(partial.conv2, torch.nn.Conv2d) and isinstance(partial.seq[0], torch.nn.Linear)
    assert isinstance(partial.seq[2], AnalogLinear)

    def per_layer(name, _module, config):
        config.mapping.max_input_size = 2 if name == "seq.2" else 3
        return config

    tuned = convert_to_analog(model, _cfg(), specific_rpu_config_fun=per_layer)
    assert tuned.seq[2].in_sizes == [2, 2, 1] and tuned.seq[0].in_sizes == [2, 2]

    in_place = _Net()
    convert_to_analog(in_place, _cfg(), inplace=True)
    assert isinstance(in_place.conv1, AnalogConv1d) and isinstance(in_place.seq[2], AnalogLinear)

    digital = convert_to_digital(analog)
    assert type(digital) is _Net and isinstance(digital.conv1, torch.nn.Conv1d)
    assert isinstance(digital.seq, torch.nn.Sequential) and isinstance(digital.seq[0], torch.nn.Linear)
    for name, param in model.state_dict().items():
        assert torch.equal(param, digital.state_dict()[name]), name
    with pytest.raises(ArgumentError):
        convert_to_analog(model, _cfg(), conversion_map=[])
    with pytest.raises(ArgumentError):
        convert_to_digital(analog, conversion_set=[])


def test_tile_stride_rule():
    """Host arithmetic of the library: aligned splits stay dense, others get a stride that is a
    multiple of 256 and holds the widest tile; fp32 has no padded layout."""
    from aihwkit_lightning.nn.modules.hip_utils.ops import tile_stride

    assert tile_stride(4096, 8, torch.bfloat16) == 0
    assert tile_stride(11008, 22, torch.bfloat16) == 512      # tiles of 501 / 500
    assert tile_stride(2304, 4, torch.bfloat16) == 768        # tiles of 576
    assert tile_stride(768, 2, torch.bfloat16) == 512         # tiles of 384
    assert tile_stride(1003, 4, torch.bfloat16) == 256
    assert tile_stride(11008, 22, torch.float32) == 0


# ---------------------------------------------------------------------------- recurrent layers
def _rnn_classes():
    from aihwkit_lightning.nn import (AnalogGRUCell, AnalogLSTMCell, AnalogLSTMCellCombinedWeight,
                                      AnalogRNN, AnalogVanillaRNNCell)
    return AnalogRNN, AnalogVanillaRNNCell, AnalogLSTMCell, AnalogGRUCell, AnalogLSTMCellCombinedWeight


def test_rnn_module_tree_and_projection_shapes():
    """reference nn/modules/rnn/rnn.py:169-214, cells.py: the tree is
    rnn.layers[i](.directions[d]).cell.weight_ih / weight_hh with gate_count * hidden rows."""
    AnalogRNN, Vanilla, Lstm, Gru, Combined = _rnn_classes()
    for cell, gates in ((Vanilla, 1), (Lstm, 4), (Gru, 3)):
        net = AnalogRNN(cell, 10, 20, num_layers=2, bidir=True, rpu_config=_cfg(max_input_size=16))
        first = net.rnn.layers[0].directions[1].cell
        second = net.rnn.layers[1].directions[0].cell
        assert isinstance(first, cell)
        assert first.weight_ih.weight.shape == (gates * 20, 10)
        assert first.weight_hh.weight.shape == (gates * 20, 20)
        assert second.weight_ih.weight.shape == (gates * 20, 40)
        assert first.weight_hh.in_sizes == [10, 10]
        assert len(list(net.analog_layers())) == 8
        # torch's initialisation range
        assert float(first.weight_ih.weight.detach().abs().max()) <= 1 / 20 ** 0.5
    net = AnalogRNN(Combined, 10, 20, rpu_config=_cfg())
    assert net.rnn.layers[0].cell.weight.weight.shape == (80, 30)
    state = net.get_zero_state(3)[0]
    assert state.hx.shape == (3, 20) and state.cx.shape == (3, 20)
    assert AnalogRNN(Gru, 4, 5, rpu_config=_cfg()).get_zero_state(2)[0].cx is None


def test_rnn_rejects_what_the_reference_rejects():
    AnalogRNN, _, Lstm, _, _ = _rnn_classes()
    with pytest.raises(RuntimeError, match="batch_first"):
        AnalogRNN(Lstm, 4, 5, batch_first=True, rpu_config=_cfg())
    with pytest.raises(RuntimeError, match="proj_size"):
        AnalogRNN(Lstm, 4, 5, proj_size=2, rpu_config=_cfg())
    with pytest.warns(UserWarning, match="dropout"):
        AnalogRNN(Lstm, 4, 5, dropout=0.5, rpu_config=_cfg())
    net = AnalogRNN(Lstm, 4, 5, num_layers=2, rpu_config=_cfg())
    with pytest.raises(RuntimeError, match="2D or 3D"):
        net(torch.zeros(4))
    with pytest.raises(RuntimeError, match="Expecting 2 states"):
        net(torch.zeros(3, 2, 4), net.get_zero_state(2)[:1])
    with pytest.raises(RuntimeError, match="input_size"):
        net(torch.zeros(3, 2, 7))
    with pytest.raises(RuntimeError, match="Expected hidden size"):
        net(torch.zeros(3, 2, 4), net.get_zero_state(3))
    with pytest.raises(RuntimeError, match="should be 2-D"):
        bad = [type(s)(s.hx[0], s.cx[0]) for s in net.get_zero_state(2)]
        net(torch.zeros(3, 2, 4), bad)


@pytest.mark.parametrize("kind", ["RNN", "LSTM", "GRU"])
@pytest.mark.parametrize("bidir", [False, True])
def test_rnn_state_dict_uses_torchs_flat_names(kind, bidir):
    """reference rnn.py:359-392: the state dict carries torch's names and loads from either."""
    AnalogRNN = _rnn_classes()[0]
    digital = getattr(torch.nn, kind)(6, 8, 2, bidirectional=bidir)
    analog = AnalogRNN.from_digital(digital, _cfg(max_input_size=4))
    state = analog.state_dict()
    for key, value in digital.state_dict().items():
        assert torch.equal(state[key], value), key
    extra = set(state) - set(digital.state_dict())
    assert "input_range_ih_l0" in extra and "input_range_update_idx_hh_l1" in extra
    if bidir:
        assert "input_range_hh_l1_reverse" in extra
    assert not [k for k in state if k.startswith("rnn.")]
    # loads its own state dict and a plain torch one
    other = AnalogRNN.from_digital(getattr(torch.nn, kind)(6, 8, 2, bidirectional=bidir),
                                   _cfg(max_input_size=4))
    assert not any(other.load_state_dict(state))
    for (_, _, a), (_, _, b) in zip(analog.cells(), other.cells()):
        assert torch.equal(a.weight_hh.weight, b.weight_hh.weight)
    report = other.load_state_dict(digital.state_dict(), strict=False)
    assert not report.unexpected_keys
    # nested in a model the prefix is kept
    nest = torch.nn.Sequential(analog)
    assert "0.weight_ih_l0" in nest.state_dict()
    assert not any(torch.nn.Sequential(other).load_state_dict(nest.state_dict()))
    back = AnalogRNN.to_digital(analog)
    assert type(back) is type(digital)
    for key, value in digital.state_dict().items():
        assert torch.equal(back.state_dict()[key], value), key


class _SeqNet(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.gru1 = torch.nn.GRU(10, 10, 1)
        self.lstm1 = torch.nn.LSTM(10, 20, 3, bidirectional=True)
        self.lstm2 = torch.nn.LSTM(40, 20, 3, bias=False, bidirectional=True)
        self.rnn1 = torch.nn.RNN(40, 20, 3, dropout=0.1)
        self.head = torch.nn.Linear(20, 4)


def test_convert_recurrent_layers_to_analog_and_back():
    """reference tests/test_conversion.py:95-150."""
    from aihwkit_lightning.nn.conversion import convert_to_analog, convert_to_digital
    AnalogRNN, Vanilla, Lstm, Gru, _ = _rnn_classes()
    model = _SeqNet()
    analog = convert_to_analog(model, _cfg(), ensure_analog_root=False)
    assert isinstance(analog.gru1, AnalogRNN) and isinstance(analog.gru1.rnn.layers[0].cell, Gru)
    assert isinstance(analog.lstm1.rnn.layers[2].directions[1].cell, Lstm)
    assert analog.lstm2.rnn.layers[0].directions[0].cell.weight_ih.bias is None
    assert isinstance(analog.rnn1.rnn.layers[0].cell, Vanilla)
    assert analog.rnn1.rnn.dropout_layer.p == 0.1
    assert isinstance(analog.head, AnalogLinear)
    digital = convert_to_digital(analog)
    for name in ("gru1", "lstm1", "lstm2", "rnn1"):
        assert type(getattr(digital, name)) is type(getattr(model, name))
    for key, value in model.state_dict().items():
        assert torch.equal(digital.state_dict()[key], value), key
    assert isinstance(convert_to_analog(model, _cfg()), AnalogWrapper)


def test_wrapped_model_can_be_pickled():
    """``torch.save(model)`` of a converted model: the wrapper's dynamic class is rebuilt on load
    (in the reference this fails with a PicklingError)."""
    import io
    import pickle

    from aihwkit_lightning.nn.conversion import convert_to_analog

    model = convert_to_analog(_Net(), _cfg())
    assert isinstance(model, AnalogWrapper)
    clone = pickle.loads(pickle.dumps(model))
    assert type(clone) is type(model) and isinstance(clone, _Net)
    for (name, a), (_, b) in zip(model.state_dict().items(), clone.state_dict().items()):
        assert torch.equal(a, b), name
    buffer = io.BytesIO()
    torch.save(model, buffer)
    buffer.seek(0)
    again = torch.load(buffer, weights_only=False)
    assert len(list(again.analog_layers())) == len(list(model.analog_layers()))


def test_module_level_helpers_of_the_reference_exist():
    """``is_at_least_volta_gpu`` and ``unfold3d`` are module-level names of the reference's
    ``linear.py`` / ``conv.py``; without a device the first says no and the second refuses."""
    from aihwkit_lightning.exceptions import HipBackendError
    from aihwkit_lightning.nn.modules import conv, linear

    assert linear.is_at_least_volta_gpu is conv.is_at_least_volta_gpu
    if not torch.cuda.is_available():
        assert linear.is_at_least_volta_gpu() is False
        with pytest.raises(HipBackendError):
            conv.unfold3d(torch.zeros(1, 1, 2, 2, 2), (1, 1, 1))
    with pytest.raises(ValueError):
        conv.unfold3d(torch.zeros(2, 2), (1, 1, 1))


def test_fake_kernels_give_shapes_without_a_gpu():
    """Every custom op has a fake kernel (what torch.compile and opcheck trace with): under
    FakeTensorMode the ops return tensors of the right shape, dtype and device and launch nothing."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from aihwkit_lightning.nn.modules.hip_utils import library as L
    from aihwkit_lightning.nn.modules.hip_utils.ops import OPS

    in_sizes = [256, 256]
    icfg = [L.AHL_IR_DYNAMIC, 0, 1, 0, 0, 0, 0]
    fcfg = [254.0, 254.0, 0.5, 0.0, 0.01, 0.95]
    with FakeTensorMode():
        x = torch.empty(64, 512, device="cuda", dtype=torch.bfloat16)
        w = torch.empty(96, 512, device="cuda", dtype=torch.bfloat16)
        wmax, tile_max, tile_min, w_eff = OPS.weight_prep(w, in_sizes, 0, 2, 1.0, 0.02, 3, 0, True)
        assert wmax.shape == (2, 96) and tile_max.shape == (2,) and tile_min.dtype == torch.float32
        assert w_eff.shape == w.shape and w_eff.dtype == w.dtype
        xq, ir_dyn = OPS.dac(x, None, in_sizes, icfg, fcfg)
        assert xq.shape == x.shape and ir_dyn.shape == (2, 64)
        y, keep, flag = OPS.linear_fwd(x, xq, w_eff, None, ir_dyn, wmax, tile_max, in_sizes, icfg, fcfg, True)
        assert y.shape == (64, 96) and y.device.type == "cuda" and keep.shape == (2, 3, 64) and flag.shape == (1,)
        dx, ir_grad = OPS.linear_bwd_dx(y, keep, flag, w_eff, x, ir_dyn, in_sizes, icfg, fcfg)
        assert dx.shape == x.shape and ir_grad.numel() == 0
        dw, db = OPS.linear_bwd_dw(y, keep, flag, x, xq, ir_dyn, in_sizes, icfg, fcfg, True)
        assert dw.shape == w.shape and db.shape == (96,)
        assert OPS.sliced_std(x.float(), in_sizes).shape == (2,)
        assert OPS.sliced_quantile(x.float(), in_sizes, 0.99).shape == (2,)
        assert OPS.pad_tiles(x, [200, 312], 512).shape == (64, 1024)
        geom = [2, 8, 1, 12, 12, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1]
        cols = OPS.im2col(torch.empty(2, 8, 1, 12, 12, device="cuda"), geom)
        assert cols.shape == (2, 144, 72) and OPS.col2im(cols, geom).shape == (2, 8, 1, 12, 12)


def test_shape_inference_switch_is_per_thread():
    """While one thread evaluates a fake kernel (torch.compile / opcheck tracing) the library stays
    live for every other thread: the autograd engine's device thread runs the backward ops and must
    launch them, not return unwritten buffers."""
    import threading

    from aihwkit_lightning.nn.modules.hip_utils import ops

    seen = {}

    def body():
        seen["tracing thread"] = ops._SHAPES_ONLY.depth   # pylint: disable=protected-access
        other = threading.Thread(target=lambda: seen.__setitem__("other thread", ops._SHAPES_ONLY.depth))
        other.start()
        other.join()
        return 0

    assert ops._shapes_only(body)() == 0   # pylint: disable=protected-access
    assert seen == {"tracing thread": 1, "other thread": 0}
    assert ops._SHAPES_ONLY.depth == 0   # pylint: disable=protected-access
