"""A training step (forward + backward) of an analog layer replayed from HIP graphs: equal to
the eager step when nothing is random, fresh noise on every replay when something is."""
import pytest
import torch

from golden_cases import case, make_inputs

pytestmark = pytest.mark.gpu


def _layer(c, w, b):
    from hip_helpers import make_layer

    return make_layer(c, inputs=(None, w, b, None))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_graphed_step_equals_eager_step_without_noise(dtype):
    from aihwkit_lightning.nn.graphs import graphed_module

    c = case("graph_plain", dtype=dtype, M=512, K=1024, N=768, max_input_size=512, ir_mode="static",
             inp_res=254, out_res=254, out_bound=0.6, clip="channel", clip_sigma=2.5, ir_decay=0.01,
             w_scale=0.05, seed=81)
    x, w, b, g = make_inputs(c)
    eager = _layer(c, w, b)
    xe = x.cuda().requires_grad_(True)
    out_e = eager(xe)
    out_e.backward(g.cuda())
    graphed_layer = _layer(c, w, b)
    step = graphed_module(graphed_layer, (x.cuda().requires_grad_(True),))
    for replay in range(3):
        for p in graphed_layer.parameters():
            p.grad = None
        xg = x.cuda().requires_grad_(True)
        out_g = step(xg)
        out_g.backward(g.cuda())
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"out, replay {replay}"
        assert torch.equal(xg.grad, xe.grad), f"dx, replay {replay}"
        assert torch.equal(graphed_layer.weight.grad, eager.weight.grad), f"dw, replay {replay}"
        assert torch.equal(graphed_layer.bias.grad, eager.bias.grad), f"db, replay {replay}"
        assert torch.equal(graphed_layer.input_range.grad, eager.input_range.grad), f"dir, replay {replay}"
        # eager work and a synchronisation between the replays
        _ = (out_g.float() @ out_g.float().t()).sum().item()


def test_whole_step_in_one_graph_equals_eager_step():
    """Forward + backward recorded into one graph (CapturedStep), replayed with eager work and
    synchronisations in between: outputs and all gradients equal the eager step bit for bit."""
    from aihwkit_lightning.nn.graphs import CapturedStep

    c = case("graph_whole", dtype="bf16", M=640, K=1536, N=512, max_input_size=512, ir_mode="static",
             inp_res=254, out_res=254, out_bound=0.6, clip="channel", clip_sigma=2.5, ir_decay=0.01,
             w_scale=0.05, seed=84)
    x, w, b, g = make_inputs(c)
    eager = _layer(c, w, b)
    xe = x.cuda().requires_grad_(True)
    out_e = eager(xe)
    out_e.backward(g.cuda())
    layer = _layer(c, w, b)
    xs, gs = x.cuda().requires_grad_(True), g.cuda()

    def step():
        xs.grad = None
        layer.zero_grad(set_to_none=True)
        out = layer(xs)
        out.backward(gs)
        return out

    replay = CapturedStep(step)
    for i in range(3):
        out = replay()
        torch.cuda.synchronize()
        assert torch.equal(out, out_e), f"out, replay {i}"
        assert torch.equal(xs.grad, xe.grad), f"dx, replay {i}"
        assert torch.equal(layer.weight.grad, eager.weight.grad), f"dw, replay {i}"
        assert torch.equal(layer.bias.grad, eager.bias.grad), f"db, replay {i}"
        assert torch.equal(layer.input_range.grad, eager.input_range.grad), f"dir, replay {i}"
        _ = (out.float() @ out.float().t()).sum().item()


def test_graphed_step_draws_fresh_noise_on_every_replay():
    """Output noise and weight noise under replay: every replay differs from the last, the
    injected output noise has the configured scale, and the weight gradient changes with the
    weight noise (dX = g W_eff)."""
    from aihwkit_lightning.nn.graphs import graphed_module
    from oracle import torch_mode as om

    c = case("graph_noise", dtype="bf16", M=2048, K=1024, N=1024, max_input_size=512, ir_mode="static",
             inp_res=254, out_noise=0.5, out_noise_per_channel=True, weight_noise="add_normal_per_channel",
             modifier_std=0.05, w_scale=0.05, seed=82, bias=False, ir_values=[3.0, 3.0])
    from aihwkit_lightning.nn.modules.hip_utils import ops

    x, w, b, g = make_inputs(c)
    torch.manual_seed(21)
    ops._NOISE_STATES.clear()   # the state (and its key) is created by the first graphed_module
    layer = _layer(c, w, b)
    step = graphed_module(layer, (x.cuda().requires_grad_(True),))
    outs, dxs = [], []
    for _ in range(4):
        xg = x.cuda().requires_grad_(True)
        out = step(xg)
        out.backward(g.cuda())
        torch.cuda.synchronize()
        outs.append(out.detach().float().clone())
        dxs.append(xg.grad.float().clone())
    for i in range(3):
        assert not torch.equal(outs[i], outs[i + 1])
        assert not torch.equal(dxs[i], dxs[i + 1])
    # the difference of two replays is twice the noise variance (output noise of 2 tiles plus
    # the effect of the weight noise); its standard deviation against the closed form
    wmax = om.sliced_abs_max(w.float(), layer.in_sizes).cuda()   # [T, N]
    s = 0.5 / 2 ** 0.5 * 3.0
    var_out = ((s * wmax) ** 2).sum(0)                              # [N]
    xq_sq = (x.float().clamp(-3, 3) ** 2).cuda()                   # DAC steps are small against this
    var_w = torch.stack([(xq_sq[:, 512 * t:512 * (t + 1)].sum(1)[:, None] * (0.05 * wmax[t]) ** 2)
                         for t in range(2)]).sum(0)                 # [M, N]
    z = (outs[0] - outs[1]) / (2.0 * (var_out[None, :] + var_w)).sqrt()
    assert abs(float(z.mean())) < 0.01
    assert abs(float(z.std()) - 1.0) < 0.02
    # replays of a second graph recorded after the same torch seed start from the same key
    torch.manual_seed(21)
    ops._NOISE_STATES.clear()
    layer2 = _layer(c, w, b)
    step2 = graphed_module(layer2, (x.cuda().requires_grad_(True),))
    out2 = step2(x.cuda().requires_grad_(True))
    torch.cuda.synchronize()
    assert torch.equal(out2.detach().float(), outs[0])


def test_capture_without_noise_state_is_refused(monkeypatch):
    """A noisy layer that finds itself under stream capture without a device noise state must say
    so (creating the state would copy from the host inside the capture). The capture is
    pretended: the refusal comes before anything is launched."""
    from aihwkit_lightning.exceptions import HipBackendError
    from aihwkit_lightning.nn.modules.hip_utils import ops

    c = case("graph_refuse", dtype="bf16", M=256, K=512, N=256, max_input_size=256, ir_mode="static",
             inp_res=254, out_noise=0.1, seed=83, bias=False)
    x, w, b, _ = make_inputs(c)
    layer = _layer(c, w, b)
    xin = x.cuda()
    layer(xin)
    saved = dict(ops._NOISE_STATES)
    ops._NOISE_STATES.clear()
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    try:
        with pytest.raises(HipBackendError, match="noise state"):
            layer(xin)
    finally:
        ops._NOISE_STATES.update(saved)


def test_recurrent_training_step_in_one_graph_equals_eager_step():
    """A two-layer LSTM's forward + backward through time recorded into one graph (hundreds of
    launches the eager step spreads over Python): outputs and every gradient equal the eager
    step's, replay after replay, and with output noise on the replays differ from each other."""
    from aihwkit_lightning.nn.graphs import CapturedStep
    from rnn_cases import rnn_case
    from test_hip_rnn import build_network

    def net_and_step(out_noise):
        c = rnn_case("graph_lstm", "lstm", 6, 8, 64, 64, layers=2, bidir=False, max_input_size=32,
                     dtype="bf16", ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5,
                     w_scale=0.2, inp_res=254, out_res=254, out_bound=10.0, out_noise=out_noise,
                     training=True, seed=74)
        net, _ = build_network(c)
        gen = torch.Generator().manual_seed(9)
        x = torch.randn(6, 8, 64, generator=gen).bfloat16().cuda().requires_grad_(True)
        g = torch.randn(6, 8, 64, generator=gen).bfloat16().cuda()

        def step():
            x.grad = None
            net.zero_grad(set_to_none=True)
            out = net(x)[0]
            out.backward(g)
            return out
        return net, x, step

    net_e, x_e, step_e = net_and_step(0.0)
    out_e = step_e()
    net_g, x_g, step_g = net_and_step(0.0)
    replay = CapturedStep(step_g)
    for i in range(3):
        out = replay()
        torch.cuda.synchronize()
        assert torch.equal(out, out_e), f"out, replay {i}"
        assert torch.equal(x_g.grad, x_e.grad), f"dx, replay {i}"
        for (name, p_g), (_, p_e) in zip(net_g.named_parameters(), net_e.named_parameters()):
            if p_e.grad is not None:
                assert torch.equal(p_g.grad, p_e.grad), f"{name}, replay {i}"
        _ = out.float().sum().item()
    _, _, step_n = net_and_step(0.1)
    noisy = CapturedStep(step_n)
    outs = []
    for _ in range(3):
        outs.append(noisy().detach().float().clone())
        torch.cuda.synchronize()
    assert not torch.equal(outs[0], outs[1]) and not torch.equal(outs[1], outs[2])


def test_convolution_step_on_the_image_in_one_graph_equals_eager_step():
    """A convolution that runs without the patch matrix, forward + backward in one graph, with a
    bound that clamps (the clamp flag under replay) and replays with a different input in between:
    every replay equals the eager step on the same input bit for bit. With output noise on, every
    replay draws new noise."""
    from conv_cases import conv_case, make_conv_inputs
    from test_hip_conv import make_conv_layer
    from aihwkit_lightning.nn.graphs import CapturedStep
    from aihwkit_lightning.nn.modules.hip_utils import hip_conv

    c = conv_case("graph_conv", 2, 4, 128, (12, 10), (3, 3), (1, 1), (1, 1), N=128, dtype="bf16",
                  max_input_size=576, ir_mode="static", ir_values=[2.0, 1.5], inp_res=254, out_res=254,
                  out_bound=2.0, clip="channel", clip_sigma=2.5, ir_decay=0.01, w_scale=0.05, seed=90)
    x, w, b, g = make_conv_inputs(c)
    inputs = [x.cuda(), (0.05 * x).cuda()]   # the second one clamps nothing
    eager_results = []
    for xin in inputs:
        eager = make_conv_layer(c, w, b)
        xe = xin.clone().requires_grad_(True)
        out = eager(xe)
        out.backward(g.cuda())
        eager_results.append((out.detach(), xe.grad, eager.weight.grad, eager.bias.grad, eager.input_range.grad))
    layer = make_conv_layer(c, w, b)
    xs, gs = inputs[0].clone().requires_grad_(True), g.cuda()
    calls = []
    real = hip_conv.HipConv.forward
    hip_conv.HipConv.forward = staticmethod(lambda *a: calls.append(1) or real(*a))
    try:
        def step():
            xs.grad = None
            layer.zero_grad(set_to_none=True)
            out = layer(xs)
            out.backward(gs)
            return out

        replay = CapturedStep(step)
    finally:
        hip_conv.HipConv.forward = real
    assert calls, "the recorded step did not take the image path"
    for i, which in enumerate([0, 1, 0, 0, 1]):
        with torch.no_grad():
            xs.copy_(inputs[which])
        out = replay()
        torch.cuda.synchronize()
        want = eager_results[which]
        got = (out, xs.grad, layer.weight.grad, layer.bias.grad, layer.input_range.grad)
        for name, a, e in zip(("out", "dx", "dw", "db", "dir"), got, want):
            assert torch.equal(a, e), f"{name}, replay {i} (input {which})"
        _ = (out.float().flatten(1) @ out.float().flatten(1).t()).sum().item()

    noisy = dict(c, out_noise=0.3, name="graph_conv_noise")
    layer = make_conv_layer(noisy, w, b)
    xn = inputs[0].clone().requires_grad_(True)

    def noisy_step():
        xn.grad = None
        layer.zero_grad(set_to_none=True)
        out = layer(xn)
        out.backward(gs)
        return out

    replay = CapturedStep(noisy_step)
    outs = []
    for _ in range(3):
        outs.append(replay().detach().clone())
        torch.cuda.synchronize()
    assert not torch.equal(outs[0], outs[1]) and not torch.equal(outs[1], outs[2])
