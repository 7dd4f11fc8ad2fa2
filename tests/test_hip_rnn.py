"""GPU parity of the recurrent layers (AnalogRNN -> cells -> AnalogLinear -> custom ops -> C ABI)
against the CPU oracle and the reference's golden vectors.

Acceptance rule as for the linear operator: 1e-5 (fp32) / 1e-2 (bf16) relative to the tensor
scale, for everything in fp32 and for the outputs and states in bf16 (which in fact agree bit for
bit). Gradients in bf16 cannot be held to an element-wise 1e-2 against ANY CPU computation:
torch's own backward kernels of sigmoid and tanh round after every operation on the CPU and once
on the GPU, so that with identical inputs 30-40 % of their results are one bf16 step (0.4-0.8 %)
apart, and the recurrence sums several such terms in bf16. For those tensors the rule is
therefore stated in norm: relative L2 error against the oracle at most 2e-2, no element further
than 1e-1 of the tensor scale, and the error against the oracle evaluated in fp32 (the gradient
both approximate) no larger than the bf16 oracle's own, up to 10 % + 1e-3.
"""
import itertools
import os

import numpy as np
import pytest
import torch

from golden_cases import DTYPES
from helpers import TieLog, assert_close_lsb, product_hook, rel_scale_mismatch
from hip_helpers import rpu_config
from rnn_cases import RNN_CASES, cell_slots, make_rnn_inputs, rnn_case, scalar_loss
from test_oracle_rnn import golden_of, oracle_run

pytestmark = pytest.mark.gpu

RTOL = {"f32": 1e-5, "bf16": 1e-2}


def build_network(case, device="cuda"):
    """The product's AnalogRNN with the case's weights; returns (network, cells in module order)."""
    from aihwkit_lightning.nn import (AnalogGRUCell, AnalogLSTMCell,
                                      AnalogLSTMCellCombinedWeight, AnalogRNN,
                                      AnalogVanillaRNNCell)
    kinds = {"rnn": AnalogVanillaRNNCell, "lstm": AnalogLSTMCell, "gru": AnalogGRUCell,
             "lstm_combined": AnalogLSTMCellCombinedWeight}
    _, params, _, _ = make_rnn_inputs(case)
    net = AnalogRNN(kinds[case["cell"]], case["inputs"], case["hidden"], case["layers"],
                    bias=case["bias"], bidir=case["bidir"], dtype=DTYPES[case["dtype"]],
                    rpu_config=rpu_config(case))
    cells = [cell for _, _, cell in net.cells()]
    assert len(cells) == len(params)
    for cell, cell_params in zip(cells, params):
        for proj, (w, b) in cell_params.items():
            getattr(cell, proj).set_weights_and_biases(w, b)
    net = net.to(device)
    net.train(case["training"])
    return net, cells


def product_run(case, net=None, cells=None):
    """Forward (+ backward in training mode) on the GPU; dict keyed like the fixtures."""
    from aihwkit_lightning.nn.modules.rnn.cells import LSTMState
    x, params, states, g = make_rnn_inputs(case)
    if net is None:
        net, cells = build_network(case)
    net_states = None
    if states is not None:
        flat = [LSTMState(h.cuda(), None if c is None else c.cuda()) for h, c in states]
        net_states = ([tuple(flat[2 * i:2 * i + 2]) for i in range(case["layers"])]
                      if case["bidir"] else flat)
    xin = x.cuda().requires_grad_(True)
    torch.manual_seed(case["noise_seed"])
    out, last = net(xin, net_states)
    last_flat = [s for pair in last for s in pair] if case["bidir"] else list(last)
    last_flat = [(s[0], s[1]) for s in last_flat]
    res = {"out": out.detach().cpu()}
    for i, (hx, cx) in enumerate(last_flat):
        res[f"h{i}"] = hx.detach().cpu()
        if cx is not None:
            res[f"c{i}"] = cx.detach().cpu()
    if case["training"]:
        scalar_loss(out, last_flat, g.cuda()).backward()
        torch.cuda.synchronize()
        res["dx"] = xin.grad.cpu()
        for i, (cell, cell_params) in enumerate(zip(cells, params)):
            for proj in cell_params:
                lin = getattr(cell, proj)
                res[f"{i}/{proj}/dw"] = lin.weight.grad.cpu()
                if lin.bias is not None:
                    res[f"{i}/{proj}/db"] = lin.bias.grad.cpu()
                if lin.input_range is not None and lin.input_range.grad is not None:
                    res[f"{i}/{proj}/dir"] = lin.input_range.grad.cpu()
    return res


def _adc_step(case):
    return 2 * case["out_bound"] / case["out_res"] if case["out_res"] > 0 else None


def _is_state(key):
    return key == "out" or (key[0] in "hc" and key[1:].isdigit())


def _rel_l2(a, b):
    norm = float(b.double().norm())
    return float((a.double() - b.double()).norm()) / norm if norm > 0 else float(a.double().norm())


def _compare(case, got, want, what, exact=None, states_in_norm=False):
    """``exact``: the same tensors from the oracle in fp32, for the bf16 gradient rule.
    ``states_in_norm``: hold the outputs and states to the norm rule as well (bf16 networks in which
    the oracle finds rounding ties, see :func:`compare_up_to_ties`)."""
    assert set(got) == set(want), set(got) ^ set(want)
    for key, ref in want.items():
        val = got[key].float().reshape(ref.shape)
        name = f"{case['name']}/{key} vs {what}"
        if case["dtype"] == "f32" or (_is_state(key) and not states_in_norm):
            assert_close_lsb(val, ref.float(), RTOL[case["dtype"]], lsb=_adc_step(case), what=name)
            continue
        assert _rel_l2(val, ref) <= 2e-2, f"{name}: relative L2 error {_rel_l2(val, ref):.3e}"
        assert not rel_scale_mismatch(val, ref.float(), 1e-1).any(), name
        if exact is not None and not _is_state(key):
            # Both are bf16 evaluations of the fp32 gradient with independent roundings: the ratio
            # of the two error norms scatters with the number of elements they are taken over (a
            # bias gradient of 8 elements, an input gradient of 6), hence the second term.
            truth = exact[key].float().reshape(ref.shape)
            factor = 1.1 + 4.0 / ref.numel() ** 0.5
            assert _rel_l2(val, truth) <= factor * _rel_l2(ref.float(), truth) + 1e-3, name


def _fp32_oracle(case):
    if case["dtype"] == "f32" or not case["training"]:
        return None
    return oracle_run({**case, "dtype": "f32"})


# What separates two fp32 evaluations of exp / tanh / sigmoid chains (CPU and GPU libraries differ in
# the last place, and a cell chains several): relative size of the difference at a later layer's input.
ACTIVATION_ERR = 4.0 * 2.0 ** -24


def oracle_with_ties(case, flip=()):
    log = TieLog(flip, input_err=ACTIVATION_ERR)
    with product_hook(log):
        ref = oracle_run(case)
    return ref, log


def compare_up_to_ties(case, got, exact=None):
    """Product against the oracle, element-wise as :func:`_compare` states. A network feeds one
    layer's rounded outputs into the next, so a single rounding tie (a tile product within the fp32
    accumulation error of an ADC level change; a DAC input within the last place of exp / tanh of a
    level change) moves everything behind it in that batch row, and element-wise bounds do not
    compose. The oracle finds its own ties (``helpers.TieLog``). If the comparison fails and ties
    exist in the rows that differ (batch rows never mix), fp32 networks must equal the oracle with
    some of THOSE ties resolved the other way, element-wise again; 16-bit networks, where ties are
    too many to enumerate, are held to the norm rule in outputs and states too. Returns the oracle
    result that matched."""
    ref, log = oracle_with_ties(case)
    try:
        _compare(case, got, ref, "oracle", exact)
        return ref
    except AssertionError as first:
        if not log.ties and not log.dac_ties:
            raise
        if case["dtype"] != "f32":
            _compare(case, got, ref, "oracle (norm rule: the oracle has rounding ties)", exact,
                     states_in_norm=True)
            return ref
        out_got, out_ref = got["out"].float().reshape(ref["out"].shape), ref["out"].float()
        if out_ref.dim() == 2:
            out_got, out_ref = out_got.unsqueeze(1), out_ref.unsqueeze(1)
        rows = set(rel_scale_mismatch(out_got, out_ref, RTOL["f32"]).nonzero()[:, 1].tolist())
        cand = [t for t in log.ties if t[1] in rows] + [t for t in log.dac_ties if t[2] in rows]
        tries = 0
        for size in range(1, min(len(cand), 3) + 1):
            for subset in itertools.combinations(cand, size):
                tries += 1
                if tries > 200:
                    raise first
                ref2, _ = oracle_with_ties(case, subset)
                try:
                    _compare(case, got, ref2, f"oracle with the ties {subset} resolved the other way", exact)
                    return ref2
                except AssertionError:
                    continue
        raise first


@pytest.mark.parametrize("case", RNN_CASES, ids=[c["name"] for c in RNN_CASES])
def test_network_matches_oracle_and_reference_vectors(case):
    print(f"case {case['name']}", flush=True)
    got = product_run(case)
    matched = compare_up_to_ties(case, got, _fp32_oracle(case))
    if all(torch.equal(matched[k], v) for k, v in oracle_run(case).items()):
        _compare(case, got, golden_of(case), "reference vectors")


BIGGER = [
    # fast-kernel shapes (bf16, output widths that are multiples of 8), uneven tiles of 43 / 42
    rnn_case("lstm_bf16_wide", "lstm", 5, 16, 96, 64, layers=2, bidir=True, max_input_size=48,
             dtype="bf16", ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5,
             ir_decay=0.01, w_scale=0.1, inp_res=254, out_res=254, out_bound=10.0, seed=70),
    rnn_case("gru_bf16_wide", "gru", 6, 24, 85, 64, layers=2, max_input_size=43, dtype="bf16",
             ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
             w_scale=0.1, inp_res=254, out_res=254, out_bound=10.0, seed=71),
    rnn_case("rnn_f32_wide", "rnn", 6, 24, 85, 64, layers=2, bidir=True, max_input_size=43,
             ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
             w_scale=0.1, inp_res=254, out_res=254, out_bound=10.0, seed=72),
]


@pytest.mark.parametrize("case", BIGGER, ids=[c["name"] for c in BIGGER])
def test_wider_networks_match_the_oracle(case):
    print(f"case {case['name']}", flush=True)
    compare_up_to_ties(case, product_run(case), _fp32_oracle(case))


# Three random networks that a longer run of such cases turned up, kept by name.
# tie_lstm_f32: the input of the second layer's cell at one step holds, in batch row 7, a value whose
# DAC quotient lies within the last place of tanh / sigmoid of a level change; the GPU's activation
# functions put it on the other level, and everything behind it in that row moves (158 of 4896
# outputs, by up to 3e-3). With that ONE tie resolved the other way the oracle equals the product to
# 1.5e-8. grad_rnn_bf16_a / _b: no converter at all (nothing to tie); their 6-element input gradient and
# 8-element bias gradient are within 0.8 % / 0.5 % of the bf16 oracle in norm, and only the ratio of the
# two bf16 evaluations' errors against fp32 (1.75, 1.95) exceeded a bound meant for large tensors.
FOUND = [
    rnn_case("tie_lstm_f32", "lstm_combined", 9, 17, 6, 16, layers=3, bidir=True, bias=False,
             max_input_size=-1, w_scale=0.2, seed=301, ir_mode="dynamic", ir_init=2.0, ir_decay=0.01,
             inp_res=254, out_res=254, out_bound=10.0, clip="none", clip_sigma=2.5, training=False),
    rnn_case("grad_rnn_bf16_a", "rnn", 2, 3, 1, 64, layers=3, bias=True, max_input_size=6, dtype="bf16",
             w_scale=0.2, seed=315),
    rnn_case("grad_rnn_bf16_b", "rnn", 2, 8, 16, 8, layers=2, bias=True, max_input_size=48, dtype="bf16",
             w_scale=0.2, seed=372),
]


@pytest.mark.parametrize("case", FOUND, ids=[c["name"] for c in FOUND])
def test_networks_found_by_random_search(case):
    print(f"case {case['name']}", flush=True)
    got = product_run(case)
    matched = compare_up_to_ties(case, got, _fp32_oracle(case))
    if case["name"] == "tie_lstm_f32":
        # the tie is there, and it is what separates the two results
        plain, log = oracle_with_ties(case)
        assert ("dac", 24, 7, 23) in log.dac_ties
        if not torch.equal(matched["out"], plain["out"]):
            flipped, _ = oracle_with_ties(case, [("dac", 24, 7, 23)])
            assert torch.equal(matched["out"], flipped["out"])


@pytest.mark.parametrize("cell", ["rnn", "lstm", "gru"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_projecting_the_sequence_ahead_equals_stepping(cell, dtype):
    """In evaluation mode the input projection of all steps is one product; the result must be
    the one of stepping the cell, bit for bit (rows of a product do not depend on each other)."""
    print(f"case {cell} {dtype}", flush=True)
    case = rnn_case("ahead", cell, 7, 5, 40, 32, layers=2, bidir=True, max_input_size=24,
                    dtype=dtype, ir_mode="dynamic" if cell == "gru" else "static", ir_init=2.0,
                    clip="channel", clip_sigma=2.5, w_scale=0.2, inp_res=254, out_res=254,
                    out_bound=10.0, training=False, seed=73)
    net, cells = build_network(case)
    ahead = product_run(case, net, cells)
    from aihwkit_lightning.nn.modules.rnn.layers import AnalogRNNLayer
    layers = [m for m in net.modules() if isinstance(m, AnalogRNNLayer)]
    assert len(layers) == 4 and all(m._project_ahead() for m in layers)
    for m in layers:
        m._project_ahead = lambda: False
    stepped = product_run(case, net, cells)
    for key, val in ahead.items():
        assert torch.equal(val, stepped[key]), key


def test_plain_network_is_torchs_lstm_on_the_gpu():
    """from_digital -> forward -> to_digital against torch.nn.LSTM itself, no non-idealities."""
    from aihwkit_lightning.nn import AnalogRNN
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig
    torch.manual_seed(5)
    digital = torch.nn.LSTM(24, 16, 2, bidirectional=True).cuda()
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 16
    analog = AnalogRNN.from_digital(digital, cfg)
    x = torch.randn(6, 4, 24, device="cuda")
    want, (h_n, c_n) = digital(x)
    got, last = analog(x)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)
    flat = [s for pair in last for s in pair]
    for i, (hx, cx) in enumerate(flat):
        assert torch.allclose(hx, h_n[i], rtol=1e-5, atol=1e-6)
        assert torch.allclose(cx, c_n[i], rtol=1e-5, atol=1e-6)
    back = AnalogRNN.to_digital(analog)
    assert torch.equal(back(x)[0], want)


@pytest.mark.parametrize("cell", ["lstm", "gru"])
def test_graph_replays_equal_the_eager_forward(cell):
    """The recorded sequence is replayed several times with new inputs and with eager work and
    synchronisations in between; every replay must equal the eager result bit for bit."""
    print(f"case graph {cell}", flush=True)
    case = rnn_case("graph", cell, 9, 4, 40, 32, layers=2, bidir=True, max_input_size=24,
                    dtype="bf16", ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5,
                    w_scale=0.2, inp_res=254, out_res=254, out_bound=10.0, training=False, seed=74)
    net, _ = build_network(case)
    gen = torch.Generator().manual_seed(3)
    example = torch.randn(9, 4, 40, generator=gen).bfloat16().cuda()
    replay = net.graphed(example)
    for trial in range(4):
        x = (torch.randn(9, 4, 40, generator=gen) * (1 + trial)).bfloat16().cuda()
        with torch.no_grad():
            want, want_states = net(x)
        scratch = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")
        torch.cuda.synchronize()
        got, got_states = replay(x)
        assert torch.equal(got, want), trial
        for pair_g, pair_w in zip(got_states, want_states):
            for s_g, s_w in zip(pair_g, pair_w):
                assert torch.equal(s_g[0], s_w[0]), trial
                if s_w[1] is not None:
                    assert torch.equal(s_g[1], s_w[1]), trial
        del scratch
    # in-place weight updates are seen by the graph
    with torch.no_grad():
        for _, _, c in net.cells():
            c.weight_hh.weight.mul_(0.5)
        want, _ = net(x)
    assert torch.equal(replay(x)[0], want)
    with pytest.raises(RuntimeError, match="recorded for input"):
        replay(x[:5])
    net.train()
    with pytest.raises(RuntimeError, match="evaluation-mode"):
        net.graphed(example)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("rows,hidden", [(3, 8), (64, 1024), (17, 40)])
def test_fused_gates_match_the_chain_of_torch_operations(dtype, rows, hidden):
    """ahl_lstm_gates_* / ahl_gru_gates_* against the element-wise torch operations they replace,
    on the same device: the forward bit for bit in fp32 up to the last place of exp / tanh and
    exactly in bf16 (both round an fp32 activation once), the gradients to the dtype's rounding."""
    from aihwkit_lightning.nn.modules.rnn import cells

    print(f"case gates {dtype} {rows}x{hidden}", flush=True)
    gen = torch.Generator().manual_seed(9)
    mk = lambda *shape: (torch.randn(*shape, generator=gen) * 1.5).to(dtype).cuda().requires_grad_(True)  # noqa: E731
    # bf16 gradients: one rounding that falls the other way (torch's kernels contract a * b + c,
    # this library does not) is one step of the larger operand where two terms cancel, so the
    # element-wise bound is a step at the operands' magnitude (~4) and the norm is checked too
    tol = dict(rtol=2e-6, atol=2e-6) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=3.2e-2)

    def close(a, b):
        a, b = a.float(), b.float()
        return torch.allclose(a, b, **tol) and float((a - b).norm()) <= 5e-3 * float(b.norm())

    def chain_lstm(ig, hg, c_x):
        i, f, g, o = (ig + hg).chunk(4, 1)
        c_y = torch.sigmoid(f) * c_x + torch.sigmoid(i) * torch.tanh(g)
        return torch.sigmoid(o) * torch.tanh(c_y), c_y

    def chain_gru(ig, hg, h_x):
        i_r, i_z, i_n = ig.chunk(3, 1)
        h_r, h_z, h_n = hg.chunk(3, 1)
        r, z = torch.sigmoid(i_r + h_r), torch.sigmoid(i_z + h_z)
        n = torch.tanh(i_n + r * h_n)
        return n + z * (h_x - n)

    # LSTM, both outputs used
    ig, hg, c_x = mk(rows, 4 * hidden), mk(rows, 4 * hidden), mk(rows, hidden)
    g_h, g_c = mk(rows, hidden).detach(), mk(rows, hidden).detach()
    assert cells.gate_ops.gates_supported(ig, hg, c_x, 4)
    h_y, c_y = cells.lstm_pointwise(ig, hg, c_x)
    ((h_y * g_h).sum() + (c_y * g_c).sum()).backward()
    got = [t.grad.clone() for t in (ig, hg, c_x)]
    for t in (ig, hg, c_x):
        t.grad = None
    want_h, want_c = chain_lstm(ig, hg, c_x)
    ((want_h * g_h).sum() + (want_c * g_c).sum()).backward()
    if dtype == torch.bfloat16:
        assert torch.equal(h_y, want_h) and torch.equal(c_y, want_c)
    else:
        assert torch.allclose(h_y, want_h, **tol) and torch.allclose(c_y, want_c, **tol)
    for a, t in zip(got, (ig, hg, c_x)):
        assert close(a, t.grad)
    # LSTM, only the hidden state used (the cell state's gradient is absent)
    for t in (ig, hg, c_x):
        t.grad = None
    h_y, _ = cells.lstm_pointwise(ig, hg, c_x)
    (h_y * g_h).sum().backward()
    got = [t.grad.clone() for t in (ig, hg, c_x)]
    for t in (ig, hg, c_x):
        t.grad = None
    (chain_lstm(ig, hg, c_x)[0] * g_h).sum().backward()
    for a, t in zip(got, (ig, hg, c_x)):
        assert close(a, t.grad)
    # GRU
    ig, hg, h_x = mk(rows, 3 * hidden), mk(rows, 3 * hidden), mk(rows, hidden)
    h_y = cells.gru_pointwise(ig, hg, h_x)
    (h_y * g_h).sum().backward()
    got = [t.grad.clone() for t in (ig, hg, h_x)]
    for t in (ig, hg, h_x):
        t.grad = None
    want = chain_gru(ig, hg, h_x)
    (want * g_h).sum().backward()
    if dtype == torch.bfloat16:
        assert torch.equal(h_y, want)
    else:
        assert torch.allclose(h_y, want, **tol)
    for a, t in zip(got, (ig, hg, h_x)):
        assert close(a, t.grad)
    # a hidden size that is not a whole number of vectors takes the torch chain
    odd = mk(rows, 6)
    assert not cells.gate_ops.gates_supported(mk(rows, 24), None, odd, 4)
    # a state in another dtype than the projections (a user-built state) takes the torch chain
    # too, which type-promotes, instead of a kernel that would read the projections out of bounds
    other = torch.float32 if dtype == torch.bfloat16 else torch.bfloat16
    ig, hg = mk(rows, 4 * hidden).detach(), mk(rows, 4 * hidden).detach()
    c_other = mk(rows, hidden).detach().to(other)
    assert not cells.gate_ops.gates_supported(ig, hg, c_other, 4)
    h_y, c_y = cells.lstm_pointwise(ig, hg, c_other)
    want_h, want_c = chain_lstm(ig, hg, c_other)
    assert torch.equal(h_y, want_h) and torch.equal(c_y, want_c)
    assert not cells.gate_ops.gates_supported(ig[:, :-8], hg, mk(rows, hidden), 4)
