"""Pins the recurrent-network oracle: torch's own RNN / LSTM / GRU (independent library routines)
with the non-idealities off, and vectors written by the real reference."""
import os

import numpy as np
import pytest
import torch

from golden_cases import DTYPES
from helpers import assert_close_lsb, oracle_cfg
from oracle import rnn_mode as orn
from oracle import torch_mode as om
from rnn_cases import RNN_CASES, cell_slots, make_rnn_inputs, projections, scalar_loss

RNN_GOLDEN = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                       "rnn_cases.npz")))
TORCH_LAYER = {"rnn": torch.nn.RNN, "lstm": torch.nn.LSTM, "gru": torch.nn.GRU}


def oracle_run(case):
    """Oracle forward (+ backward in training mode) of a case; dict keyed like the fixtures."""
    dtype = DTYPES[case["dtype"]]
    x, params, states, g = make_rnn_inputs(case)
    cfg = oracle_cfg(case)
    cells = []
    for (layer, _), cell_params in zip(cell_slots(case), params):
        cell = {}
        for proj, (w, b) in cell_params.items():
            n_tiles = len(om.split_sizes(projections(case, layer)[proj][0], case["max_input_size"]))
            ir = (torch.full((n_tiles,), case["ir_init"], dtype=dtype)
                  if case["ir_mode"] in ("static", "fast") else None)
            cell[proj] = orn.Projection(w, b, ir)
        cells.append(cell)
    x3 = (x if case["batch"] > 0 else x.unsqueeze(1)).clone().requires_grad_(True)
    out, last = orn.rnn_forward(case["cell"], x3, cells, cfg, case["training"], case["layers"],
                                case["bidir"], states)
    res = {"out": out.detach()}
    for i, (hx, cx) in enumerate(last):
        res[f"h{i}"] = hx.detach()
        if cx is not None:
            res[f"c{i}"] = cx.detach()
    if case["training"]:
        scalar_loss(out, last, g).backward()
        res["dx"] = x3.grad.reshape(x.shape)
        for i, cell in enumerate(cells):
            for proj, p in cell.items():
                res[f"{i}/{proj}/dw"] = p.weight.grad
                if p.bias is not None:
                    res[f"{i}/{proj}/db"] = p.bias.grad
                if p.input_range is not None and p.input_range.grad is not None:
                    res[f"{i}/{proj}/dir"] = p.input_range.grad
    return res


def golden_of(case):
    prefix = case["name"] + "/"
    return {k[len(prefix):]: torch.from_numpy(v) for k, v in RNN_GOLDEN.items()
            if k.startswith(prefix)}


PLAIN = [c for c in RNN_CASES if c["name"].endswith("_plain")]


@pytest.mark.parametrize("case", PLAIN, ids=[c["name"] for c in PLAIN])
def test_plain_network_is_torchs_recurrent_layer(case):
    """Without non-idealities the oracle is torch.nn.RNN / LSTM / GRU: outputs, last states and
    every gradient. A wrong gate order, direction wiring or state hand-over fails here."""
    x, params, _, g = make_rnn_inputs(case)
    layer = TORCH_LAYER[case["cell"]](case["inputs"], case["hidden"], case["layers"],
                                      bias=case["bias"], bidirectional=case["bidir"])
    with torch.no_grad():
        for (lay, d), cell_params in zip(cell_slots(case), params):
            tag = f"l{lay}" + ("_reverse" if d == 1 else "")
            for part in ("ih", "hh"):
                w, b = cell_params[f"weight_{part}"]
                getattr(layer, f"weight_{part}_{tag}").copy_(w)
                if b is not None:
                    getattr(layer, f"bias_{part}_{tag}").copy_(b)
    xin = x.clone().requires_grad_(True)
    out, last = layer(xin)
    h_n = last[0] if case["cell"] == "lstm" else last
    c_n = last[1] if case["cell"] == "lstm" else None
    states = [(h_n[i], None if c_n is None else c_n[i]) for i in range(h_n.size(0))]
    scalar_loss(out, states, g).backward()
    got = oracle_run(case)
    assert torch.allclose(got["out"], out, rtol=1e-5, atol=1e-6)
    assert torch.allclose(got["dx"], xin.grad, rtol=1e-4, atol=1e-5)
    for i, ((lay, d), cell_params) in enumerate(zip(cell_slots(case), params)):
        tag = f"l{lay}" + ("_reverse" if d == 1 else "")
        assert torch.allclose(got[f"h{i}"], states[i][0], rtol=1e-5, atol=1e-6)
        if c_n is not None:
            assert torch.allclose(got[f"c{i}"], states[i][1], rtol=1e-5, atol=1e-6)
        for part in ("ih", "hh"):
            want = getattr(layer, f"weight_{part}_{tag}").grad
            assert torch.allclose(got[f"{i}/weight_{part}/dw"], want, rtol=1e-4, atol=1e-5), (i, part)
            if case["bias"]:
                want = getattr(layer, f"bias_{part}_{tag}").grad
                assert torch.allclose(got[f"{i}/weight_{part}/db"], want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("case", RNN_CASES, ids=[c["name"] for c in RNN_CASES])
def test_oracle_matches_the_reference_vectors(case):
    """Outputs, last states and all gradients against the real reference."""
    got, want = oracle_run(case), golden_of(case)
    assert set(got) == set(want), set(got) ^ set(want)
    bf16 = case["dtype"] == "bf16"
    for key, ref in want.items():
        val = got[key].float().reshape(ref.shape)
        if bf16:
            assert_close_lsb(val, ref, 1e-2, lsb=None, what=f"{case['name']}/{key}")
        else:
            assert_close_lsb(val, ref, 1e-5, lsb=None, what=f"{case['name']}/{key}")
