"""Writes ``rnn_cases.npz`` by RUNNING THE REFERENCE's ``AnalogRNN`` on the CPU.

Run once, in the build container, where the reference is mounted read-only:

    PYTHONPATH=/root/reference/src python tests/golden/make_golden_rnn.py

Evaluates ``RNN_CASES`` (torch-mode, CPU, fixed seeds) and stores the outputs, the last states and
all gradients (bf16 as float32, which holds it exactly). Only data is written. The fixtures pin
the gate order inside the stacked projections, the direction and layer wiring, the state
hand-over between steps and the gradients through the recurrence.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from golden_cases import DTYPES  # noqa: E402  pylint: disable=wrong-import-position
from make_golden import f32, ref_config  # noqa: E402  pylint: disable=wrong-import-position
from rnn_cases import RNN_CASES, cell_slots, make_rnn_inputs, scalar_loss  # noqa: E402  pylint: disable=wrong-import-position

from aihwkit_lightning.nn import (  # noqa: E402  (the reference)
    AnalogGRUCell, AnalogLSTMCell, AnalogLSTMCellCombinedWeight, AnalogRNN, AnalogVanillaRNNCell,
)
from aihwkit_lightning.nn.modules.rnn.cells import LSTMState  # noqa: E402

CELLS = {"rnn": AnalogVanillaRNNCell, "lstm": AnalogLSTMCell, "gru": AnalogGRUCell,
         "lstm_combined": AnalogLSTMCellCombinedWeight}


def cell_modules(net, case):
    """The cell modules in module order."""
    out = []
    for layer, d in cell_slots(case):
        mod = net.rnn.layers[layer]
        out.append(mod.directions[d].cell if case["bidir"] else mod.cell)
    return out


def run_case(case, store):
    name, dtype = case["name"], DTYPES[case["dtype"]]
    x, params, states, g = make_rnn_inputs(case)
    net = AnalogRNN(CELLS[case["cell"]], case["inputs"], case["hidden"], case["layers"],
                    bias=case["bias"], bidir=case["bidir"], dtype=dtype,
                    rpu_config=ref_config(case))
    cells = cell_modules(net, case)
    for cell, cell_params in zip(cells, params):
        for proj, (w, b) in cell_params.items():
            getattr(cell, proj).set_weights_and_biases(w, b)
    net.train(case["training"])
    ref_states = None
    if states is not None:
        flat = [LSTMState(h if case["batch"] > 0 else h[0],
                          None if c is None else (c if case["batch"] > 0 else c[0]))
                for h, c in states]
        ref_states = ([tuple(flat[2 * i:2 * i + 2]) for i in range(case["layers"])]
                      if case["bidir"] else flat)
    xin = x.clone().requires_grad_(True)
    torch.manual_seed(case["noise_seed"])
    out, last = net(xin, ref_states)
    last_flat = [s for pair in last for s in pair] if case["bidir"] else list(last)
    last_flat = [(s[0], s[1]) for s in last_flat]
    store[f"{name}/out"] = f32(out)
    for i, (hx, cx) in enumerate(last_flat):
        store[f"{name}/h{i}"] = f32(hx)
        if cx is not None:
            store[f"{name}/c{i}"] = f32(cx)
    if not case["training"]:
        return
    scalar_loss(out, last_flat, g).backward()
    store[f"{name}/dx"] = f32(xin.grad)
    for i, (cell, cell_params) in enumerate(zip(cells, params)):
        for proj in cell_params:
            lin = getattr(cell, proj)
            store[f"{name}/{i}/{proj}/dw"] = f32(lin.weight.grad)
            if lin.bias is not None:
                store[f"{name}/{i}/{proj}/db"] = f32(lin.bias.grad)
            if lin.input_range is not None and lin.input_range.grad is not None:
                store[f"{name}/{i}/{proj}/dir"] = f32(lin.input_range.grad)


def main():
    store = {}
    for case in RNN_CASES:
        run_case(case, store)
        print("done", case["name"])
    path = os.path.join(HERE, "rnn_cases.npz")
    np.savez_compressed(path, **store)
    print(f"wrote {path}: {os.path.getsize(path) / 1e3:.1f} kB, {len(store)} arrays")


if __name__ == "__main__":
    main()
