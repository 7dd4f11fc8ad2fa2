"""Recurrent-network cases shared by the fixture writer (``make_golden_rnn.py``) and the tests.

Every case is a golden-case dict of ``golden_cases.py`` (same configuration keys; ``M``, ``K``,
``N`` unused) plus ``cell`` ("rnn", "lstm", "gru" or "lstm_combined"), ``steps``, ``batch`` (0 =
one unbatched sequence), ``inputs`` (feature size), ``hidden``, ``layers``, ``bidir`` and
``random_state`` (start from a random instead of the all-zero state). Inputs, weights and the
output gradient are regenerated from seeds.
"""
import torch

from golden_cases import DEFAULTS, DTYPES

_ADC8 = dict(inp_res=254, out_res=254, out_bound=10.0)
GATES = {"rnn": 1, "lstm": 4, "gru": 3, "lstm_combined": 4}


def rnn_case(name, cell, steps, batch, inputs, hidden, layers=1, bidir=False, random_state=False,
             **kw):
    out = dict(DEFAULTS)
    unknown = set(kw) - set(DEFAULTS)
    assert not unknown, unknown
    out.update(kw)
    out.update(name=name, cell=cell, steps=steps, batch=batch, inputs=inputs, hidden=hidden,
               layers=layers, bidir=bidir, random_state=random_state)
    return out


_ANALOG = dict(ir_mode="static", ir_init=2.0, clip="channel", clip_sigma=2.5, ir_decay=0.01,
               w_scale=0.3, **_ADC8)

RNN_CASES = [
    # no non-idealities: must equal torch's own recurrent layers
    rnn_case("rnn_f32_plain", "rnn", 5, 3, 6, 8, layers=2, w_scale=0.3, seed=50),
    rnn_case("lstm_f32_plain", "lstm", 5, 3, 6, 8, layers=2, bidir=True, w_scale=0.3, seed=51),
    rnn_case("gru_f32_plain", "gru", 5, 3, 6, 8, layers=2, bidir=True, bias=False, w_scale=0.3,
             seed=52),
    # analog tiles (two per projection of the first layer), learned input range, 8-bit converters
    rnn_case("lstm_f32_adc", "lstm", 4, 3, 10, 8, layers=2, max_input_size=6, seed=53, **_ANALOG),
    rnn_case("lstm_bf16_adc", "lstm", 4, 3, 10, 8, layers=2, max_input_size=6, dtype="bf16",
             seed=53, **_ANALOG),
    rnn_case("gru_f32_adc_bidir", "gru", 4, 2, 10, 8, layers=2, bidir=True, max_input_size=6,
             seed=54, **_ANALOG),
    rnn_case("gru_bf16_adc", "gru", 4, 2, 10, 8, max_input_size=6, dtype="bf16", seed=54,
             **_ANALOG),
    rnn_case("rnn_f32_adc_bidir", "rnn", 6, 2, 10, 8, bidir=True, max_input_size=6, seed=55,
             **_ANALOG),
    # given initial states (the reference accepts them for cells with a cell state only)
    rnn_case("lstm_f32_adc_bidir_state", "lstm", 4, 2, 10, 8, layers=2, bidir=True,
             max_input_size=6, random_state=True, seed=60, **_ANALOG),
    rnn_case("lstm_combined_f32_adc", "lstm_combined", 4, 3, 10, 8, max_input_size=6, seed=56,
             **_ANALOG),
    # evaluation mode (the input projection of all steps may be computed ahead of the loop),
    # per-row dynamic input range, one unbatched sequence
    rnn_case("lstm_f32_eval_dynamic", "lstm", 6, 3, 10, 8, layers=2, bidir=True, max_input_size=6,
             ir_mode="dynamic", clip="channel", clip_sigma=2.5, w_scale=0.3, training=False,
             seed=57, **_ADC8),
    rnn_case("gru_bf16_eval", "gru", 6, 3, 10, 8, layers=2, max_input_size=6, dtype="bf16",
             training=False, seed=58, **_ANALOG),
    rnn_case("lstm_f32_unbatched", "lstm", 5, 0, 10, 8, max_input_size=6, seed=59, **_ANALOG),
]

RNN_CASES_BY_NAME = {c["name"]: c for c in RNN_CASES}


def cell_slots(c):
    """``(layer, direction)`` of every cell in module order."""
    dirs = (0, 1) if c["bidir"] else (0,)
    return [(layer, d) for layer in range(c["layers"]) for d in dirs]


def projections(c, layer):
    """``{name: (in_features, out_features)}`` of the projections of one cell of ``layer``."""
    fan_in = c["inputs"] if layer == 0 else c["hidden"] * (2 if c["bidir"] else 1)
    width = GATES[c["cell"]] * c["hidden"]
    if c["cell"] == "lstm_combined":
        return {"weight": (fan_in + c["hidden"], width)}
    return {"weight_ih": (fan_in, width), "weight_hh": (c["hidden"], width)}


def make_rnn_inputs(c):
    """``x [steps, batch, inputs]`` (``[steps, inputs]`` unbatched), per-cell parameters (list in
    module order of ``{projection: (weight, bias or None)}``), initial states (list in module
    order of ``(hx, cx or None)``, or None for the all-zero state) and the gradient of the
    output, all in the case's dtype."""
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(3000 + c["seed"])
    lead = (c["steps"], c["batch"]) if c["batch"] > 0 else (c["steps"],)
    x = (torch.randn(*lead, c["inputs"], generator=gen) * c["x_scale"]).to(dtype)
    params = []
    for layer, _ in cell_slots(c):
        cell = {}
        for name, (fan_in, width) in projections(c, layer).items():
            w = (torch.randn(width, fan_in, generator=gen) * c["w_scale"]).to(dtype)
            b = (torch.randn(width, generator=gen) * 0.1).to(dtype) if c["bias"] else None
            cell[name] = (w, b)
        params.append(cell)
    states = None
    if c["random_state"]:
        rows = max(c["batch"], 1)
        has_cx = c["cell"].startswith("lstm")
        states = []
        for _ in cell_slots(c):
            hx = (torch.randn(rows, c["hidden"], generator=gen) * 0.5).to(dtype)
            cx = (torch.randn(rows, c["hidden"], generator=gen) * 0.5).to(dtype) if has_cx else None
            states.append((hx, cx))
    fan_out = c["hidden"] * (2 if c["bidir"] else 1)
    g = torch.randn(*lead, fan_out, generator=gen).to(dtype)
    return x, params, states, g


def scalar_loss(out, last_states, g):
    """The scalar both sides differentiate: the output weighted by ``g`` plus a quarter of the
    sum of every last hidden state and an eighth of every last cell state, so that the gradient
    also flows through the returned states."""
    loss = (out * g.reshape(out.shape)).sum()
    for hx, cx in last_states:
        loss = loss + hx.sum() * 0.25
        if cx is not None:
            loss = loss + cx.sum() * 0.125
    return loss
