"""The paths a user of the reference walks, end to end on the GPU: convert a digital model with
linear, convolution and recurrent layers and train it with ``AnalogOptimizer`` under noise, evaluate,
save and reload the state dict, convert back; or convert a trained digital model for inference,
calibrate its input ranges from data and switch the converters on (reference README /
``tests/test_conversion.py``, ``optim/analog_optimizer.py``, ``inference/calibration``)."""
import io

import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu


class Net(nn.Module):
    """conv -> pool -> LSTM over image rows -> linear head."""

    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(3, 8, 3, padding=1)
        self.lstm = nn.LSTM(8 * 8, 32, 1)
        self.head = nn.Sequential(nn.Linear(32, 64), nn.ReLU(), nn.Linear(64, 10))

    def forward(self, img):
        feat = torch.relu(self.conv(img))                     # [B, 8, 16, 16]
        feat = nn.functional.avg_pool2d(feat, 2)              # [B, 8, 8, 8]
        seq = feat.permute(2, 0, 1, 3).reshape(8, img.size(0), 64)   # rows as time steps
        out, _ = self.lstm(seq)
        return self.head(out[-1])


def _config():
    from aihwkit_lightning.simulator.configs import (TorchInferenceRPUConfig, WeightClipType,
                                                     WeightNoiseInjectionType)
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 32
    cfg.forward.inp_res = 254
    cfg.forward.out_res = 254
    cfg.forward.out_bound = 12.0
    cfg.forward.out_noise = 0.02
    cfg.clip.type = WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
    cfg.clip.sigma = 3.0
    cfg.modifier.noise_type = WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL
    cfg.modifier.std_dev = 0.02
    cfg.pre_post.input_range.enable = True
    cfg.pre_post.input_range.init_from_data = 5
    cfg.pre_post.input_range.init_std_alpha = 3.0
    return cfg


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_convert_train_save_load_convert_back(dtype):
    from aihwkit_lightning.nn import AnalogConv2d, AnalogLinear, AnalogRNN
    from aihwkit_lightning.nn.conversion import convert_to_analog, convert_to_digital
    from aihwkit_lightning.optim import AnalogOptimizer

    torch.manual_seed(0)
    gen = torch.Generator().manual_seed(1)
    # four classes: a fixed random pattern per class under unit noise
    patterns = torch.randn(4, 3, 16, 16, generator=gen)
    labels = torch.randint(0, 4, (256,), generator=gen)
    images = 0.8 * patterns[labels] + torch.randn(256, 3, 16, 16, generator=gen)
    images, labels = images.to("cuda", dtype), labels.cuda()

    digital = Net().to("cuda", dtype)
    model = convert_to_analog(digital, _config())
    kinds = {type(m) for m in model.modules()}
    assert {AnalogConv2d, AnalogRNN, AnalogLinear} <= kinds
    n_analog = len(list(model.analog_layers()))
    assert n_analog == 5  # conv, two LSTM projections, two linear layers

    optim = AnalogOptimizer(torch.optim.Adam, model.analog_layers, model.parameters(), lr=3e-3)
    model.train()
    losses = []
    for step in range(100):
        idx = torch.randperm(256, generator=gen)[:64].cuda()
        optim.zero_grad()
        loss = nn.functional.cross_entropy(model(images[idx]).float(), labels[idx])
        loss.backward()
        optim.step()
        losses.append(float(loss.detach()))
    assert all(torch.isfinite(torch.tensor(losses)))
    assert sum(losses[-10:]) / 10 < 0.8 * sum(losses[:5]) / 5, losses
    for layer in model.analog_layers():   # the ranges were initialised from data and then learned
        assert int(layer.input_range_update_idx.min()) >= 5
        assert layer.input_range.grad is not None

    model.eval()
    # evaluation is deterministic, accurate on the training data, and survives a state-dict trip
    with torch.no_grad():
        out = model(images)
        assert torch.equal(out, model(images))
    accuracy = float((out.argmax(1) == labels).float().mean())
    assert accuracy > 0.75, accuracy
    buffer = io.BytesIO()
    torch.save(model.state_dict(), buffer)
    buffer.seek(0)
    fresh = convert_to_analog(Net().to("cuda", dtype), _config())
    fresh.load_state_dict(torch.load(buffer, weights_only=False))
    fresh.eval()
    with torch.no_grad():
        assert torch.equal(fresh(images), out)

    # back to digital: same weights, and (noise and quantisers gone) nearly the same predictions
    back = convert_to_digital(model)
    assert isinstance(back, Net) and isinstance(back.lstm, nn.LSTM)
    with torch.no_grad():
        agree = float((back(images).argmax(1) == out.argmax(1)).float().mean())
    assert agree > 0.9, agree


@pytest.mark.parametrize("strategy", ["MAX", "MOVING_STD", "CACHE_QUANTILE"])
def test_post_training_calibration_then_8_bit_inference(strategy):
    """A digital model converted without input ranges, calibrated from data, then run with 8-bit
    converters: the analog predictions follow the digital ones."""
    from aihwkit_lightning.inference.calibration import (InputRangeCalibrationType,
                                                         calibrate_input_ranges)
    from aihwkit_lightning.nn.conversion import convert_to_analog
    from aihwkit_lightning.simulator.configs import TorchInferenceRPUConfig

    torch.manual_seed(3)
    gen = torch.Generator().manual_seed(4)
    images = torch.randn(256, 3, 16, 16, generator=gen).cuda()
    digital = Net().cuda().eval()
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 32
    model = convert_to_analog(digital, cfg).eval()
    with torch.no_grad():
        want = digital(images)
        assert torch.allclose(model(images), want, rtol=1e-4, atol=1e-5)  # no non-idealities yet
    calibrate_input_ranges(
        model, InputRangeCalibrationType[strategy],
        (((images[i:i + 64],), {}) for i in range(0, 256, 64)), quantile=0.9999, max_samples=2000,
        std_alpha=4.0, verbose=False,
    )
    for layer in model.analog_layers():
        assert layer.rpu_config.pre_post.input_range.enable
        assert torch.isfinite(layer.input_range).all() and (layer.input_range > 0).all()
        layer.rpu_config.forward.inp_res = 254
        layer.rpu_config.forward.out_res = 254
        layer.rpu_config.forward.out_bound = 12.0
    with torch.no_grad():
        got = model(images)
    assert not torch.equal(got, want)
    rel = float((got - want).norm() / want.norm())
    assert rel < 0.1, rel
    assert float((got.argmax(1) == want.argmax(1)).float().mean()) > 0.9


def test_tiny_llama_converts_trains_and_generates():
    """The reference's main use: a Hugging Face decoder converted layer by layer and fine-tuned in
    bf16. Covers tiles of 256 inputs, an intermediate size that is no multiple of the tile, a
    vocabulary that is no multiple of 8, and ``generate`` (one row per call)."""
    transformers = pytest.importorskip("transformers")
    from aihwkit_lightning.nn.conversion import convert_to_analog, convert_to_digital
    from aihwkit_lightning.optim import AnalogOptimizer

    conf = transformers.LlamaConfig(vocab_size=1003, hidden_size=256, intermediate_size=688,
                                    num_hidden_layers=2, num_attention_heads=4,
                                    num_key_value_heads=4, max_position_embeddings=128)
    torch.manual_seed(0)
    llm = transformers.LlamaForCausalLM(conf).to("cuda", torch.bfloat16)
    cfg = _config()
    cfg.mapping.max_input_size = 256
    model = convert_to_analog(llm, cfg)
    assert len(list(model.analog_layers())) == 2 * 7 + 1  # q, k, v, o, gate, up, down; lm_head
    ids = torch.randint(0, 1003, (4, 64), generator=torch.Generator().manual_seed(2)).cuda()
    optim = AnalogOptimizer(torch.optim.AdamW, model.analog_layers, model.parameters(), lr=1e-3)
    model.train()
    losses = []
    for _ in range(12):
        optim.zero_grad()
        loss = model(input_ids=ids, labels=ids).loss
        loss.backward()
        optim.step()
        losses.append(float(loss.detach()))
    assert all(v == v for v in losses) and losses[-1] < 0.8 * losses[0], losses
    model.eval()
    with torch.no_grad():
        generated = model.generate(ids[:, :8], attention_mask=torch.ones_like(ids[:, :8]),
                                   max_new_tokens=8, do_sample=False, pad_token_id=0)
    assert generated.shape == (4, 16)
    assert type(convert_to_digital(model)).__name__ == "LlamaForCausalLM"
