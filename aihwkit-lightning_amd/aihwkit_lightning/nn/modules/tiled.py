"""State and methods shared by the layers that map a weight matrix onto analog tiles along its
input dimension: ``AnalogLinear`` directly, the convolution layers through their
``weight.view(out_channels, -1)``. Tile split, input-range state, the call into the HIP
operator, weight clipping and post-training quantisation follow the reference
(``nn/modules/linear.py:53-317``, ``nn/modules/conv.py:121-367``)."""
import math
from contextlib import contextmanager
from copy import deepcopy
from typing import List, Optional, Tuple

import torch
from torch import Tensor, no_grad

from .base import AnalogLayerBase
from .hip_utils import library as L
from .hip_utils.hip_linear import HipLinear, QUANT_IDS, check_supported
from .hip_utils.ops import OPS, direct
from ...exceptions import HipBackendError
from ...simulator.configs import WeightClipType, WeightQuantizationType


def get_split_sizes(size: int, split_max_size: int) -> List[int]:
    """Sizes of the K-tiles for ``size`` inputs with at most ``split_max_size`` per tile:
    ``ceil(size / max)`` tiles whose sizes differ by at most one, larger ones first
    (reference ``linear.py:155-170``)."""
    if split_max_size <= 0:
        return [size]
    n_splits = (size + split_max_size - 1) // split_max_size
    base, extra = divmod(size, n_splits)
    return [base + 1] * extra + [base] * (n_splits - extra)


class TiledAnalogLayer(AnalogLayerBase):
    """Mixin for a module with a ``weight`` whose 2-D view ``[out, in]`` is tiled along ``in``."""

    # pylint: disable=no-member, attribute-defined-outside-init, too-many-instance-attributes

    def weight_matrix(self) -> Tensor:
        """The weight as the ``[out_features, in_features]`` matrix the tiles are cut from."""
        return self.weight.view(self.weight.size(0), -1)

    def _setup_tiles(self, in_features: int, device, dtype) -> None:
        rpu_config = self.rpu_config
        if str(device) == "meta":
            device = "cpu"  # the small per-tile state is always materialised
        self.in_sizes = get_split_sizes(in_features, rpu_config.mapping.max_input_size)
        ends, acc = [], 0
        for size in self.in_sizes:
            acc += size
            ends.append(acc)
        # int32 tile ends straight from Python ints (never routed through the layer dtype)
        self.upper_end_of_slices = torch.tensor(ends, dtype=torch.int32, device=device)
        self.init_ir(
            init_value_ir=rpu_config.pre_post.input_range.init_value,
            init_value_counter=0,
            device=device,
            dtype=dtype,
        )
        self._init_learnable_clip(device, dtype)
        self.deprecation_adjustment()
        # Host-side view of "is the input-range data initialisation still running?":
        # None = unknown (ask the device once), True/False = known without a sync.
        self._ir_init_active: Optional[bool] = None
        self._ir_init_calls = 0

    def _init_learnable_clip(self, device, dtype) -> None:
        if self.rpu_config.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL:
            weight = self.weight_matrix().detach()
            if not weight.is_cuda:
                # plain bookkeeping on the host copy: per-tile per-channel abs-max
                parts = torch.split(weight.abs(), self.in_sizes, dim=1)
                init = torch.stack([p.amax(dim=1) for p in parts])
            else:
                init = OPS.sliced_absmax(weight, self.in_sizes, False)[0]
            self.init_learnable_weight_ranges(init_value=init, device=device, dtype=dtype)
        else:
            self.learnable_weight_clip = None  # type: ignore[assignment]

    def get_split_sizes(self, size: int, split_max_size: int) -> List[int]:
        """Method form of :func:`get_split_sizes` kept for API compatibility."""
        return get_split_sizes(size, split_max_size)

    # ------------------------------------------------------------------ forward
    def _init_phase_active(self) -> bool:
        """Whether a training forward must still run the input-range data initialisation.

        The per-tile counters live on the device. They advance by one per training forward
        (unless a batch has zero variance), so the host only looks at them when it cannot know:
        on the first call and when its own call count says the phase should be over.
        """
        ir_params = self.rpu_config.pre_post.input_range
        stored_range = ir_params.enable and (ir_params.fast_mode or not ir_params.dynamic)
        if not stored_range or ir_params.init_from_data <= 0:
            return False
        if self._ir_init_active is False:
            return False
        if self._ir_init_active is None or self._ir_init_calls >= ir_params.init_from_data:
            idx_min = float(self.input_range_update_idx.min().item())
            # a counter that is not finite (calibration leaves -inf, calibration.py:159) means
            # "the ranges are set": the initialisation from data is over
            self._ir_init_active = math.isfinite(idx_min) and idx_min < ir_params.init_from_data
            self._ir_init_calls = int(idx_min) if self._ir_init_active else 0
        return bool(self._ir_init_active)

    #: set by :meth:`frozen_weights`; None means "the weights may change between calls"
    _weight_cache = None

    @contextmanager
    def frozen_weights(self):
        """Promise that the weights do not change inside the block: what a call computes from the
        weights alone (per-tile abs-max, padded operand copies) is computed once and reused by
        the following calls. For callers that apply one layer many times in a row, like the steps
        of a recurrent sequence. Nothing is reused while a weight modifier is active."""
        outer = self._weight_cache
        if outer is None:
            self._weight_cache = {}
        try:
            yield self
        finally:
            self._weight_cache = outer

    # torch.compile does not trace into the operator: its host side draws seeds, keeps per-layer
    # state and calls the library through ctypes. It runs as an opaque eager call between the
    # compiled parts of a model (the custom ops it is made of carry fake kernels for callers
    # that trace them directly).
    @torch.compiler.disable
    def analog_mvm(self, rows: Tensor) -> Tensor:
        """``rows[..., in] @ weight_matrix^T + bias`` through the analog tile model."""
        init_active = self.training and self._init_phase_active()
        weight, bias = self.weight_matrix(), self.bias
        input_range, weight_clip = self.input_range, self.learnable_weight_clip
        if not torch.is_grad_enabled():
            # Nothing will be differentiated. The operator decides from its arguments'
            # requires_grad what to keep for a backward pass (the clamp mask, the quantised
            # input, the padded operands), and that flag ignores the grad mode.
            rows, weight, bias, input_range, weight_clip = (
                None if t is None else t.detach()
                for t in (rows, weight, bias, input_range, weight_clip)
            )
        out = HipLinear.apply(
            rows,
            weight,
            bias,
            input_range,
            self.input_range_update_idx,
            self.in_sizes,
            self.rpu_config,
            self.training,
            init_active,
            self.x_min,
            self.x_max,
            weight_clip,
            self._weight_cache,
        )
        if init_active:
            self._ir_init_calls += 1
        return out

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        super()._load_from_state_dict(
            state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs
        )
        if "rpu_config" in local_metadata:
            self.rpu_config = deepcopy(local_metadata["rpu_config"])
        self._ir_init_active = None

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        # pylint: disable=protected-access
        destination._metadata[prefix.split(".")[0]]["rpu_config"] = deepcopy(self.rpu_config)

    # ------------------------------------------------------------------ weights
    @classmethod
    def move_to_meta(cls, module):
        """Release a digital module's storage during conversion."""
        module.to(device="meta")

    def set_weights(self, weight: Tensor) -> None:
        """Copy ``weight`` into the layer."""
        assert (
            self.weight.shape == weight.shape
        ), f"weight shape mismatch. Got {weight.shape}, expected {self.weight.shape}"
        self.weight.data = weight.detach().clone()
        self._init_learnable_clip(weight.device, weight.dtype)

    def set_weights_and_biases(self, weight: Tensor, bias: Optional[Tensor] = None) -> None:
        """Copy ``weight`` and, if given, ``bias`` into the layer."""
        self.set_weights(weight)
        if bias is not None:
            assert (
                self.bias is not None and self.bias.shape == bias.shape
            ), f"bias shape mismatch. Got {bias.shape}, expected " \
               f"{None if self.bias is None else self.bias.shape}"
            self.bias.data = bias.detach().clone()

    def get_weights_and_biases(self) -> Tuple[Tensor, Optional[Tensor]]:
        """The weight and bias tensors."""
        return (self.weight, self.bias)

    def clip_weights(self) -> None:
        """Clamp the weight matrix at ``clip.sigma`` standard deviations (whole matrix or per
        row); called by ``AnalogOptimizer`` after every step (reference ``linear.py:269-283``,
        ``conv.py:647-663``)."""
        clip_type = self.rpu_config.clip.type
        if clip_type in (WeightClipType.NONE, WeightClipType.LEARNABLE_PER_CHANNEL):
            return
        sigma = self.rpu_config.clip.sigma
        assert sigma > 0, "Clip sigma must be greater than 0"
        if clip_type == WeightClipType.LAYER_GAUSSIAN:
            kind = L.AHL_CLIP_LAYER
        elif clip_type == WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL:
            kind = L.AHL_CLIP_PER_CHANNEL
        else:
            raise ValueError(f"Unknown clip type {clip_type}")
        self._require_device("clip_weights")
        # called after every optimizer step of every layer and never traced: no dispatcher hop
        weights = self.weight_matrix().data
        direct(weights).clip_weights(weights, float(sigma), kind)

    @no_grad()
    def quantize_weights(self) -> None:
        """Quantise the weights in place, tile by tile, then switch the on-the-fly quantiser
        and the clipping off (reference ``linear.py:285-303``, ``conv.py:267-288`` +
        ``base.py:208-212``)."""
        check_supported(self.rpu_config)
        quant_type = self.rpu_config.modifier.quantization_type
        if self.rpu_config.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL:
            # the learned clip is the clamp (no quantiser) or the quantiser's range: what the
            # training forward applies on the fly, written back (quant_utils.py:184-233)
            assert self.learnable_weight_clip is not None, "learnable_weight_clip should not be None"
            self._require_device("quantize_weights")
            quantised = QUANT_IDS[quant_type] != L.AHL_QUANT_NONE
            w_new = OPS.weight_prep_clip(
                self.weight_matrix().data, self.learnable_weight_clip.data, self.in_sizes,
                L.AHL_QUANT_DISCRETIZE_PER_CHANNEL if quantised else L.AHL_QUANT_CLIP_LEARNED,
                L.AHL_NOISE_NONE, float(self.rpu_config.modifier.res) if quantised else 1.0, 0.0, 0, 0,
            )[2]
            self.weight_matrix().data.copy_(w_new)
        elif quant_type != WeightQuantizationType.NONE:
            self._require_device("quantize_weights")
            weights = self.weight_matrix().data
            direct(weights).quantize_weights(weights, self.in_sizes, QUANT_IDS[quant_type],
                                             float(self.rpu_config.modifier.res))
        super().quantize_weights()

    def _require_device(self, what: str) -> None:
        if not self.weight.is_cuda:
            raise HipBackendError(f"{what} needs the layer on a ROCm device; there is no CPU path")
        if not self.weight.is_contiguous():
            raise HipBackendError(f"{what} needs a contiguous weight")
