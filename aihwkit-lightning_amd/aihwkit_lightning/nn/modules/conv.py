"""``AnalogConv1d/2d/3d``: convolutions whose patch-by-kernel product runs on analog tiles.

A convolution is the AnalogLinear operator applied to the patches of the input: patches are the
rows, ``weight.view(out_channels, -1)`` is the tiled matrix (reference ``nn/modules/conv.py``:
``_AnalogConvNd`` :121-367, ``AnalogConv1d`` :370-512, ``AnalogConv2d`` :515-677,
``AnalogConv3d`` :680-945). Patch extraction, its adjoint and the layout change of the result are
HIP kernels behind the same C ABI as the operator; this module only strings them together.
"""
from functools import reduce
from typing import List, Optional, Tuple, Union

import torch
from torch import Tensor
from torch.autograd import Function
from torch.nn import Conv1d, Conv2d, Conv3d
from torch.nn.modules.conv import _ConvNd
from torch.nn.modules.utils import _pair, _single, _triple

from .hip_utils.hip_conv import HipConv, direct_conv_applies
from .hip_utils.ops import OPS, conv_out_size
from .linear import is_at_least_volta_gpu  # noqa: F401  (re-exported)
from .tiled import TiledAnalogLayer
from ...exceptions import HipBackendError
from ...simulator.configs import TorchInferenceRPUConfig


class PatchRows(Function):
    """``x [B, C, D, H, W] -> patches [B, L, C * kD * kH * kW]``; the gradient folds the patch
    gradients back onto the input."""

    # pylint: disable=abstract-method, arguments-differ

    @staticmethod
    def forward(ctx, inp: Tensor, geom: List[int]) -> Tensor:
        ctx.geom = geom
        ctx.inp_shape = inp.shape
        return OPS.im2col(inp, geom)

    @staticmethod
    def backward(ctx, grad: Tensor):
        return OPS.col2im(grad, ctx.geom).view(ctx.inp_shape), None


class SwapLastTwo(Function):
    """``[B, R, C] -> [B, C, R]`` as a contiguous tensor, in both directions."""

    # pylint: disable=abstract-method, arguments-differ

    @staticmethod
    def forward(ctx, inp: Tensor) -> Tensor:
        return OPS.transpose_batched(inp)

    @staticmethod
    def backward(ctx, grad: Tensor):
        return OPS.transpose_batched(grad)


def unfold3d(
    inp: Tensor,
    kernel_size: Tuple[int, int, int],
    padding: Tuple[int, int, int] = (0, 0, 0),
    stride: Tuple[int, int, int] = (1, 1, 1),
) -> Tensor:
    """Patches of a volume in ``torch.nn.functional.unfold``'s layout:
    ``[B, C, D, H, W] -> [B, C * kD * kH * kW, L]`` (``[C, D, H, W] -> [C * kD * kH * kW, L]``
    without a batch), dilation 1 (reference ``nn/modules/conv.py``: ``unfold3d``). One patch
    kernel launch and one transpose; differentiable."""
    unbatched = inp.dim() == 4
    if unbatched:
        inp = inp.unsqueeze(0)
    if inp.dim() != 5:
        raise ValueError("expected a 4-D or 5-D input")
    if not inp.is_cuda:
        raise HipBackendError("patch extraction runs on a ROCm device; there is no CPU path")
    geom = (
        [int(inp.shape[0]), int(inp.shape[1])]
        + [int(v) for v in inp.shape[2:]]
        + [int(v) for v in _triple(kernel_size)]
        + [int(v) for v in _triple(stride)]
        + [int(v) for v in _triple(padding)]
        + [1, 1, 1]
    )
    cols = SwapLastTwo.apply(PatchRows.apply(inp.contiguous(), geom))
    return cols.squeeze(0) if unbatched else cols


def _three(values: Tuple[int, ...], fill: int) -> List[int]:
    """Pad a 1-, 2- or 3-tuple on the left to three entries."""
    values = tuple(int(v) for v in values)
    return [fill] * (3 - len(values)) + list(values)


class _AnalogConvNd(TiledAnalogLayer, _ConvNd):
    """Common part of the analog convolutions: geometry checks, tile set-up, forward."""

    # pylint: disable=abstract-method, too-many-arguments

    SPATIAL_DIMS = 2

    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: Tuple[int, ...],
        stride: Tuple[int, ...],
        padding: Tuple[int, ...],
        dilation: Tuple[int, ...],
        transposed: bool,
        output_padding: Tuple[int, ...],
        groups: int,
        bias: bool,
        padding_mode: str,
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        if groups != 1:
            raise ValueError("Only one group is supported")
        if padding_mode != "zeros":
            raise ValueError('Only "zeros" padding mode is supported')
        if isinstance(padding, str):
            raise ValueError("Padding must be given as integers")
        assert rpu_config is not None, "RPU config must be provided"
        _ConvNd.__init__(
            self, in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
            output_padding, groups, bias, padding_mode, device, dtype,
        )
        self.rpu_config = rpu_config
        self.in_features = self.get_tile_size(in_channels, groups, kernel_size)
        self.out_features = out_channels
        self._setup_tiles(self.in_features, device, dtype)

    def get_tile_size(self, in_channels: int, groups: int, kernel_size: Tuple[int, ...]) -> int:
        """Patch length: input channels per group times the kernel volume."""
        return (in_channels // groups) * reduce(lambda x, y: x * y, kernel_size)

    def geometry(self, inp_shape: Tuple[int, ...]) -> List[int]:
        """``[batch, channels, in(3), kernel(3), stride(3), padding(3), dilation(3)]`` for a
        batched input shape ``[B, C, *spatial]`` (spatial dimensions as stored by the layer)."""
        spatial = tuple(inp_shape[2:])
        if len(spatial) != len(self.kernel_size) or inp_shape[1] != self.in_channels:
            raise ValueError(
                f"input of shape {tuple(inp_shape)} does not fit a convolution over "
                f"{self.in_channels} channels with kernel {self.kernel_size}"
            )
        return (
            [int(inp_shape[0]), int(inp_shape[1])]
            + _three(spatial, 1)
            + _three(self.kernel_size, 1)
            + _three(self.stride, 1)
            + _three(self.padding, 0)
            + _three(self.dilation, 1)
        )

    def _batched(self, inp: Tensor) -> Tuple[Tensor, bool]:
        if not inp.is_cuda:
            raise HipBackendError("analog convolutions run on a ROCm device; there is no CPU path")
        n_spatial = len(self.kernel_size)
        unbatched = inp.dim() == n_spatial + 1
        if unbatched:
            inp = inp.unsqueeze(0)
        if inp.dim() != n_spatial + 2:
            raise ValueError(f"expected a {n_spatial + 1}-D or {n_spatial + 2}-D input")
        return inp, unbatched

    def patch_rows(self, inp: Tensor) -> Tensor:
        """The rows the tiles see for ``inp``: its patches ``[B, L, in_features]``."""
        inp, _ = self._batched(inp)
        return PatchRows.apply(inp, self.geometry(tuple(inp.shape)))

    def forward(self, inp: Tensor) -> Tensor:  # pylint: disable=arguments-renamed
        """Convolution of ``inp [B, C, *spatial]`` (or unbatched ``[C, *spatial]``)."""
        inp, unbatched = self._batched(inp)
        n_spatial = len(self.kernel_size)
        geom = self.geometry(tuple(inp.shape))
        out_size = conv_out_size(geom)[3 - n_spatial:]
        if direct_conv_applies(self, inp, geom, self.training and self._init_phase_active()):
            # the three products read the (padded, channels-last) image itself: no patch matrix
            out = self._conv_on_the_image(inp, geom).view(geom[0], self.out_channels, *out_size)
            return out.squeeze(0) if unbatched else out
        rows = PatchRows.apply(inp, geom)  # [B, L, K]
        out = self.analog_mvm(rows)  # [B, L, N]
        out = SwapLastTwo.apply(out)  # [B, N, L]
        out = out.view(geom[0], self.out_channels, *out_size)
        return out.squeeze(0) if unbatched else out

    @torch.compiler.disable
    def _conv_on_the_image(self, inp: Tensor, geom: List[int]) -> Tensor:
        weight, bias, input_range = self.weight_matrix(), self.bias, self.input_range
        if not torch.is_grad_enabled():   # see TiledAnalogLayer.analog_mvm
            inp, weight, bias, input_range = (None if t is None else t.detach()
                                              for t in (inp, weight, bias, input_range))
        return HipConv.apply(inp, weight, bias, input_range, self.in_sizes, self.rpu_config,
                             self.training, geom)

    @classmethod
    def _from_digital(cls, module: _ConvNd, rpu_config: TorchInferenceRPUConfig, weight: Tensor):
        layer = cls(
            module.in_channels, module.out_channels, module.kernel_size, module.stride,
            module.padding, module.dilation, module.groups, module.bias is not None,
            module.padding_mode, None, None, rpu_config,
        )
        layer.set_weights_and_biases(weight, module.bias)
        return layer.to(device=module.weight.device, dtype=module.weight.dtype)

    @staticmethod
    def _to_digital(digital: _ConvNd, module: "_AnalogConvNd", weight: Tensor) -> _ConvNd:
        digital.weight.data = weight.detach().clone()
        if module.bias is not None:
            assert digital.bias is not None, "Bias must be present"
            digital.bias.data = module.bias.data.detach().clone()
        return digital.to(device=module.weight.device, dtype=module.weight.dtype)


class AnalogConv1d(_AnalogConvNd):
    """1-d convolution on analog tiles. Like the reference, the layer stores its weight as a
    2-d kernel of height one (``[out, in, 1, k]``) and converts state dicts to and from the
    ``nn.Conv1d`` shape, so checkpoints stay interchangeable with ``nn.Conv1d``."""

    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: Union[int, Tuple[int]],
        stride: Union[int, Tuple[int]] = 1,
        padding: Union[int, Tuple[int]] = 0,
        dilation: Union[int, Tuple[int]] = 1,
        groups: int = 1,
        bias: bool = True,
        padding_mode: str = "zeros",
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        # pylint: disable=too-many-arguments
        if isinstance(padding, str):
            raise ValueError("Padding must be given as integers")
        kernel_size, stride = _single(kernel_size), _single(stride)
        padding, dilation = _single(padding), _single(dilation)
        if dilation != _single(1):
            raise ValueError("Only dilation = 1 is supported")
        super().__init__(
            in_channels, out_channels, (1, kernel_size[0]), (1, stride[0]), (0, padding[0]),
            (1, dilation[0]), False, _pair(0), groups, bias, padding_mode, device, dtype,
            rpu_config,
        )
        self._register_load_state_dict_pre_hook(self.update_state_dict)
        self._register_state_dict_hook(self.return_pytorch_state_dict)
        self.tensor_view = (-1, 1)

    def forward(self, inp: Tensor) -> Tensor:
        return super().forward(inp.unsqueeze(-2)).squeeze(-2)

    def patch_rows(self, inp: Tensor) -> Tensor:
        return super().patch_rows(inp.unsqueeze(-2))

    @classmethod
    def from_digital(cls, module: Conv1d, rpu_config: TorchInferenceRPUConfig) -> "AnalogConv1d":
        """Analog layer with the weights (and bias) of an ``nn.Conv1d``."""
        return cls._from_digital(module, rpu_config, module.weight.unsqueeze(-2))

    @classmethod
    def to_digital(cls, module: "AnalogConv1d") -> Conv1d:
        """``nn.Conv1d`` with the same weights."""
        digital = Conv1d(
            module.in_channels, module.out_channels, module.kernel_size[1], module.stride[1],
            module.padding[1], module.dilation[1], module.groups, module.bias is not None,
            module.padding_mode,
        )
        return cls._to_digital(digital, module, module.weight.data.squeeze(-2))

    def update_state_dict(self, state_dict, *args, **kwargs):  # pylint: disable=unused-argument
        """Loading: give ``nn.Conv1d``-shaped weights the stored height-one dimension."""
        for name, item in state_dict.items():
            if "weight" in name and item.dim() == 3:
                state_dict[name] = item.unsqueeze(-2)

    def return_pytorch_state_dict(self, module, state_dict, prefix, local_metadata):
        """Saving: write the weight in the ``nn.Conv1d`` shape."""
        # pylint: disable=unused-argument
        for name in [key for key in state_dict.keys() if prefix in key]:
            if "weight" in name and state_dict[name].dim() == 4:
                state_dict[name] = state_dict[name].squeeze(-2)


class AnalogConv2d(_AnalogConvNd):
    """2-d convolution on analog tiles."""

    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: Union[int, Tuple],
        stride: Union[int, Tuple] = 1,
        padding: Union[int, Tuple] = 0,
        dilation: Union[int, Tuple] = 1,
        groups: int = 1,
        bias: bool = True,
        padding_mode: str = "zeros",
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        # pylint: disable=too-many-arguments
        if isinstance(padding, str):
            raise ValueError("Padding must be given as integers")
        super().__init__(
            in_channels, out_channels, _pair(kernel_size), _pair(stride), _pair(padding),
            _pair(dilation), False, _pair(0), groups, bias, padding_mode, device, dtype,
            rpu_config,
        )

    @classmethod
    def from_digital(cls, module: Conv2d, rpu_config: TorchInferenceRPUConfig) -> "AnalogConv2d":
        """Analog layer with the weights (and bias) of an ``nn.Conv2d``."""
        return cls._from_digital(module, rpu_config, module.weight)

    @classmethod
    def to_digital(cls, module: "AnalogConv2d") -> Conv2d:
        """``nn.Conv2d`` with the same weights."""
        digital = Conv2d(
            module.in_channels, module.out_channels, module.kernel_size, module.stride,
            module.padding, module.dilation, module.groups, module.bias is not None,
            module.padding_mode,
        )
        return cls._to_digital(digital, module, module.weight.data)


class AnalogConv3d(_AnalogConvNd):
    """3-d convolution on analog tiles (dilation 1 only, as in the reference)."""

    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: Union[int, Tuple],
        stride: Union[int, Tuple] = 1,
        padding: Union[int, Tuple] = 0,
        dilation: Union[int, Tuple] = 1,
        groups: int = 1,
        bias: bool = True,
        padding_mode: str = "zeros",
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        # pylint: disable=too-many-arguments
        if isinstance(padding, str):
            raise ValueError("Padding must be given as integers")
        dilation = _triple(dilation)
        assert dilation == (1, 1, 1), "Dilation must be 1."
        super().__init__(
            in_channels, out_channels, _triple(kernel_size), _triple(stride), _triple(padding),
            dilation, False, _triple(0), groups, bias, padding_mode, device, dtype, rpu_config,
        )

    @classmethod
    def from_digital(cls, module: Conv3d, rpu_config: TorchInferenceRPUConfig) -> "AnalogConv3d":
        """Analog layer with the weights (and bias) of an ``nn.Conv3d``."""
        return cls._from_digital(module, rpu_config, module.weight)

    @classmethod
    def to_digital(cls, module: "AnalogConv3d") -> Conv3d:
        """``nn.Conv3d`` with the same weights."""
        digital = Conv3d(
            module.in_channels, module.out_channels, module.kernel_size, module.stride,
            module.padding, module.dilation, module.groups, module.bias is not None,
            module.padding_mode,
        )
        return cls._to_digital(digital, module, module.weight.data)
