"""CPU oracle for the analog convolutions -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Restates what the reference's ``AnalogConv1d/2d/3d`` compute in torch-mode (paths relative to the
reference's ``src/aihwkit_lightning/``): the input is unfolded into patches
(``nn/modules/conv.py:310-322`` through ``torch.nn.functional.unfold`` for 1-d/2-d, ``:40-103``
``unfold3d`` for 3-d), the patches go through the AnalogLinear computation with
``weight.view(out_channels, -1)`` (``:324-354``), and the result is transposed into
``[B, out_channels, *out_size]`` (``:356-367``, ``:822-851``). The backward is the adjoint of the
same chain. Only ``tests/`` may import this module, and only as a checker.

Patch extraction is written here with explicit loops over the kernel offsets and strided slices
(no ``unfold``), so that ``torch.nn.functional.unfold`` and ``F.conv1d/2d/3d`` stay independent
library routines to pin it against (``tests/test_oracle_conv.py``), next to the golden vectors
written by the real reference (``tests/golden/make_golden_conv.py``).

The fold (gradient with respect to the input) accumulates in fp32 in ascending kernel-offset
order and rounds once. For fp32 tensors that is the reference's result up to summation order;
for bf16 the reference sums in bf16 inside ATen's col2im / unfold_backward, so the oracle (and
the HIP kernel, which follows the oracle bit for bit) is the more accurate of the two and agrees
with the golden vectors to bf16 rounding.
"""
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from .torch_mode import OracleCfg, linear_backward, linear_forward


def _three(values: Sequence[int], fill: int) -> List[int]:
    values = [int(v) for v in values]
    return [fill] * (3 - len(values)) + values


def out_extent(size: int, kernel: int, stride: int, padding: int, dilation: int) -> int:
    """``(in + 2 pad - dil (ker - 1) - 1) // stride + 1`` (nn/modules/conv.py:357-362)."""
    return (size + 2 * padding - dilation * (kernel - 1) - 1) // stride + 1


def _slices(k: Sequence[int], out: Sequence[int], stride: Sequence[int], dilation: Sequence[int]):
    """Strided slices of the padded input that kernel offset ``k`` reads, one per dimension."""
    return tuple(
        slice(k[d] * dilation[d], k[d] * dilation[d] + stride[d] * (out[d] - 1) + 1, stride[d])
        for d in range(3)
    )


def conv_patches(x: Tensor, kernel: Sequence[int], stride: Sequence[int], padding: Sequence[int],
                 dilation: Sequence[int]) -> Tuple[Tensor, List[int]]:
    """Patches ``[B, L, C * kD * kH * kW]`` of ``x [B, C, D, H, W]`` (channel-major, then kernel
    offsets with the last dimension fastest: the order of ``weight.view(out_channels, -1)``) and
    the output extents."""
    batch, chan = x.shape[:2]
    size = list(x.shape[2:])
    out = [out_extent(size[d], kernel[d], stride[d], padding[d], dilation[d]) for d in range(3)]
    padded = x.new_zeros(batch, chan, *[size[d] + 2 * padding[d] for d in range(3)])
    padded[:, :, padding[0]:padding[0] + size[0], padding[1]:padding[1] + size[1],
           padding[2]:padding[2] + size[2]] = x
    n_pos = out[0] * out[1] * out[2]
    cols = x.new_zeros(batch, n_pos, chan, kernel[0], kernel[1], kernel[2])
    for kd in range(kernel[0]):
        for kh in range(kernel[1]):
            for kw in range(kernel[2]):
                sl = _slices((kd, kh, kw), out, stride, dilation)
                slab = padded[:, :, sl[0], sl[1], sl[2]]  # [B, C, oD, oH, oW]
                cols[:, :, :, kd, kh, kw] = slab.permute(0, 2, 3, 4, 1).reshape(batch, n_pos, chan)
    return cols.reshape(batch, n_pos, -1), out


def conv_fold(dcols: Tensor, in_shape: Sequence[int], kernel: Sequence[int], stride: Sequence[int],
              padding: Sequence[int], dilation: Sequence[int]) -> Tensor:
    """Adjoint of :func:`conv_patches`: every input element receives the sum of the patch
    entries copied from it (fp32, ascending kernel offset, one rounding)."""
    batch, chan = in_shape[:2]
    size = list(in_shape[2:])
    out = [out_extent(size[d], kernel[d], stride[d], padding[d], dilation[d]) for d in range(3)]
    n_pos = out[0] * out[1] * out[2]
    grads = dcols.float().reshape(batch, n_pos, chan, kernel[0], kernel[1], kernel[2])
    padded = torch.zeros(batch, chan, *[size[d] + 2 * padding[d] for d in range(3)])
    for kd in range(kernel[0]):
        for kh in range(kernel[1]):
            for kw in range(kernel[2]):
                sl = _slices((kd, kh, kw), out, stride, dilation)
                slab = grads[:, :, :, kd, kh, kw].reshape(batch, out[0], out[1], out[2], chan)
                padded[:, :, sl[0], sl[1], sl[2]] += slab.permute(0, 4, 1, 2, 3)
    dx = padded[:, :, padding[0]:padding[0] + size[0], padding[1]:padding[1] + size[1],
                padding[2]:padding[2] + size[2]]
    return dx.to(dcols.dtype)


def conv_forward(
    x: Tensor,
    weight: Tensor,
    bias: Optional[Tensor],
    stride: Sequence[int],
    padding: Sequence[int],
    dilation: Sequence[int],
    cfg: OracleCfg,
    input_range: Optional[Tensor],
    training: bool,
    out_xi: Optional[Sequence[Tensor]] = None,
    w_xi: Optional[Sequence[Tensor]] = None,
    learnable_weight_clip: Optional[Tensor] = None,
) -> Tuple[Tensor, Dict]:
    """Analog convolution of ``x [B, C, *spatial]`` with ``weight [N, C, *kernel]`` (1 to 3
    spatial dimensions). Returns ``[B, N, *out_size]`` and what :func:`conv_backward` needs."""
    n_spatial = weight.dim() - 2
    assert x.dim() == n_spatial + 2
    kernel3 = _three(weight.shape[2:], 1)
    stride3, pad3, dil3 = _three(stride, 1), _three(padding, 0), _three(dilation, 1)
    x5 = x.reshape(x.size(0), x.size(1), *_three(x.shape[2:], 1))
    cols, out = conv_patches(x5, kernel3, stride3, pad3, dil3)
    batch, n_pos, k_in = cols.shape
    y, saved = linear_forward(
        cols.reshape(batch * n_pos, k_in), weight.reshape(weight.size(0), -1), bias, cfg,
        input_range, training, out_xi=out_xi, w_xi=w_xi,
        learnable_weight_clip=learnable_weight_clip,
    )
    y = y.reshape(batch, n_pos, -1).transpose(1, 2).contiguous()
    saved["conv"] = dict(in_shape=tuple(x5.shape), x_shape=tuple(x.shape), kernel=kernel3,
                         stride=stride3, padding=pad3, dilation=dil3, w_shape=tuple(weight.shape))
    return y.reshape(batch, weight.size(0), *out[3 - n_spatial:]), saved


def conv_backward(grad_out: Tensor, saved: Dict):
    """Explicit backward of :func:`conv_forward`: (dx, dweight, dbias, ir_grad or None)."""
    geo = saved["conv"]
    batch, n_out = grad_out.shape[:2]
    g_rows = grad_out.reshape(batch, n_out, -1).transpose(1, 2).reshape(-1, n_out)
    dcols, dw, dbias, ir_grad = linear_backward(g_rows, saved)
    dx = conv_fold(dcols.reshape(batch, -1, dcols.size(-1)), geo["in_shape"], geo["kernel"],
                   geo["stride"], geo["padding"], geo["dilation"])
    return dx.reshape(geo["x_shape"]), dw.reshape(geo["w_shape"]), dbias, ir_grad
