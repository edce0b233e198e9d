"""Deformable convolution without modulation (DCNv1): the Python op layer.

Same names, argument order and error behaviour as mmcv/ops/deform_conv.py
(``DeformConv2dFunction`` :22-219, ``deform_conv2d`` :222, ``DeformConv2d``
:225-354, ``DeformConv2dPack`` :357-437), bound to ``mmcv_amd._ext``.  The
forward is the DCNv2 kernel run with mask 1 and no bias: the reference's two
samplers are the same function
(mmcv/ops/csrc/pytorch/cpu/deform_conv.cpp:5-38 and
cpu/modulated_deform_conv.cpp:5-33).
"""
import logging
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn.modules.utils import _pair, _single

from ..utils import ext_loader
from .modulated_deform_conv import _conv_output_size, _renamed_kwargs
from .registry import MODELS

ext_module = ext_loader.load_ext('_ext', [
    'deform_conv_forward', 'deform_conv_backward_input',
    'deform_conv_backward_parameters'
])


def _ext_kwargs(ctx, weight, step):
    """Keyword arguments shared by the three extension ops
    (mmcv/ops/csrc/pytorch/pybind.cpp:525-547)."""
    return dict(
        kW=weight.size(3), kH=weight.size(2),
        dW=ctx.stride[1], dH=ctx.stride[0],
        padW=ctx.padding[1], padH=ctx.padding[0],
        dilationW=ctx.dilation[1], dilationH=ctx.dilation[0],
        group=ctx.groups, deformable_group=ctx.deform_groups,
        im2col_step=step)


class DeformConv2dFunction(Function):

    @staticmethod
    def symbolic(g, input, offset, weight, stride, padding, dilation, groups,
                 deform_groups, bias=False, im2col_step=32):
        # ONNX node of mmcv/ops/deform_conv.py:25-46
        return g.op(
            'mmcv::MMCVDeformConv2d',
            input,
            offset,
            weight,
            stride_i=stride,
            padding_i=padding,
            dilation_i=dilation,
            groups_i=groups,
            deform_groups_i=deform_groups,
            bias_i=bias,
            im2col_step_i=im2col_step)

    @staticmethod
    def forward(ctx,
                input: Tensor,
                offset: Tensor,
                weight: Tensor,
                stride: Union[int, Tuple[int, ...]] = 1,
                padding: Union[int, Tuple[int, ...]] = 0,
                dilation: Union[int, Tuple[int, ...]] = 1,
                groups: int = 1,
                deform_groups: int = 1,
                bias: bool = False,
                im2col_step: int = 32) -> Tensor:
        if input is not None and input.dim() != 4:
            raise ValueError(
                f'Expected 4D tensor as input, got {input.dim()}D tensor '
                'instead.')
        assert bias is False, 'Only support bias is False.'
        ctx.stride = _pair(stride)
        ctx.padding = _pair(padding)
        ctx.dilation = _pair(dilation)
        ctx.groups = groups
        ctx.deform_groups = deform_groups
        ctx.im2col_step = im2col_step
        ctx.device = input.device.type
        # offset's dtype decides the compute dtype, as under autocast
        # (mmcv/ops/deform_conv.py:93-101)
        input = input.type_as(offset)
        weight = weight.type_as(input)
        ctx.save_for_backward(input, offset, weight)
        output = input.new_empty(
            _conv_output_size(input, weight, ctx.stride, ctx.padding,
                              ctx.dilation))
        ctx.bufs_ = [input.new_empty(0), input.new_empty(0)]  # columns, ones
        step = min(ctx.im2col_step, input.size(0))
        assert input.size(0) % step == 0, \
            'batch size must be divisible by im2col_step'
        ext_module.deform_conv_forward(input, weight, offset, output,
                                       ctx.bufs_[0], ctx.bufs_[1],
                                       **_ext_kwargs(ctx, weight, step))
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output: Tensor):
        input, offset, weight = ctx.saved_tensors
        grad_input = grad_offset = grad_weight = None
        step = min(ctx.im2col_step, input.size(0))
        assert input.size(0) % step == 0, \
            'batch size must be divisible by im2col_step'
        grad_output = grad_output.contiguous()
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            grad_input = torch.zeros_like(input, memory_format=torch.contiguous_format)
            grad_offset = torch.zeros_like(offset, memory_format=torch.contiguous_format)
            ext_module.deform_conv_backward_input(
                input, offset, grad_output, grad_input, grad_offset, weight,
                ctx.bufs_[0], **_ext_kwargs(ctx, weight, step))
        if ctx.needs_input_grad[2]:
            grad_weight = torch.zeros_like(weight, memory_format=torch.contiguous_format)
            ext_module.deform_conv_backward_parameters(
                input, offset, grad_output, grad_weight, ctx.bufs_[0],
                ctx.bufs_[1], scale=1, **_ext_kwargs(ctx, weight, step))
        return (grad_input, grad_offset, grad_weight, None, None, None, None,
                None, None, None)


deform_conv2d = DeformConv2dFunction.apply


class DeformConv2d(nn.Module):
    r"""Deformable 2D convolution (https://arxiv.org/abs/1703.06211), the layer
    of mmcv/ops/deform_conv.py:225-354.

    Args:
        in_channels (int): Number of channels in the input image.
        out_channels (int): Number of channels produced by the convolution.
        kernel_size (int, tuple): Size of the convolving kernel.
        stride (int, tuple): Stride of the convolution. Default: 1.
        padding (int or tuple): Zero-padding added to both sides of the input.
            Default: 0.
        dilation (int or tuple): Spacing between kernel elements. Default: 1.
        groups (int): Number of blocked connections from input channels to
            output channels. Default: 1.
        deform_groups (int): Number of deformable group partitions.
        bias (bool): Must be False; the layer has no bias.
        im2col_step (int): Kept for compatibility: it sized the reference's
            scratch buffers.  ``batch_size`` must still be divisible by
            ``min(im2col_step, batch_size)``. Default: 32.
    """

    @_renamed_kwargs({'deformable_groups': 'deform_groups'}, 'DeformConv2d')
    def __init__(self,
                 in_channels: int,
                 out_channels: int,
                 kernel_size: Union[int, Tuple[int, ...]],
                 stride: Union[int, Tuple[int, ...]] = 1,
                 padding: Union[int, Tuple[int, ...]] = 0,
                 dilation: Union[int, Tuple[int, ...]] = 1,
                 groups: int = 1,
                 deform_groups: int = 1,
                 bias: bool = False,
                 im2col_step: int = 32) -> None:
        super().__init__()
        assert not bias, f'bias={bias} is not supported in DeformConv2d.'
        assert in_channels % groups == 0, \
            f'in_channels {in_channels} cannot be divisible by groups {groups}'
        assert out_channels % groups == 0, \
            f'out_channels {out_channels} cannot be divisible by groups {groups}'
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.groups = groups
        self.deform_groups = deform_groups
        self.im2col_step = im2col_step
        # attributes nn.Conv2d consumers look for
        self.transposed = False
        self.output_padding = _single(0)
        self.weight = nn.Parameter(
            torch.Tensor(out_channels, in_channels // self.groups,
                         *self.kernel_size))
        self.reset_parameters()

    def reset_parameters(self):
        # He-uniform, as mmcv/ops/deform_conv.py:299-304
        nn.init.kaiming_uniform_(self.weight, nonlinearity='relu')

    def forward(self, x: Tensor, offset: Tensor) -> Tensor:
        """``offset`` is (B, deform_groups * 2 * kh * kw, H_out, W_out), laid out
        ``[y0, x0, y1, x1, ...]`` over the taps in row-major order."""
        # an input smaller than the kernel is zero-padded at the bottom/right and
        # the output cropped again (mmcv/ops/deform_conv.py:327-343)
        too_small = x.size(2) < self.kernel_size[0] or x.size(3) < self.kernel_size[1]
        if too_small:
            extra_h = max(self.kernel_size[0] - x.size(2), 0)
            extra_w = max(self.kernel_size[1] - x.size(3), 0)
            x = F.pad(x, (0, extra_w, 0, extra_h), 'constant', 0).contiguous()
            offset = F.pad(offset, (0, extra_w, 0, extra_h), 'constant', 0).contiguous()
        out = deform_conv2d(x, offset, self.weight, self.stride, self.padding,
                            self.dilation, self.groups, self.deform_groups,
                            False, self.im2col_step)
        if too_small:
            out = out[:, :, :out.size(2) - extra_h, :out.size(3) - extra_w].contiguous()
        return out

    def __repr__(self):
        fields = ('in_channels', 'out_channels', 'kernel_size', 'stride',
                  'padding', 'dilation', 'groups', 'deform_groups')
        body = ''.join(f'{k}={getattr(self, k)},\n' for k in fields)
        return f'{self.__class__.__name__}({body}bias=False)'


@MODELS.register_module('DCN')
class DeformConv2dPack(DeformConv2d):
    """DCNv1 that predicts its own offsets with a zero-initialised
    ``conv_offset`` and so acts like a plain conv layer
    (mmcv/ops/deform_conv.py:357-437)."""

    _version = 2

    #: ``'full'``: conv_offset and the deformable convolution in one extension
    #: call for device tensors that need no gradient; ``'none'``: the
    #: reference's two steps.
    fuse = 'full'

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.conv_offset = nn.Conv2d(
            self.in_channels,
            self.deform_groups * 2 * self.kernel_size[0] * self.kernel_size[1],
            kernel_size=self.kernel_size,
            stride=_pair(self.stride),
            padding=_pair(self.padding),
            dilation=_pair(self.dilation),
            bias=True)
        self.init_offset()

    def init_offset(self):
        self.conv_offset.weight.data.zero_()
        self.conv_offset.bias.data.zero_()

    def forward(self, x: Tensor) -> Tensor:  # type: ignore
        needs_grad = torch.is_grad_enabled() and (
            x.requires_grad or any(p.requires_grad for p in self.parameters()))
        if self.fuse == 'full' and x.is_cuda and x.dim() == 4 and not needs_grad \
                and x.dtype != torch.float64 \
                and not torch.is_autocast_enabled():
            step = min(self.im2col_step, x.size(0))
            assert x.size(0) % step == 0, 'batch size must be divisible by im2col_step'
            return deform_conv2d_pack(x, self.conv_offset, self.weight, self.stride,
                                      self.padding, self.dilation, self.groups,
                                      self.deform_groups)
        offset = self.conv_offset(x)
        return deform_conv2d(x, offset, self.weight, self.stride, self.padding,
                             self.dilation, self.groups, self.deform_groups,
                             False, self.im2col_step)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict,
                              missing_keys, unexpected_keys, error_msgs):
        # checkpoints older than version 2 call the offset conv "<module>_offset"
        version = local_metadata.get('version', None)
        if version is None or version < 2:
            stem = prefix[:-1]
            for leaf in ('weight', 'bias'):
                new_key = prefix + 'conv_offset.' + leaf
                old_key = stem + '_offset.' + leaf
                if new_key not in state_dict and old_key in state_dict:
                    state_dict[new_key] = state_dict.pop(old_key)
        if version is not None and version > 1:
            logging.getLogger('mmcv_amd').info(
                'DeformConv2dPack %s is upgraded to version 2.', prefix.rstrip('.'))
        super()._load_from_state_dict(state_dict, prefix, local_metadata,
                                      strict, missing_keys, unexpected_keys,
                                      error_msgs)


def deform_conv2d_pack(x, conv_offset, weight, stride, padding, dilation, groups,
                       deform_groups, return_raw=False):
    """Forward of ``DeformConv2dPack`` (mmcv/ops/deform_conv.py:405-409) as one
    extension call: ``conv_offset`` runs on the kernel's own input copy and its
    output is read in place as the offsets.  No autograd."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    cw, cb = conv_offset.weight, conv_offset.bias
    x = x.type_as(cw)
    weight = weight.type_as(x)
    output = x.new_empty(_conv_output_size(x, weight, stride, padding, dilation))
    empty = x.new_empty(0)
    raw = x.new_empty((x.size(0), cw.size(0)) + tuple(output.shape[2:])) if return_raw else empty
    ext_module.modulated_deform_conv_pack_forward(
        x, cw.detach(), cb.detach() if cb is not None else empty, raw, weight.detach(),
        empty, output, kernel_h=weight.size(2), kernel_w=weight.size(3),
        stride_h=stride[0], stride_w=stride[1], pad_h=padding[0], pad_w=padding[1],
        dilation_h=dilation[0], dilation_w=dilation[1], group=groups,
        deformable_group=deform_groups, with_bias=False, timed=False, unmodulated=True)
    return (output, raw) if return_raw else output
