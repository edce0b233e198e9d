"""Modulated deformable convolution (DCNv2): the Python op layer.

Same names, argument order and error behaviour as
mmcv/ops/modulated_deform_conv.py (``ModulatedDeformConv2dFunction`` :22-230,
``modulated_deform_conv2d`` :233, ``ModulatedDeformConv2d`` :236-286,
``ModulatedDeformConv2dPack`` :289-363), bound to ``mmcv_amd._ext`` whose
forward runs the fused HIP kernel.  mmengine is optional here: when it is
importable the Pack is registered in its ``MODELS`` registry as ``'DCNv2'``,
otherwise in the small registry of ``mmcv_amd.ops.registry``.
"""
import functools
import logging
import math
import warnings
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn.modules.utils import _pair, _single

from ..utils import ext_loader
from .registry import MODELS

ext_module = ext_loader.load_ext(
    '_ext',
    ['modulated_deform_conv_forward', 'modulated_deform_conv_backward'])


def _renamed_kwargs(renames, cls_name):
    """Accept legacy keyword names (mmcv's ``deprecated_api_warning`` as used at
    mmcv/ops/modulated_deform_conv.py:238-239): warn and forward under the new
    name; passing both spellings is an error."""

    def decorate(fn):

        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            for old, new in renames.items():
                if old in kwargs:
                    if new in kwargs:
                        raise AssertionError(
                            f'The expected behavior is to replace the '
                            f'deprecated key `{old}` to new key `{new}`, but '
                            f'got them in the arguments at the same time.')
                    warnings.warn(
                        f'"{old}" is deprecated in `{cls_name}.{fn.__name__}`, '
                        f'please use "{new}" instead', DeprecationWarning)
                    kwargs[new] = kwargs.pop(old)
            return fn(*args, **kwargs)

        return wrapper

    return decorate


def _conv_output_size(input, weight, stride, padding, dilation):
    """(N, Cout, Ho, Wo); ValueError when a size is not positive
    (mmcv/ops/modulated_deform_conv.py:216-230)."""
    size = [input.size(0), weight.size(0)]
    for d in range(input.dim() - 2):
        extent = dilation[d] * (weight.size(d + 2) - 1) + 1
        size.append((input.size(d + 2) + 2 * padding[d] - extent) // stride[d] + 1)
    if min(size) <= 0:
        raise ValueError('convolution input is too small (output would be ' +
                         'x'.join(str(s) for s in size) + ')')
    return tuple(int(s) for s in size)


def _geometry_kwargs(ctx, weight):
    """The eleven keyword arguments of the extension ops
    (mmcv/ops/csrc/pytorch/pybind.cpp:641-657)."""
    return dict(
        kernel_h=weight.size(2), kernel_w=weight.size(3),
        stride_h=ctx.stride[0], stride_w=ctx.stride[1],
        pad_h=ctx.padding[0], pad_w=ctx.padding[1],
        dilation_h=ctx.dilation[0], dilation_w=ctx.dilation[1],
        group=ctx.groups, deformable_group=ctx.deform_groups,
        with_bias=ctx.with_bias)


class ModulatedDeformConv2dFunction(Function):

    @staticmethod
    def symbolic(g, input, offset, mask, weight, bias, stride, padding,
                 dilation, groups, deform_groups):
        # ONNX node of mmcv/ops/modulated_deform_conv.py:25-37
        operands = [input, offset, mask, weight]
        if bias is not None:
            operands.append(bias)
        return g.op(
            'mmcv::MMCVModulatedDeformConv2d',
            *operands,
            stride_i=stride,
            padding_i=padding,
            dilation_i=dilation,
            groups_i=groups,
            deform_groups_i=deform_groups)

    @staticmethod
    def forward(ctx,
                input: torch.Tensor,
                offset: torch.Tensor,
                mask: torch.Tensor,
                weight: nn.Parameter,
                bias: Optional[nn.Parameter] = None,
                stride: int = 1,
                padding: int = 0,
                dilation: int = 1,
                groups: int = 1,
                deform_groups: int = 1) -> torch.Tensor:
        if input is not None and input.dim() != 4:
            raise ValueError(
                f'Expected 4D tensor as input, got {input.dim()}D tensor '
                'instead.')
        ctx.stride = _pair(stride)
        ctx.padding = _pair(padding)
        ctx.dilation = _pair(dilation)
        ctx.groups = groups
        ctx.deform_groups = deform_groups
        ctx.with_bias = bias is not None
        ctx.device = input.device.type
        if not ctx.with_bias:
            bias = input.new_empty(0)  # 0-element stand-in, never read
        # offset's dtype decides the compute dtype: under autocast the offset
        # conv yields half/bf16 while input and parameters may still be fp32
        # (mmcv/ops/modulated_deform_conv.py:129-139).
        input = input.type_as(offset)
        weight = weight.type_as(input)
        bias = bias.type_as(input)
        mask = mask.type_as(input)
        ctx.save_for_backward(input, offset, mask, weight, bias)
        output = input.new_empty(
            _conv_output_size(input, weight, ctx.stride, ctx.padding,
                              ctx.dilation))
        # scratch placeholders of the two-pass design; the fused kernel needs none
        ctx._bufs = [input.new_empty(0), input.new_empty(0)]
        ext_module.modulated_deform_conv_forward(
            input, weight, bias, ctx._bufs[0], offset, mask, output,
            ctx._bufs[1],
            **_geometry_kwargs(ctx, weight))
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output: torch.Tensor) -> tuple:
        input, offset, mask, weight, bias = ctx.saved_tensors
        # dense gradients whatever the memory format of the saved tensors (the op writes NCHW)
        grads = [torch.zeros_like(t, memory_format=torch.contiguous_format)
                 for t in (input, offset, mask, weight, bias)]
        grad_input, grad_offset, grad_mask, grad_weight, grad_bias = grads
        ext_module.modulated_deform_conv_backward(
            input, weight, bias, ctx._bufs[0], offset, mask, ctx._bufs[1],
            grad_input, grad_weight, grad_bias, grad_offset, grad_mask,
            grad_output.contiguous(),
            **_geometry_kwargs(ctx, weight))
        if not ctx.with_bias:
            grad_bias = None
        return (grad_input, grad_offset, grad_mask, grad_weight, grad_bias,
                None, None, None, None, None)

    @staticmethod
    def _output_size(ctx, input, weight):
        return _conv_output_size(input, weight, ctx.stride, ctx.padding,
                                 ctx.dilation)


modulated_deform_conv2d = ModulatedDeformConv2dFunction.apply


class ModulatedDeformConv2d(nn.Module):
    """DCNv2 layer taking (x, offset, mask); parameters and attributes as in
    mmcv/ops/modulated_deform_conv.py:236-286."""

    @_renamed_kwargs({'deformable_groups': 'deform_groups'},
                     cls_name='ModulatedDeformConv2d')
    def __init__(self,
                 in_channels: int,
                 out_channels: int,
                 kernel_size: Union[int, Tuple[int]],
                 stride: int = 1,
                 padding: int = 0,
                 dilation: int = 1,
                 groups: int = 1,
                 deform_groups: int = 1,
                 bias: Union[bool, str] = True):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.groups = groups
        self.deform_groups = deform_groups
        # attributes nn.Conv2d consumers look for
        self.transposed = False
        self.output_padding = _single(0)

        self.weight = nn.Parameter(
            torch.empty(out_channels, in_channels // groups, *self.kernel_size))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_channels))
        else:
            self.register_parameter('bias', None)
        self.init_weights()

    def init_weights(self):
        # U(-1/sqrt(Cin*kh*kw), +1/sqrt(Cin*kh*kw)), zero bias (:270-279)
        fan = self.in_channels * self.kernel_size[0] * self.kernel_size[1]
        bound = 1. / math.sqrt(fan)
        self.weight.data.uniform_(-bound, bound)
        if self.bias is not None:
            self.bias.data.zero_()

    def forward(self, x: torch.Tensor, offset: torch.Tensor,
                mask: torch.Tensor) -> torch.Tensor:
        return modulated_deform_conv2d(x, offset, mask, self.weight, self.bias,
                                       self.stride, self.padding,
                                       self.dilation, self.groups,
                                       self.deform_groups)


def modulated_deform_conv2d_pack(x, conv_offset, weight, bias, stride, padding,
                                 dilation, groups, deform_groups, own_conv=True,
                                 return_raw=False, timed=False):
    """Forward of ``ModulatedDeformConv2dPack``
    (mmcv/ops/modulated_deform_conv.py:327-335) as one extension call: the
    offsets are the first two thirds of ``conv_offset``'s output channels as they
    lie, the mask is the sigmoid of the last third, both read by the kernel
    itself.  ``own_conv=False`` leaves ``conv_offset`` to torch.  No autograd."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    cw, cb = conv_offset.weight, conv_offset.bias
    x = x.type_as(cw)
    weight = weight.type_as(x)
    with_bias = bias is not None
    bias = bias.type_as(x) if with_bias else x.new_empty(0)
    output = x.new_empty(_conv_output_size(x, weight, stride, padding, dilation))
    empty = x.new_empty(0)
    if own_conv:
        raw = x.new_empty((x.size(0), cw.size(0)) + tuple(output.shape[2:])) if return_raw else empty
        ow, ob = cw, (cb if cb is not None else empty)
    else:
        with torch.no_grad():
            raw = conv_offset(x)
        ow = ob = empty
    ms = ext_module.modulated_deform_conv_pack_forward(
        x, ow.detach(), ob.detach(), raw, weight.detach(), bias.detach(), output,
        kernel_h=weight.size(2), kernel_w=weight.size(3),
        stride_h=stride[0], stride_w=stride[1], pad_h=padding[0], pad_w=padding[1],
        dilation_h=dilation[0], dilation_w=dilation[1], group=groups,
        deformable_group=deform_groups, with_bias=with_bias, timed=timed)
    out = (output,)
    if return_raw:
        out += (raw,)
    if timed:
        out += (ms,)
    return out[0] if len(out) == 1 else out


@MODELS.register_module('DCNv2')
class ModulatedDeformConv2dPack(ModulatedDeformConv2d):
    """DCNv2 that predicts its own offsets and mask with a zero-initialised
    ``conv_offset`` and so acts like a plain conv layer
    (mmcv/ops/modulated_deform_conv.py:289-363).

    Args:
        in_channels (int): Same as nn.Conv2d.
        out_channels (int): Same as nn.Conv2d.
        kernel_size (int or tuple[int]): Same as nn.Conv2d.
        stride (int): Same as nn.Conv2d, while tuple is not supported.
        padding (int): Same as nn.Conv2d, while tuple is not supported.
        dilation (int): Same as nn.Conv2d, while tuple is not supported.
        groups (int): Same as nn.Conv2d.
        bias (bool or str): ``'auto'`` is treated as True.
    """

    _version = 2

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        taps = self.kernel_size[0] * self.kernel_size[1]
        self.conv_offset = nn.Conv2d(
            self.in_channels,
            self.deform_groups * 3 * taps,
            kernel_size=self.kernel_size,
            stride=self.stride,
            padding=self.padding,
            dilation=self.dilation,
            bias=True)
        self.init_weights()

    def init_weights(self) -> None:
        super().init_weights()
        if hasattr(self, 'conv_offset'):
            self.conv_offset.weight.data.zero_()
            self.conv_offset.bias.data.zero_()

    #: How much of ``forward`` runs inside the HIP library for device tensors
    #: that need no gradient: ``'full'`` = conv_offset, channel split, sigmoid
    #: and the deformable convolution in one extension call; ``'split'`` =
    #: conv_offset by torch, the rest fused; ``'none'`` = the reference's
    #: sequence of tensor operations.
    fuse = 'full'

    def forward(self, x: torch.Tensor) -> torch.Tensor:  # type: ignore
        needs_grad = torch.is_grad_enabled() and (
            x.requires_grad or any(p.requires_grad for p in self.parameters()))
        if self.fuse != 'none' and x.is_cuda and x.dim() == 4 and not needs_grad \
                and x.dtype != torch.float64 \
                and not torch.is_autocast_enabled():
            return modulated_deform_conv2d_pack(
                x, self.conv_offset, self.weight, self.bias, self.stride,
                self.padding, self.dilation, self.groups, self.deform_groups,
                own_conv=self.fuse == 'full')
        # first two thirds of conv_offset's channels are the offsets, the last
        # third the mask logits (:328-331)
        raw = self.conv_offset(x)
        dy_dx_a, dy_dx_b, logits = torch.chunk(raw, 3, dim=1)
        offset = torch.cat((dy_dx_a, dy_dx_b), dim=1)
        mask = torch.sigmoid(logits)
        return modulated_deform_conv2d(x, offset, mask, self.weight, self.bias,
                                       self.stride, self.padding,
                                       self.dilation, self.groups,
                                       self.deform_groups)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict,
                              missing_keys, unexpected_keys, error_msgs):
        # Checkpoints written before version 2 name the offset conv
        # "<module>_offset.*" instead of "<module>.conv_offset.*" (:341-353).
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
                'ModulatedDeformConvPack %s is upgraded to version 2.',
                prefix.rstrip('.'))
        super()._load_from_state_dict(state_dict, prefix, local_metadata,
                                      strict, missing_keys, unexpected_keys,
                                      error_msgs)
