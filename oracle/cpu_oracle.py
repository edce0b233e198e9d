"""TEST INFRASTRUCTURE ONLY: ctypes front-end of ``libmdcn_oracle.so``.

``libmdcn_oracle.so`` is the plain-C restatement (``mdcn_oracle.c``) of mmcv's CPU
algorithm for ``modulated_deform_conv_forward``
(mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:5-33,109-168 and
mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:62-138).  ``reference_forward``
calls the reference's own compiled C++ (``_ref/``) when that was built.
"""
import ctypes
import glob
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = False  # False = not looked for yet, None = absent


def build(ref=True):
    """Compile the C restatement (and the reference, when its tree is here)."""
    subprocess.check_call(['make', '-s', '-C', _HERE, 'oracle'])
    if ref:
        subprocess.check_call(['make', '-s', '-C', _HERE, 'ref'])


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, 'libmdcn_oracle.so')
        if not os.path.exists(path):
            build(ref=False)
        _LIB = ctypes.CDLL(path)
        for t, ct in (('f32', ctypes.c_float), ('f64', ctypes.c_double)):
            getattr(_LIB, f'mdcn_oracle_{t}_sample').restype = ct
            getattr(_LIB, f'mdcn_oracle_{t}_sample').argtypes = [
                ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ct, ct]
            getattr(_LIB, f'mdcn_oracle_{t}_im2col').restype = None
            getattr(_LIB, f'mdcn_oracle_{t}_im2col').argtypes = (
                [ctypes.c_void_p] * 3 + [ctypes.c_int] * 14 + [ctypes.c_void_p])
            getattr(_LIB, f'mdcn_oracle_{t}_forward').restype = ctypes.c_int
            getattr(_LIB, f'mdcn_oracle_{t}_backward').restype = ctypes.c_int
            getattr(_LIB, f'mdcn_oracle_{t}_backward').argtypes = (
                [ctypes.c_void_p] * 11 + [ctypes.c_int] * 16)
            getattr(_LIB, f'mdcn_oracle_{t}_forward').argtypes = (
                [ctypes.c_void_p] * 7 + [ctypes.c_int] * 16)
    return _LIB


def _pair(v):
    return (int(v), int(v)) if np.isscalar(v) else (int(v[0]), int(v[1]))


def _tag(dtype):
    if dtype == np.float32:
        return 'f32'
    if dtype == np.float64:
        return 'f64'
    raise TypeError(f'oracle handles float32/float64, got {dtype}')


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def output_hw(H, W, kh, kw, stride, padding, dilation):
    """Output size rule of modulated_deform_conv.cpp:87-90."""
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    return ((H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def sample(plane, h, w):
    """One modulated-im2col sample of a (H, W) plane at real position (h, w)."""
    plane = np.ascontiguousarray(plane)
    t = _tag(plane.dtype)
    return getattr(_lib(), f'mdcn_oracle_{t}_sample')(
        _ptr(plane), plane.shape[0], plane.shape[1], h, w)


def im2col(im, offset, mask, kernel, stride=1, padding=0, dilation=1,
           deform_groups=1):
    """Columns (C*kh*kw, Ho*Wo) of one sample ``im`` (C, H, W)."""
    im = np.ascontiguousarray(im)
    t = _tag(im.dtype)
    offset = np.ascontiguousarray(offset, dtype=im.dtype)
    mask = np.ascontiguousarray(mask, dtype=im.dtype)
    kh, kw = _pair(kernel)
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    C, H, W = im.shape
    Ho, Wo = output_hw(H, W, kh, kw, stride, padding, dilation)
    assert offset.shape == (deform_groups * 2 * kh * kw, Ho, Wo), offset.shape
    assert mask.shape == (deform_groups * kh * kw, Ho, Wo), mask.shape
    col = np.empty((C * kh * kw, Ho * Wo), dtype=im.dtype)
    getattr(_lib(), f'mdcn_oracle_{t}_im2col')(
        _ptr(im), _ptr(offset), _ptr(mask), C, H, W, kh, kw, ph, pw, sh, sw,
        dh, dw, deform_groups, Ho, Wo, _ptr(col))
    return col


def forward(input, offset, mask, weight, bias=None, stride=1, padding=0,
            dilation=1, groups=1, deform_groups=1):
    """Whole DCNv2 forward on numpy arrays (float32 or float64), NCHW."""
    input = np.ascontiguousarray(input)
    t = _tag(input.dtype)
    dt = input.dtype
    offset = np.ascontiguousarray(offset, dtype=dt)
    mask = np.ascontiguousarray(mask, dtype=dt)
    weight = np.ascontiguousarray(weight, dtype=dt)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=dt)
    N, Cin, H, W = input.shape
    Cout, wcin, kh, kw = weight.shape
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    Ho, Wo = output_hw(H, W, kh, kw, stride, padding, dilation)
    if Ho <= 0 or Wo <= 0:
        raise ValueError('convolution input is too small')
    assert offset.shape == (N, deform_groups * 2 * kh * kw, Ho, Wo), offset.shape
    assert mask.shape == (N, deform_groups * kh * kw, Ho, Wo), mask.shape
    out = np.empty((N, Cout, Ho, Wo), dtype=dt)
    columns = np.empty((Cin * kh * kw, Ho * Wo), dtype=dt)
    rc = getattr(_lib(), f'mdcn_oracle_{t}_forward')(
        _ptr(input), _ptr(weight), _ptr(bias) if bias is not None else None,
        _ptr(offset), _ptr(mask), _ptr(out), _ptr(columns), N, Cin, H, W, Cout,
        wcin, kh, kw, sh, sw, ph, pw, dh, dw, groups, deform_groups)
    if rc != 0:
        raise RuntimeError("Input shape and kernel channels won't match: "
                           f'({Cin} vs {wcin * groups}).')
    return out


def backward(input, offset, mask, weight, grad_output, with_bias=True, stride=1,
             padding=0, dilation=1, groups=1, deform_groups=1):
    """Whole DCNv2 backward on numpy arrays (float32 or float64): returns
    (grad_input, grad_offset, grad_mask, grad_weight, grad_bias or None)."""
    input = np.ascontiguousarray(input)
    t = _tag(input.dtype)
    dt = input.dtype
    offset = np.ascontiguousarray(offset, dtype=dt)
    mask = np.ascontiguousarray(mask, dtype=dt)
    weight = np.ascontiguousarray(weight, dtype=dt)
    grad_output = np.ascontiguousarray(grad_output, dtype=dt)
    N, Cin, H, W = input.shape
    Cout, wcin, kh, kw = weight.shape
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    Ho, Wo = output_hw(H, W, kh, kw, stride, padding, dilation)
    assert grad_output.shape == (N, Cout, Ho, Wo), grad_output.shape
    assert offset.shape == (N, deform_groups * 2 * kh * kw, Ho, Wo), offset.shape
    assert mask.shape == (N, deform_groups * kh * kw, Ho, Wo), mask.shape
    g_in = np.empty_like(input)
    g_off = np.zeros_like(offset)
    g_mask = np.zeros_like(mask)
    g_w = np.empty_like(weight)
    g_b = np.empty((Cout,), dtype=dt) if with_bias else None
    columns = np.empty((Cin * kh * kw, Ho * Wo), dtype=dt)
    rc = getattr(_lib(), f'mdcn_oracle_{t}_backward')(
        _ptr(input), _ptr(weight), _ptr(offset), _ptr(mask), _ptr(grad_output),
        _ptr(g_in), _ptr(g_w), _ptr(g_b) if with_bias else None, _ptr(g_off),
        _ptr(g_mask), _ptr(columns), N, Cin, H, W, Cout, wcin, kh, kw, sh, sw,
        ph, pw, dh, dw, groups, deform_groups)
    if rc != 0:
        raise RuntimeError("Input shape and kernel channels won't match: "
                           f'({Cin} vs {wcin * groups}).')
    return g_in, g_off, g_mask, g_w, g_b


def reference_backward(input, offset, mask, weight, grad_output, with_bias=True,
                       stride=1, padding=0, dilation=1, groups=1, deform_groups=1):
    """mmcv's compiled CPU ``modulated_deform_conv_backward`` on torch CPU tensors,
    called the way mmcv/ops/modulated_deform_conv.py:172-213 calls it."""
    import torch
    ext = load_reference_ext()
    if ext is None or not hasattr(ext, 'modulated_deform_conv_backward'):
        raise RuntimeError('oracle/_ref is not built (or predates the backward binding)')
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    kh, kw = weight.shape[2:]
    bias = input.new_zeros(weight.shape[0]) if with_bias else input.new_empty(0)
    g_in, g_off, g_mask = torch.zeros_like(input), torch.zeros_like(offset), torch.zeros_like(mask)
    g_w, g_b = torch.zeros_like(weight), torch.zeros_like(bias)
    ext.modulated_deform_conv_backward(
        input.contiguous(), weight.contiguous(), bias, input.new_empty(0),
        offset.contiguous(), mask.contiguous(), input.new_empty(0), g_in, g_w, g_b,
        g_off, g_mask, grad_output.contiguous(), kernel_h=kh, kernel_w=kw,
        stride_h=sh, stride_w=sw, pad_h=ph, pad_w=pw, dilation_h=dh, dilation_w=dw,
        group=groups, deformable_group=deform_groups, with_bias=with_bias)
    return g_in, g_off, g_mask, g_w, (g_b if with_bias else None)


def load_reference_ext():
    """The reference's own C++ for this path, compiled into ``_ref/`` (or None)."""
    global _REF
    if _REF is False:
        _REF = None
        hits = sorted(glob.glob(os.path.join(_HERE, '_ref', 'mmcv_ref_ext*.so')))
        if hits:
            import torch  # noqa: F401  (the extension links against libtorch)
            spec = importlib.util.spec_from_file_location('mmcv_ref_ext', hits[0])
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            _REF = mod
    return _REF


def reference_forward(input, offset, mask, weight, bias=None, stride=1,
                      padding=0, dilation=1, groups=1, deform_groups=1):
    """mmcv's compiled CPU ``modulated_deform_conv_forward`` on torch CPU tensors,
    called the way mmcv/ops/modulated_deform_conv.py:145-169 calls it."""
    import torch
    ext = load_reference_ext()
    if ext is None:
        raise RuntimeError('oracle/_ref is not built')
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    N, _, H, W = input.shape
    Cout, _, kh, kw = weight.shape
    Ho, Wo = output_hw(H, W, kh, kw, stride, padding, dilation)
    with_bias = bias is not None
    if not with_bias:
        bias = input.new_empty(0)
    out = input.new_empty((N, Cout, Ho, Wo))
    ext.modulated_deform_conv_forward(
        input.contiguous(), weight.contiguous(), bias, input.new_empty(0),
        offset.contiguous(), mask.contiguous(), out, input.new_empty(0),
        kernel_h=kh, kernel_w=kw, stride_h=sh, stride_w=sw, pad_h=ph, pad_w=pw,
        dilation_h=dh, dilation_w=dw, group=groups,
        deformable_group=deform_groups, with_bias=with_bias)
    return out
