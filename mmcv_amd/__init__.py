"""mmcv_amd: MI355X-native modulated deformable convolution (DCNv2) forward
behind mmcv's own API for that path.

    from mmcv_amd.ops import (ModulatedDeformConv2d, ModulatedDeformConv2dPack,
                              modulated_deform_conv2d)

The device code is hand-written HIP for gfx950 in ``lib/libmdcn_hip.so`` (C ABI:
``include/mdcn.h``); ``mmcv_amd._ext`` is the PyTorch-ROCm extension module that
mmcv's Python op layer binds to.  Build both with ``python -m mmcv_amd.build``.
``mmcv_amd.patch()`` binds an installed mmcv to it at run time.
"""
__version__ = '0.2.0'

from .patch import patch, unpatch  # noqa: E402,F401
