from .deform_conv import (DeformConv2d, DeformConv2dFunction, DeformConv2dPack,
                          deform_conv2d, deform_conv2d_pack)
from .modulated_deform_conv import (ModulatedDeformConv2d,
                                    ModulatedDeformConv2dFunction,
                                    ModulatedDeformConv2dPack,
                                    modulated_deform_conv2d,
                                    modulated_deform_conv2d_pack)
from .registry import MODELS, build_conv_layer

__all__ = [
    'ModulatedDeformConv2d', 'ModulatedDeformConv2dPack',
    'ModulatedDeformConv2dFunction', 'modulated_deform_conv2d',
    'modulated_deform_conv2d_pack', 'DeformConv2d', 'DeformConv2dPack',
    'DeformConv2dFunction', 'deform_conv2d', 'deform_conv2d_pack', 'MODELS',
    'build_conv_layer'
]
