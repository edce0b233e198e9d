"""Registry the DCNv2 layer is published in.

mmcv registers ``ModulatedDeformConv2dPack`` under ``'DCNv2'`` in mmengine's
``MODELS`` registry (mmcv/ops/modulated_deform_conv.py:289) so that
``build_conv_layer(dict(type='DCNv2'), ...)`` finds it
(mmcv/cnn/bricks/conv.py:38-49).  mmengine is used when it is importable;
otherwise a minimal stand-in with the same ``register_module`` / ``get`` /
``build`` surface keeps the lookup working."""


class _LocalRegistry:

    def __init__(self, name):
        self.name = name
        self._modules = {}

    def register_module(self, name=None, force=False, module=None):

        def add(cls):
            keys = [name] if isinstance(name, str) else (name or [cls.__name__])
            for key in keys:
                if key in self._modules and not force:
                    raise KeyError(f'{key} is already registered in {self.name}')
                self._modules[key] = cls
            return cls

        return add(module) if module is not None else add

    def get(self, key):
        return self._modules.get(key)

    def __contains__(self, key):
        return key in self._modules

    def build(self, cfg, *args, **kwargs):
        cfg = dict(cfg)
        key = cfg.pop('type')
        cls = self.get(key)
        if cls is None:
            raise KeyError(f'{key} is not in the {self.name} registry')
        return cls(*args, **cfg, **kwargs)


try:  # pragma: no cover - mmengine is optional
    from mmengine.registry import MODELS
except ImportError:
    MODELS = _LocalRegistry('model')


def build_conv_layer(cfg, *args, **kwargs):
    """``build_conv_layer(dict(type='DCNv2', deform_groups=1), Cin, Cout, 3, ...)``
    for the layer types this package provides (mmcv/cnn/bricks/conv.py:14-51)."""
    if cfg is None or not isinstance(cfg, dict) or 'type' not in cfg:
        raise TypeError('cfg must be a dict containing the key "type"')
    cfg = dict(cfg)
    layer_type = cfg.pop('type')
    cls = MODELS.get(layer_type)
    if cls is None:
        raise KeyError(f'Cannot find {layer_type} in registry')
    return cls(*args, **kwargs, **cfg)
