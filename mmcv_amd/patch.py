"""Bind an already imported mmcv to this package at run time, without editing
mmcv's sources.

mmcv's DCN layers reach their compiled ops through one module-level name,
``ext_module`` (``mmcv/ops/modulated_deform_conv.py:17-19`` and
``mmcv/ops/deform_conv.py:18-21``, both filled by
``mmcv/utils/ext_loader.py:12-16``).  ``patch()`` replaces that name by a
dispatcher: calls whose ``input`` lives on the GPU go to ``mmcv_amd._ext`` (same
op names, same named arguments), everything else to the module mmcv loaded
itself, if it had one.  With ``classes=True`` the public names
``mmcv.ops.ModulatedDeformConv2d``, ``ModulatedDeformConv2dPack``,
``modulated_deform_conv2d`` (and their DCNv1 counterparts) and the ``'DCNv2'`` /
``'DCN'`` entries of the ``MODELS`` registry are rebound to this package's
layers as well, which adds the fused Pack-level call and channels-last inputs
read in place.  ``unpatch()`` puts everything back.
"""
import importlib

_DCN_OPS = ('modulated_deform_conv_forward', 'modulated_deform_conv_backward',
            'deform_conv_forward', 'deform_conv_backward_input',
            'deform_conv_backward_parameters')
_saved = []  # (object, attribute name, had it, old value)


class _ExtDispatch:
    """Stands in for ``mmcv._ext``: the DCN ops on device tensors go to
    ``mmcv_amd._ext``; every other attribute is the original module's."""

    def __init__(self, ours, original):
        self._ours = ours
        self._original = original
        for name in _DCN_OPS:
            setattr(self, name, self._route(name))

    def _route(self, name):
        ours = getattr(self._ours, name)
        theirs = getattr(self._original, name, None) if self._original is not None else None

        def op(*args, **kwargs):
            first = args[0] if args else kwargs.get('input')
            if theirs is not None and not getattr(first, 'is_cuda', False):
                return theirs(*args, **kwargs)
            return ours(*args, **kwargs)

        op.__name__ = name
        return op

    def __getattr__(self, name):  # ops of other layers
        if self._original is None:
            raise AttributeError(name)
        return getattr(self._original, name)


def _set(obj, name, value):
    _saved.append((obj, name, hasattr(obj, name), getattr(obj, name, None)))
    setattr(obj, name, value)


def _registry_set(registry, key, cls):
    table = getattr(registry, '_module_dict', None)
    if table is None:
        table = getattr(registry, '_modules', None)
    if table is None:
        registry.register_module(name=key, force=True, module=cls)
        return
    _saved.append((table, ('item', key), key in table, table.get(key)))
    table[key] = cls


def patch(mmcv=None, classes=True, registry=None):
    """Route the DCN path of ``mmcv`` (default: ``import mmcv``) to this package.

    ``mmcv`` may be the package or its ``ops`` subpackage.  ``registry`` is the
    ``MODELS`` registry to update when ``classes`` is true (default:
    ``mmengine.registry.MODELS`` when importable).  Returns the list of names
    that were rebound."""
    from . import ops as ours
    from .utils import ext_loader
    ext = ext_loader.load_ext('_ext', _DCN_OPS)
    if mmcv is None:
        mmcv = importlib.import_module('mmcv')
    mm_ops = getattr(mmcv, 'ops', mmcv)
    done = []
    for sub in ('modulated_deform_conv', 'deform_conv'):
        mod = getattr(mm_ops, sub, None)
        if mod is None:
            try:
                mod = importlib.import_module(f'{mm_ops.__name__}.{sub}')
            except ImportError:
                continue
        _set(mod, 'ext_module', _ExtDispatch(ext, getattr(mod, 'ext_module', None)))
        done.append(f'{sub}.ext_module')
        if classes:
            for name in ('ModulatedDeformConv2d', 'ModulatedDeformConv2dPack', 'ModulatedDeformConv2dFunction',
                         'modulated_deform_conv2d', 'DeformConv2d', 'DeformConv2dPack', 'DeformConv2dFunction',
                         'deform_conv2d'):
                if hasattr(mod, name):
                    _set(mod, name, getattr(ours, name))
                    done.append(f'{sub}.{name}')
    if classes:
        for name in ('ModulatedDeformConv2d', 'ModulatedDeformConv2dPack', 'modulated_deform_conv2d',
                     'DeformConv2d', 'DeformConv2dPack', 'deform_conv2d'):
            if hasattr(mm_ops, name):
                _set(mm_ops, name, getattr(ours, name))
                done.append(f'ops.{name}')
        if registry is None:
            try:
                from mmengine.registry import MODELS as registry
            except ImportError:
                registry = None
        if registry is not None:
            _registry_set(registry, 'DCNv2', ours.ModulatedDeformConv2dPack)
            _registry_set(registry, 'DCN', ours.DeformConv2dPack)
            done += ['MODELS[DCNv2]', 'MODELS[DCN]']
    return done


def unpatch():
    """Undo every ``patch()`` since the last ``unpatch()``."""
    while _saved:
        obj, name, had, old = _saved.pop()
        if isinstance(name, tuple):
            if had:
                obj[name[1]] = old
            else:
                obj.pop(name[1], None)
        elif had:
            setattr(obj, name, old)
        else:
            delattr(obj, name)
