"""Loader of the compiled extension module, the counterpart of
mmcv/utils/ext_loader.py:12-16: import ``mmcv_amd.<name>`` and insist that every
requested op is there.  A missing build is an error, never a silent fallback."""
import importlib


def load_ext(name, funcs):
    try:
        ext = importlib.import_module('mmcv_amd.' + name)
    except ImportError as e:
        raise ImportError(
            f'mmcv_amd.{name} is not built or cannot be loaded ({e}); '
            'run `python -m mmcv_amd.build` in the repository root') from e
    for fun in funcs:
        assert hasattr(ext, fun), f'{fun} miss in module {name}'
    return ext
