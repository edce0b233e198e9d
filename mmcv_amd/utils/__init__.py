from . import ext_loader  # noqa: F401
