"""TEST INFRASTRUCTURE ONLY: CPU checkers for the DCNv2 forward path.

Nothing under ``mmcv_amd`` may import this package.  It may be used by
``tests/``, by ``__graft_entry__.smoke()`` and by the CPU-baseline leg of
``bench.py`` -- as the checker, never as the thing measured or shipped.
"""
from .cpu_oracle import (backward, forward, im2col, sample, output_hw,  # noqa: F401
                         reference_backward,
                         load_reference_ext, reference_forward, build)
