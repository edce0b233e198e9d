"""Builds bench_probe/libmfma_probe.so: the MFMA-rate probe bench.py reports beside the
kernel's roofline figure (what the matrix cores of the box sustain on back-to-back
MFMAs).  Measurement aid of the benchmark, not part of the library.

Run ``python bench_probe/build.py``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, ROOT)
PROBE_LIB = os.path.join(HERE, 'libmfma_probe.so')


def build():
    from mmcv_amd.build import HIPCC_FLAGS, ROCM
    cmd = [os.path.join(ROCM, 'bin', 'hipcc'), *HIPCC_FLAGS, '-I', os.path.join(ROOT, 'include'),
           '-o', PROBE_LIB, os.path.join(HERE, 'mfma_probe.hip')]
    print(' '.join(cmd), flush=True)
    subprocess.check_call(cmd)
    return PROBE_LIB


if __name__ == '__main__':
    build()
