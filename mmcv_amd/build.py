"""Builds the native parts of mmcv_amd in-tree.

``libmdcn_hip.so``  hand-written HIP for gfx950 behind the C ABI of include/mdcn.h
                    (hipcc cross-compiles it without a GPU),
``_ext*.so``        the PyTorch-ROCm extension module ``mmcv_amd._ext`` (host
                    compiler only) that mmcv's Python op layer binds to.

Run ``python -m mmcv_amd.build``.
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, 'csrc')
LIBDIR = os.path.join(PKG, 'lib')
HIP_LIB = os.path.join(LIBDIR, 'libmdcn_hip.so')
EXT_LIB = os.path.join(PKG, '_ext' + sysconfig.get_config_var('EXT_SUFFIX'))
ROCM = os.environ.get('ROCM_PATH', '/opt/rocm')

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared',
    # packed-fp32 VALU forms are kept out of the generated code
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # '#pragma unroll' loops whose bodies index register arrays must unroll whatever their size
    '-mllvm', '-pragma-unroll-threshold=100000',
    '-Wno-unused-command-line-argument',
]


def _run(cmd):
    print(' '.join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip(extra=(), check=True):
    """Compile the library; with `check`, keep the device assembly of the compile
    and scan it (asm_check.py) before the library is accepted."""
    import shutil
    import tempfile
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.path.join(ROCM, 'bin', 'hipcc')
    cmd = [hipcc, *HIPCC_FLAGS, *extra, '-I', os.path.join(ROOT, 'include')]
    src = os.path.join(CSRC, 'mdcn_api.hip')
    if not check:
        _run([*cmd, '-o', HIP_LIB, src])
        return HIP_LIB
    from . import asm_check
    tmp = tempfile.mkdtemp(prefix='mdcn_build_')
    try:
        out = os.path.join(tmp, 'libmdcn_hip.so')
        print(' '.join([*cmd, '-save-temps=obj', '-o', out, src]), flush=True)
        subprocess.check_call([*cmd, '-save-temps=obj', '-o', out, src], cwd=tmp)
        asm = [os.path.join(tmp, f) for f in os.listdir(tmp) if f.endswith('.s') and 'gfx950' in f]
        if not asm:
            raise RuntimeError('no device assembly found to check')
        bad = sum(asm_check.check_file(f) for f in asm)
        if bad:
            raise RuntimeError(f'{bad} finding(s) in the device assembly around inline-asm memory instructions '
                               '(see above and asm_check.py)')
        print(f'asm_check: {len(asm)} device assembly file(s) clean', flush=True)
        shutil.move(out, HIP_LIB)
        # the assembly the library was built from stays beside it (git-ignored): tests scan it again
        for f in asm:
            shutil.copy(f, os.path.join(LIBDIR, 'libmdcn_hip.s' if len(asm) == 1 else os.path.basename(f)))
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return HIP_LIB


def build_ext():
    import torch
    tdir = os.path.dirname(torch.__file__)
    tlib = os.path.join(tdir, 'lib')
    cmd = [
        'g++', '-O2', '-std=c++17', '-fPIC', '-shared', '-w',
        '-D__HIP_PLATFORM_AMD__=1', '-DUSE_ROCM=1',
        '-DTORCH_EXTENSION_NAME=_ext', '-DTORCH_API_INCLUDE_EXTENSION_H',
        '-D_GLIBCXX_USE_CXX11_ABI=1',
        '-I', os.path.join(ROOT, 'include'),
        '-I', os.path.join(tdir, 'include'),
        '-I', os.path.join(tdir, 'include', 'torch', 'csrc', 'api', 'include'),
        '-I', os.path.join(ROCM, 'include'),
        '-I', sysconfig.get_paths()['include'],
        os.path.join(CSRC, 'ext.cpp'), '-o', EXT_LIB,
        '-L', LIBDIR, '-lmdcn_hip', '-Wl,-rpath,$ORIGIN/lib',
        '-L', tlib, '-Wl,-rpath,' + tlib,
        '-lc10', '-lc10_hip', '-ltorch', '-ltorch_cpu', '-ltorch_hip',
        '-ltorch_python',
    ]
    _run(cmd)
    return EXT_LIB


def build_all():
    build_hip()
    build_ext()


if __name__ == '__main__':
    build_all()
    sys.exit(0)
