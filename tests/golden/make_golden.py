"""Writes tests/golden/ref_cases.npz: outputs of the reference's OWN compiled CPU
``modulated_deform_conv_forward`` (oracle/_ref, built from the reference's C++
by oracle/Makefile) on small seeded cases.  Run in the build container, where
the reference tree exists:

    make -C oracle ref && python tests/golden/make_golden.py

Only the expected outputs are stored; inputs are regenerated from the seed by
tests/common.py:make_case, whose parameters are stored next to each output."""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from common import make_case  # noqa: E402

CASES = {
    'g_base': dict(seed=101, N=2, Cin=32, Cout=48, H=9, W=11),
    'g_oob': dict(seed=102, N=1, Cin=32, Cout=32, H=8, W=8, sigma=6.0),
    'g_stride2_dg2': dict(seed=103, N=2, Cin=64, Cout=32, H=13, W=12, stride=2, deform_groups=2),
    'g_groups2_dil2': dict(seed=104, N=1, Cin=64, Cout=64, H=11, W=10, groups=2, dilation=2, padding=2),
    'g_k2_pad1_nobias': dict(seed=105, N=1, Cin=32, Cout=16, H=6, W=7, k=2, padding=1, bias=False),
    'g_odd_channels': dict(seed=106, N=2, Cin=6, Cout=4, H=7, W=9, groups=2, deform_groups=3),
    'g_f64': dict(seed=107, N=1, Cin=32, Cout=32, H=7, W=7),
}


def main():
    assert oracle.load_reference_ext() is not None, 'build oracle/_ref first'
    out = {}
    meta = {}
    for name, kw in CASES.items():
        kw = dict(kw)
        seed = kw.pop('seed')
        case = make_case(seed, **kw)
        dt = torch.float64 if name.endswith('f64') else torch.float32
        t = {k: (v.to(dt) if torch.is_tensor(v) else v) for k, v in case.items()}
        y = oracle.reference_forward(t['input'], t['offset'], t['mask'], t['weight'],
                                     t['bias'], t['stride'], t['padding'],
                                     t['dilation'], t['groups'], t['deform_groups'])
        out[name] = y.numpy()
        meta[name] = dict(seed=seed, dtype=str(dt).split('.')[-1], **kw)
    np.savez_compressed(os.path.join(HERE, 'ref_cases.npz'), **out)
    with open(os.path.join(HERE, 'ref_cases.json'), 'w') as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print('wrote', len(out), 'cases')


if __name__ == '__main__':
    main()
