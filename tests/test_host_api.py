"""Host-side checks that need no GPU: the C-ABI library loads and exports what
include/mdcn.h declares, its parameter validation, and the Python op layer's
mmcv-compatible behaviour (names, errors, registry, state-dict upgrade)."""
import ctypes
import os
import re
import warnings

import pytest
import torch

from mmcv_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, 'include', 'mdcn.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(mdcn_[a-z_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_functions()
    assert sorted(names) == sorted(capi.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.mdcn_abi_version() == 5
    assert capi.status_string(0) == 'ok'
    assert 'workspace' in capi.status_string(-4)


def test_params_struct_matches_header_order():
    text = open(os.path.join(ROOT, 'include', 'mdcn.h')).read()
    body = re.search(r'typedef struct mdcn_params \{(.*?)\} mdcn_params;', text, re.S).group(1)
    body = re.sub(r'/\*.*?\*/', '', body, flags=re.S)
    fields = []
    for decl in body.split(';'):
        decl = decl.strip()
        if not decl:
            continue
        for name in decl.split(','):
            fields.append(name.strip().split()[-1].lstrip('*'))
    assert fields == [f[0] for f in capi.MdcnParams._fields_]


def test_output_size_and_shape_errors():
    p = capi.make_params(capi.MDCN_F32, 16, 512, 50, 50, 512, 3, 3, (2, 2), (1, 1),
                         (1, 1), 1, 4)
    assert capi.output_size(p) == (0, 25, 25)
    p = capi.make_params(capi.MDCN_F32, 1, 4, 2, 2, 4, 3, 3)  # 2x2 input, 3x3 kernel, no pad
    assert capi.output_size(p)[0] == -2
    p = capi.make_params(capi.MDCN_F32, 1, 6, 8, 8, 4, 3, 3, groups=4)
    assert capi.output_size(p)[0] == -2  # Cin % groups
    p = capi.make_params(capi.MDCN_F32, 1, 6, 8, 8, 6, 3, 3, deform_groups=4)
    assert capi.output_size(p)[0] == -2
    p = capi.make_params(7, 1, 4, 8, 8, 4, 3, 3)
    assert capi.output_size(p)[0] == -3
    assert capi.load().mdcn_output_size(None, None, None) == -1


def test_eligibility_and_workspace():
    lib = capi.load()
    # N=16, C=256, 100x152 bf16: fused; copy (102*154*256*2 B per image) + weights
    p = capi.make_params(capi.MDCN_BF16, 16, 256, 100, 152, 256, 3, 3, (1, 1), (1, 1))
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 1
    ws = lib.mdcn_workspace_bytes(ctypes.byref(p))
    assert ws >= 16 * 102 * 154 * 256 * 2 + 256 * 256 * 9 * 2
    # ... and, for 16-bit 256-channel tiles, one 128 x 256 fp32 buffer and a counter per workgroup
    # for the tiles that are cut along K (256 workgroups when no device tells the CU count)
    split = 256 * 128 * 256 * 4 + 256 * 4
    assert ws < 1.02 * (16 * 102 * 154 * 256 * 2 + 256 * 256 * 9 * 2) + split + 4096
    # a K step is 128 bytes of channels: Cin/groups and Cin/deform_groups must be
    # multiples of 32 (fp32) resp. 64 (fp16, bf16)
    p = capi.make_params(capi.MDCN_F32, 1, 32, 8, 8, 4, 3, 3)
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 1
    p = capi.make_params(capi.MDCN_F16, 1, 32, 8, 8, 4, 3, 3)
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    p = capi.make_params(capi.MDCN_F32, 1, 64, 8, 8, 4, 3, 3, deform_groups=4)
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0
    p = capi.make_params(capi.MDCN_F32, 1, 64, 8, 8, 4, 6, 6)  # 36 taps exceed the table
    assert lib.mdcn_fused_eligible(ctypes.byref(p)) == 0
    p.path = capi.PATH_DIRECT
    assert lib.mdcn_workspace_bytes(ctypes.byref(p)) == 0


def test_forward_rejects_bad_calls_before_touching_the_device():
    lib = capi.load()
    p = capi.make_params(capi.MDCN_F32, 1, 32, 8, 8, 4, 3, 3, (1, 1), (1, 1))
    assert lib.mdcn_forward(ctypes.byref(p), None) == -1  # null tensors
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(buf)
    p.input = p.offset = p.mask = p.weight = p.output = addr
    assert lib.mdcn_forward(ctypes.byref(p), None) == -4  # fused path, no workspace
    p.workspace, p.workspace_bytes = addr + 1, 1 << 30
    assert lib.mdcn_forward(ctypes.byref(p), None) == -4  # misaligned
    p2 = capi.make_params(capi.MDCN_F32, 1, 3, 8, 8, 4, 3, 3, path=capi.PATH_FUSED)
    p2.input = p2.offset = p2.mask = p2.weight = p2.output = addr
    assert lib.mdcn_forward(ctypes.byref(p2), None) == -5
    assert lib.mdcn_forward_timed(ctypes.byref(p), None, None) == -1


# ---- Python op layer ----------------------------------------------------------

def test_ext_module_exports():
    from mmcv_amd.utils import ext_loader
    ext = ext_loader.load_ext('_ext', ['modulated_deform_conv_forward',
                                       'modulated_deform_conv_backward'])
    assert ext.abi_version() == 5
    with pytest.raises(AssertionError):
        ext_loader.load_ext('_ext', ['no_such_op'])
    with pytest.raises(ImportError):
        ext_loader.load_ext('_missing', [])


def test_public_names():
    import mmcv_amd.ops as ops
    for n in ('ModulatedDeformConv2d', 'ModulatedDeformConv2dPack', 'modulated_deform_conv2d'):
        assert hasattr(ops, n)
    assert ops.MODELS.get('DCNv2') is ops.ModulatedDeformConv2dPack
    layer = ops.build_conv_layer(dict(type='DCNv2', deform_groups=2), 8, 6, 3, stride=2, padding=1)
    assert isinstance(layer, ops.ModulatedDeformConv2dPack)
    assert layer.conv_offset.out_channels == 2 * 3 * 9
    assert layer.conv_offset.stride == (2, 2)
    assert layer.weight.shape == (6, 8, 3, 3) and layer.bias.shape == (6,)
    assert layer.transposed is False and layer.output_padding == (0,)
    assert float(layer.conv_offset.weight.detach().abs().sum()) == 0.0
    bound = 1.0 / (8 * 9) ** 0.5
    assert float(layer.weight.detach().abs().max()) <= bound and float(layer.bias.detach().abs().sum()) == 0.0


def test_deprecated_kwarg():
    from mmcv_amd.ops import ModulatedDeformConv2d
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter('always')
        m = ModulatedDeformConv2d(4, 4, 3, deformable_groups=2, bias=False)
    assert m.deform_groups == 2 and m.bias is None
    assert any(issubclass(x.category, DeprecationWarning) for x in w)
    with pytest.raises(AssertionError):
        ModulatedDeformConv2d(4, 4, 3, deformable_groups=2, deform_groups=2)


def test_python_errors():
    from mmcv_amd.ops import modulated_deform_conv2d
    w = torch.zeros(4, 4, 3, 3)
    with pytest.raises(ValueError, match='Expected 4D tensor'):
        modulated_deform_conv2d(torch.zeros(4, 8, 8), torch.zeros(1, 18, 8, 8),
                                torch.zeros(1, 9, 8, 8), w)
    with pytest.raises(ValueError, match='too small'):
        modulated_deform_conv2d(torch.zeros(1, 4, 2, 2), torch.zeros(1, 18, 1, 1),
                                torch.zeros(1, 9, 1, 1), w)
    # there is no CPU implementation behind this extension: loud error, no fallback
    with pytest.raises(RuntimeError, match='implementation for device cpu not found'):
        modulated_deform_conv2d(torch.zeros(1, 4, 8, 8), torch.zeros(1, 18, 8, 8),
                                torch.zeros(1, 9, 8, 8), w, None, 1, 1)
    with pytest.raises(RuntimeError, match="kernel channels won't match"):
        modulated_deform_conv2d(torch.zeros(1, 6, 8, 8), torch.zeros(1, 18, 8, 8),
                                torch.zeros(1, 9, 8, 8), w, None, 1, 1)


def test_state_dict_upgrade():
    from mmcv_amd.ops import ModulatedDeformConv2dPack

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv2 = ModulatedDeformConv2dPack(4, 4, 3, padding=1)

    net = Net()
    sd = net.state_dict()
    old = {}
    for k, v in sd.items():
        old[k.replace('conv2.conv_offset.', 'conv2_offset.')] = torch.full_like(v, 0.5)
    assert 'conv2_offset.weight' in old
    # mmengine-style loaders hand every module the whole dict (torch's own
    # load_state_dict filters it by prefix first, which hides the legacy keys)
    missing, unexpected, errors = [], [], []
    net.conv2._load_from_state_dict(old, 'conv2.', {'version': 1}, True, missing,
                                    unexpected, errors)
    assert not missing and not errors
    assert 'conv2.conv_offset.weight' in old and 'conv2_offset.weight' not in old
    net.conv2.conv_offset._load_from_state_dict(old, 'conv2.conv_offset.', {}, True,
                                                missing, unexpected, errors)
    assert float(net.conv2.conv_offset.weight.mean()) == 0.5
    assert float(net.conv2.conv_offset.bias.mean()) == 0.5
    # current-format dicts load unchanged through torch's own loader
    net.load_state_dict(Net().state_dict())


def test_onnx_symbolic_name():
    from mmcv_amd.ops import ModulatedDeformConv2dFunction

    class G:
        def op(self, name, *args, **kw):
            return name, len(args), kw

    name, nargs, kw = ModulatedDeformConv2dFunction.symbolic(G(), 1, 2, 3, 4, None, 1, 1, 1, 1, 1)
    assert name == 'mmcv::MMCVModulatedDeformConv2d' and nargs == 4
    assert set(kw) == {'stride_i', 'padding_i', 'dilation_i', 'groups_i', 'deform_groups_i'}


def test_dcnv1_python_layer():
    import pytest
    from mmcv_amd.ops import MODELS, DeformConv2d, DeformConv2dPack
    import mmcv_amd._ext as ext
    for n in ('deform_conv_forward', 'deform_conv_backward_input', 'deform_conv_backward_parameters'):
        assert hasattr(ext, n)
    assert MODELS.get('DCN') is DeformConv2dPack
    layer = DeformConv2dPack(8, 6, 3, stride=2, padding=1, deformable_groups=2)
    assert layer.deform_groups == 2 and layer.conv_offset.out_channels == 2 * 2 * 9
    assert layer.conv_offset.stride == (2, 2) and not hasattr(layer, 'bias')
    assert float(layer.conv_offset.weight.detach().abs().sum()) == 0.0
    assert 'bias=False' in repr(layer)
    with pytest.raises(AssertionError):
        DeformConv2d(1, 1, 2, bias=True)
    with pytest.raises(AssertionError):
        DeformConv2d(3, 2, 3, groups=2)
    with pytest.raises(AssertionError):
        DeformConv2d(3, 4, 3, groups=3)
    with pytest.raises(ValueError, match='Expected 4D tensor'):
        layer(torch.zeros(8, 5, 5))
    # version-1 checkpoints name the offset conv "<module>_offset"
    sd = {'w': layer.weight.detach().clone(), 'o.weight': torch.ones(36, 8, 3, 3), 'o.bias': torch.ones(36)}
    state = {'dcn.weight': sd['w'], 'dcn_offset.weight': sd['o.weight'], 'dcn_offset.bias': sd['o.bias']}
    missing, unexpected, errors = [], [], []
    layer._load_from_state_dict(state, 'dcn.', {}, True, missing, unexpected, errors)
    assert not errors
    assert 'dcn.conv_offset.weight' in state and 'dcn.conv_offset.bias' in state
    assert 'dcn_offset.weight' not in state and 'dcn_offset.bias' not in state


def _stub_mmcv():
    """A module tree shaped like the part of mmcv that patch() touches."""
    import types
    mmcv = types.ModuleType('mmcv_stub')
    ops = types.ModuleType('mmcv_stub.ops')
    mdc = types.ModuleType('mmcv_stub.ops.modulated_deform_conv')
    dc = types.ModuleType('mmcv_stub.ops.deform_conv')
    calls = []

    class TheirExt:
        def modulated_deform_conv_forward(self, *a, **k):
            calls.append('their_forward')

        def nms(self, *a, **k):
            return 'their_nms'

    mdc.ext_module = TheirExt()
    for name in ('ModulatedDeformConv2d', 'ModulatedDeformConv2dPack', 'modulated_deform_conv2d'):
        setattr(mdc, name, object())
        setattr(ops, name, getattr(mdc, name))
    dc.DeformConv2d = ops.DeformConv2d = object()  # (no ext_module: as if mmcv was built without ops)
    ops.modulated_deform_conv, ops.deform_conv, mmcv.ops = mdc, dc, ops

    class Registry:
        def __init__(self):
            self._module_dict = {'DCNv2': 'theirs', 'Conv': 'conv'}

    return mmcv, calls, Registry()


def test_patch_rebinds_an_imported_mmcv_and_unpatch_restores_it():
    import mmcv_amd
    from mmcv_amd import ops as ours
    mmcv, calls, reg = _stub_mmcv()
    before = (mmcv.ops.modulated_deform_conv.ext_module, mmcv.ops.ModulatedDeformConv2dPack, dict(reg._module_dict))
    done = mmcv_amd.patch(mmcv, registry=reg)
    assert 'modulated_deform_conv.ext_module' in done and 'MODELS[DCNv2]' in done
    ext = mmcv.ops.modulated_deform_conv.ext_module
    # CPU tensors keep going to the module mmcv loaded, ops of other layers too
    ext.modulated_deform_conv_forward(torch.zeros(1))
    assert calls == ['their_forward'] and ext.nms() == 'their_nms'
    # device tensors go to this package's op: here it rejects the bogus call itself
    class FakeCuda:
        is_cuda = True
    with pytest.raises(TypeError):
        ext.modulated_deform_conv_forward(FakeCuda())
    assert mmcv.ops.deform_conv.ext_module.deform_conv_forward.__name__ == 'deform_conv_forward'
    assert mmcv.ops.ModulatedDeformConv2dPack is ours.ModulatedDeformConv2dPack
    assert mmcv.ops.modulated_deform_conv.modulated_deform_conv2d is ours.modulated_deform_conv2d
    assert mmcv.ops.DeformConv2d is ours.DeformConv2d
    assert reg._module_dict['DCNv2'] is ours.ModulatedDeformConv2dPack and reg._module_dict['Conv'] == 'conv'
    assert reg._module_dict['DCN'] is ours.DeformConv2dPack
    mmcv_amd.unpatch()
    assert mmcv.ops.modulated_deform_conv.ext_module is before[0]
    assert mmcv.ops.ModulatedDeformConv2dPack is before[1]
    assert reg._module_dict == before[2]
    assert not hasattr(mmcv.ops.deform_conv, 'ext_module')


def test_patch_ext_only_keeps_mmcv_classes():
    import mmcv_amd
    mmcv, _, reg = _stub_mmcv()
    pack = mmcv.ops.ModulatedDeformConv2dPack
    done = mmcv_amd.patch(mmcv.ops, classes=False, registry=reg)
    assert done == ['modulated_deform_conv.ext_module', 'deform_conv.ext_module']
    assert mmcv.ops.ModulatedDeformConv2dPack is pack and reg._module_dict['DCNv2'] == 'theirs'
    mmcv_amd.unpatch()


def test_asm_check_flags_scalar_written_too_close_to_inline_vector_memory():
    """The build's scan of the device assembly (mmcv_amd/asm_check.py) on synthetic text."""
    from mmcv_amd import asm_check
    bad = '''
	v_readlane_b32 s7, v253, 57
	;;#ASMSTART
	global_store_dwordx4 v1, v[66:69], s[6:7] sc1
	;;#ASMEND
'''
    hits = asm_check.violations(bad)
    assert len(hits) == 1 and hits[0][2] == [7] and hits[0][3] == 0
    # enough wait states, another register, or an instruction the compiler emitted itself: fine
    ok = '''
	v_readlane_b32 s7, v253, 57
	;;#ASMSTART
	s_nop 4
	global_store_dwordx4 v1, v[66:69], s[6:7] sc1
	;;#ASMEND
	v_readlane_b32 s9, v253, 58
	;;#ASMSTART
	global_load_dwordx4 v[2:5], v1, s[6:7] offset:64
	;;#ASMEND
	v_readfirstlane_b32 s10, v4
	s_nop 4
	global_load_dword v9, v1, s[10:11]
	v_readlane_b32 s12, v253, 1
	global_load_dword v9, v1, s[12:13]
'''
    assert asm_check.violations(ok) == []
    # five instructions in between are as good as an s_nop
    spaced = '\tv_readlane_b32 s7, v253, 57\n' + '\tv_mov_b32_e32 v2, v3\n' * 5 + \
        '\t;;#ASMSTART\n\tglobal_load_dwordx4 v[2:5], v1, s[6:7]\n\t;;#ASMEND\n'
    assert asm_check.violations(spaced) == []
    assert len(asm_check.violations(spaced.replace('\tv_mov_b32_e32 v2, v3\n' * 5, '\tv_mov_b32_e32 v2, v3\n' * 4))) == 1


def test_asm_check_flags_registers_touched_while_an_inline_load_is_in_flight():
    """Second scan of mmcv_amd/asm_check.py: a register that an asm-issued load has not
    delivered yet (no wait that names it, no wait for count 0) must not be touched --
    the compiler would otherwise copy stale data or reuse the register as a temporary."""
    from mmcv_amd import asm_check
    head = 'kern:\n'
    load = '\t;;#ASMSTART\n\tglobal_load_dwordx4 v[2:5], v[8:9], off\n\t;;#ASMEND\n'
    wait = '\t;;#ASMSTART\n\ts_waitcnt vmcnt(8) ; v[2:5] v[10:13]\n\t;;#ASMEND\n'
    use = '\tv_xor_b32_e32 v20, v2, v20\n'
    assert asm_check.inflight_violations(head + load + wait + use + '\ts_endpgm\n') == []
    # a copy before the wait, or a wait that names other registers
    early = asm_check.inflight_violations(head + load + '\tv_mov_b64_e32 v[36:37], v[4:5]\n' + wait + use + '\ts_endpgm\n')
    assert [(v[1], v[3]) for v in early] == [(5, (4, 5))]
    other = wait.replace('v[2:5]', 'v[14:17]')
    assert len(asm_check.inflight_violations(head + load + other + use + '\ts_endpgm\n')) == 1
    # a wait for everything releases everything, named or not, asm or compiler
    assert asm_check.inflight_violations(head + load + '\ts_waitcnt vmcnt(0)\n' + use + '\ts_endpgm\n') == []
    assert len(asm_check.inflight_violations(head + load + '\ts_waitcnt vmcnt(3)\n' + use + '\ts_endpgm\n')) == 1
    # loads the compiler issued itself are its own business
    assert asm_check.inflight_violations(head + '\tglobal_load_dwordx4 v[2:5], v[8:9], off\n' + use + '\ts_endpgm\n') == []
    # around a loop: the load at the bottom of the body is in flight at the top
    loop = (head + load + '.LBB0_1:\n' + '\tv_mov_b32_e32 v30, v3\n' + wait + use + load +
            '\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n')
    hits = asm_check.inflight_violations(loop)
    assert len(hits) == 1 and hits[0][2].startswith('v_mov_b32_e32 v30, v3')
    # a rotated loop (latch placed before the header in the text) is followed along its edges, not in text order
    rotated = (head + load + '\ts_branch .LBB0_2\n' + '.LBB0_1:\n' + use + load + '.LBB0_2:\n' + wait +
               '\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n')
    assert asm_check.inflight_violations(rotated) == []
    # LDS reads: the other counter
    ds = '\t;;#ASMSTART\n\tds_read_b128 v[40:43], v7 offset:4096\n\t;;#ASMEND\n'
    dwait = '\t;;#ASMSTART\n\ts_waitcnt lgkmcnt(2) ; v[40:43]\n\t;;#ASMEND\n'
    mfma = '\tv_mfma_f32_32x32x16_bf16 v[100:115], v[40:43], v[44:47], v[100:115]\n'
    assert asm_check.inflight_violations(head + ds + dwait + mfma + '\ts_endpgm\n') == []
    assert len(asm_check.inflight_violations(head + ds + mfma + dwait + '\ts_endpgm\n')) == 1
    assert len(asm_check.inflight_violations(head + ds + '\ts_waitcnt vmcnt(0)\n' + mfma + '\ts_endpgm\n')) == 1


def test_asm_check_follows_role_markers():
    """A kernel that branches on a wave's role in two places: without markers the scan also
    follows the paths that take one role's side first and the other's later, and reports them;
    with `; mdcn-role` markers in the role-specific blocks those paths are dropped."""
    from mmcv_amd import asm_check
    load = lambda r: f'\t;;#ASMSTART\n\tglobal_load_dwordx4 v[{r}:{r + 3}], v[8:9], off\n\t;;#ASMEND\n'
    wait = lambda r: f'\t;;#ASMSTART\n\ts_waitcnt vmcnt(4) ; v[{r}:{r + 3}]\n\t;;#ASMEND\n'
    mark = lambda name: f'\t;;#ASMSTART\n\t; mdcn-role {name}\n\t;;#ASMEND\n'
    def kernel(marked):
        m = mark if marked else (lambda name: '')
        return ('kern:\n'
                '\ts_cbranch_scc1 .LBB0_2\n'                       # role test 1
                + m('early') + load(20) + '\ts_branch .LBB0_3\n'
                '.LBB0_2:\n' + m('late') + load(30) +
                '.LBB0_3:\n'
                '\ts_cbranch_scc1 .LBB0_5\n'                       # role test 2 (same flag)
                + m('early') + wait(20) + '\tv_mov_b32_e32 v1, v20\n' + load(30) + wait(30) + '\ts_branch .LBB0_6\n'
                '.LBB0_5:\n' + m('late') + wait(30) + '\tv_mov_b32_e32 v1, v30\n' + load(20) + wait(20) +
                '.LBB0_6:\n\ts_endpgm\n')
    assert len(asm_check.inflight_violations(kernel(False))) == 2   # the two mixed paths reissue a locked set
    assert asm_check.inflight_violations(kernel(True)) == []
    # a real violation on a consistent path is still found
    bad = kernel(True).replace(wait(20) + '\tv_mov_b32_e32 v1, v20\n', '\tv_mov_b32_e32 v1, v20\n' + wait(20))
    assert len(asm_check.inflight_violations(bad)) == 1


def test_asm_check_counts_wait_states_along_branches():
    """A reload of a scalar at the end of a block reaches an inline-asm memory instruction at a
    branch target as well: the scan counts wait states along every edge into the instruction,
    not only along the text in front of it."""
    from mmcv_amd import asm_check
    load = '\t;;#ASMSTART\n\tglobal_load_dwordx4 v[2:5], v1, s[6:7]\n\t;;#ASMEND\n'
    # loop whose latch reloads s7 right in front of the back edge; the loop header starts with the load
    loop = ('kern:\n\ts_mov_b32 s1, 0\n\tv_mov_b32_e32 v9, v8\n' * 1 + '\tv_mov_b32_e32 v9, v8\n' * 5 +
            '.LBB0_1:\n' + load + '\tv_mov_b32_e32 v9, v8\n' * 6 +
            '\tv_readlane_b32 s7, v253, 57\n\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n')
    hits = asm_check.violations(loop)
    assert len(hits) == 1 and hits[0][2] == [7] and hits[0][3] == 1   # (the branch itself is one slot)
    # far enough from the back edge, or an s_nop at the head of the asm statement: fine
    assert asm_check.violations(loop.replace('\tv_readlane_b32 s7, v253, 57\n', '\tv_readlane_b32 s7, v253, 57\n' +
                                             '\tv_mov_b32_e32 v9, v8\n' * 4)) == []
    assert asm_check.violations(loop.replace('\tglobal_load_dwordx4 v[2:5]', '\ts_nop 4\n\tglobal_load_dwordx4 v[2:5]')) == []
    # a forward branch over harmless code into the statement
    fwd = ('kern:\n\tv_readlane_b32 s6, v253, 3\n\ts_cbranch_scc1 .LBB0_2\n' + '\tv_mov_b32_e32 v9, v8\n' * 8 +
           '.LBB0_2:\n' + load + '\ts_endpgm\n')
    assert len(asm_check.violations(fwd)) == 1


def test_asm_check_verifies_wait_counts():
    """Third scan of mmcv_amd/asm_check.py: a wait that names a register must not allow more
    loads in flight than were issued behind that register's load."""
    from mmcv_amd import asm_check
    head = 'kern:\n\t;;#ASMSTART\n\t; mdcn-counted-waits\n\t;;#ASMEND\n'
    load = lambda r: f'\t;;#ASMSTART\n\tglobal_load_dwordx4 v[{r}:{r + 3}], v[8:9], off\n\t;;#ASMEND\n'
    wait = lambda n, r: f'\t;;#ASMSTART\n\ts_waitcnt vmcnt({n}) ; v[{r}:{r + 3}]\n\t;;#ASMEND\n'
    tail = '\ts_endpgm\n'
    notes = []
    ok = head + load(20) + load(30) + load(40) + wait(2, 20) + wait(1, 30) + wait(0, 40) + tail
    assert asm_check.wait_count_findings(ok, notes) == []
    assert sorted(n[2:] for n in notes) == [(0, 0), (1, 0), (2, 0)]          # every count exactly right
    bad = asm_check.wait_count_findings(head + load(20) + load(30) + load(40) + wait(3, 20) + tail)
    assert len(bad) == 4 and bad[0][4] == 2                                  # v20..v23, two loads behind them
    # stores and compiler loads in between: stores do not count, loads do
    mixed = head + load(20) + '\tglobal_store_dwordx4 v[8:9], v[50:53], off\n' + load(30) + wait(2, 20) + tail
    assert len(asm_check.wait_count_findings(mixed)) == 4
    assert asm_check.wait_count_findings(mixed.replace('global_store_dwordx4 v[8:9], v[50:53], off',
                                                       'global_load_dword v60, v[8:9], off')) == []
    # a loop: the count must hold on the shortest way round
    loop = (head + load(20) + '.LBB0_1:\n' + load(30) + wait(1, 20) + load(20) + wait(1, 30) +
            '\ts_cbranch_scc1 .LBB0_1\n' + wait(0, 20) + tail)
    assert asm_check.wait_count_findings(loop) == []
    assert len(asm_check.wait_count_findings(loop.replace(wait(1, 30), wait(2, 30)))) == 4
    # direct-to-LDS copies: a wait marked `lds-copies` is about the youngest of them
    copy = '\t;;#ASMSTART\n\tglobal_load_lds_dwordx4 v7, s[2:3] offset:1024\n\t;;#ASMEND\n'
    bar = lambda n: f'\t;;#ASMSTART\n\ts_waitcnt vmcnt({n}) lgkmcnt(0) ; lds-copies\n\ts_barrier\n\t;;#ASMEND\n'
    assert asm_check.wait_count_findings(head + copy + copy + load(20) + load(30) + bar(2) + wait(0, 20) + tail) == []
    assert len(asm_check.wait_count_findings(head + copy + copy + load(20) + load(30) + bar(3) + tail)) == 1
    # kernels that do not ask for the check are left alone
    assert asm_check.wait_count_findings('kern:\n' + load(20) + wait(5, 20) + tail) == []


def test_built_library_passes_the_assembly_scans():
    """The device assembly the library in mmcv_amd/lib was built from (kept beside it by
    mmcv_amd.build.build_hip) passes all three scans, every count-based wait of the 256-pixel
    kernel is exactly right on its shortest path, and a count shifted by one is found."""
    import os
    import re
    import pytest
    from mmcv_amd import asm_check, build
    path = os.path.join(build.LIBDIR, 'libmdcn_hip.s')
    if not os.path.exists(path) or os.path.getmtime(path) + 5 < os.path.getmtime(build.HIP_LIB):
        pytest.skip('no device assembly beside the built library (mmcv_amd/lib/libmdcn_hip.s): built elsewhere '
                    'or by a build without the scans')
    text = open(path).read()
    assert asm_check.violations(text) == []
    assert asm_check.inflight_violations(text) == []
    notes = []
    assert asm_check.wait_count_findings(text, notes) == []
    eight_wave = [n for n in notes if 'fused3_kernel' in n[0]]
    assert len(eight_wave) >= 40
    # waits for a count above zero are tight; waits for zero may have any number of loads behind them
    assert all(slack == 0 for _, _, count, slack in eight_wave if count > 0), \
        [n for n in eight_wave if n[2] > 0 and n[3] != 0][:5]
    # shift one count of the 256-pixel kernel up by one: found
    k0 = text.index('fused3_kernel')
    m = re.compile(r's_waitcnt vmcnt\(([1-9]\d*)\) ; v\[').search(text, k0)
    assert m
    shifted = text[:m.start(1)] + str(int(m.group(1)) + 1) + text[m.end(1):]
    assert len(asm_check.wait_count_findings(shifted)) >= 1


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus above 1 ends with a message and exit status 2 before anything
    touches a device."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert 'ONE GPU' in r.stderr
    assert r.stdout.strip() == ''
