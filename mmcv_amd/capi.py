"""ctypes binding of the C ABI in ``include/mdcn.h`` (``lib/libmdcn_hip.so``).

This is the binding a non-PyTorch caller would write; the tests use it to drive
the library with raw device pointers.  ``import torch`` first so that the process
holds a single HIP runtime."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libmdcn_hip.so')

MDCN_F32, MDCN_F16, MDCN_BF16, MDCN_F64 = 0, 1, 2, 3
PATH_AUTO, PATH_FUSED, PATH_DIRECT, PATH_FUSED_SPLIT, PATH_FUSED_WIDE, PATH_FUSED_NARROW = 0, 1, 2, 3, 4, 5
MDCN_OK = 0
NOALLOC_SCRATCH_BYTES = 64 << 20

EXPORTS = ('mdcn_abi_version', 'mdcn_set_pass_limits', 'mdcn_status_string', 'mdcn_output_size',
           'mdcn_fused_eligible', 'mdcn_forward_kernels', 'mdcn_workspace_bytes', 'mdcn_forward', 'mdcn_forward_noalloc',
           'mdcn_forward_timed', 'mdcn_pack_workspace_bytes', 'mdcn_pack_forward',
           'mdcn_pack_forward_timed', 'mdcn_backward_workspace_bytes', 'mdcn_backward')


class MdcnParams(ctypes.Structure):
    _fields_ = ([(n, ctypes.c_void_p) for n in
                 ('input', 'offset', 'mask', 'weight', 'bias', 'output',
                  'workspace')] +
                [('workspace_bytes', ctypes.c_size_t)] +
                [(n, ctypes.c_int32) for n in
                 ('dtype', 'path', 'N', 'Cin', 'H', 'W', 'Cout', 'kh', 'kw',
                  'sh', 'sw', 'ph', 'pw', 'dh', 'dw', 'groups', 'dgroups', 'input_nhwc', 'no_k_split')])


class MdcnPackParams(ctypes.Structure):
    _fields_ = [('conv', MdcnParams), ('offset_weight', ctypes.c_void_p),
                ('offset_bias', ctypes.c_void_p), ('raw', ctypes.c_void_p),
                ('unmodulated', ctypes.c_int32)]


class MdcnBwdParams(ctypes.Structure):
    _fields_ = [('conv', MdcnParams)] + [(n, ctypes.c_void_p) for n in
                                         ('grad_output', 'grad_input', 'grad_offset', 'grad_mask',
                                          'grad_weight', 'grad_bias')]


_lib = None


def load():
    """dlopen the library (raises OSError when it is not built)."""
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(LIB_PATH)
        P = ctypes.POINTER(MdcnParams)
        lib.mdcn_abi_version.restype = ctypes.c_int
        lib.mdcn_abi_version.argtypes = []
        lib.mdcn_set_pass_limits.restype = None
        lib.mdcn_set_pass_limits.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        lib.mdcn_status_string.restype = ctypes.c_char_p
        lib.mdcn_status_string.argtypes = [ctypes.c_int]
        lib.mdcn_output_size.restype = ctypes.c_int
        lib.mdcn_output_size.argtypes = [P, ctypes.POINTER(ctypes.c_int32),
                                         ctypes.POINTER(ctypes.c_int32)]
        lib.mdcn_fused_eligible.restype = ctypes.c_int
        lib.mdcn_fused_eligible.argtypes = [P]
        lib.mdcn_forward_kernels.restype = ctypes.c_char_p
        lib.mdcn_forward_kernels.argtypes = [P]
        lib.mdcn_workspace_bytes.restype = ctypes.c_size_t
        lib.mdcn_workspace_bytes.argtypes = [P]
        lib.mdcn_forward.restype = ctypes.c_int
        lib.mdcn_forward.argtypes = [P, ctypes.c_void_p]
        lib.mdcn_forward_noalloc.restype = ctypes.c_int
        lib.mdcn_forward_noalloc.argtypes = [P, ctypes.c_void_p]
        lib.mdcn_forward_timed.restype = ctypes.c_int
        lib.mdcn_forward_timed.argtypes = [P, ctypes.c_void_p,
                                           ctypes.POINTER(ctypes.c_float)]
        PP = ctypes.POINTER(MdcnPackParams)
        lib.mdcn_pack_workspace_bytes.restype = ctypes.c_size_t
        lib.mdcn_pack_workspace_bytes.argtypes = [PP]
        lib.mdcn_pack_forward.restype = ctypes.c_int
        lib.mdcn_pack_forward.argtypes = [PP, ctypes.c_void_p]
        lib.mdcn_pack_forward_timed.restype = ctypes.c_int
        lib.mdcn_pack_forward_timed.argtypes = [PP, ctypes.c_void_p,
                                                ctypes.POINTER(ctypes.c_float)]
        BP = ctypes.POINTER(MdcnBwdParams)
        lib.mdcn_backward_workspace_bytes.restype = ctypes.c_size_t
        lib.mdcn_backward_workspace_bytes.argtypes = [BP]
        lib.mdcn_backward.restype = ctypes.c_int
        lib.mdcn_backward.argtypes = [BP, ctypes.c_void_p]
        _lib = lib
    return _lib


def status_string(rc):
    return load().mdcn_status_string(rc).decode()


def make_params(dtype, N, Cin, H, W, Cout, kh, kw, stride=(1, 1), padding=(0, 0),
                dilation=(1, 1), groups=1, deform_groups=1, path=PATH_AUTO):
    p = MdcnParams()
    p.dtype, p.path = dtype, path
    p.N, p.Cin, p.H, p.W, p.Cout, p.kh, p.kw = N, Cin, H, W, Cout, kh, kw
    p.sh, p.sw = stride
    p.ph, p.pw = padding
    p.dh, p.dw = dilation
    p.groups, p.dgroups = groups, deform_groups
    return p


def output_size(p):
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    rc = load().mdcn_output_size(ctypes.byref(p), ctypes.byref(ho), ctypes.byref(wo))
    return rc, ho.value, wo.value
