"""ctypes binding of ``libflyhip.so`` (the C ABI declared in ``include/flyhip.h``).

The library is loaded lazily from the package directory.  There is no CPU fallback: if the
shared object is missing, or a tensor is not on a GPU, the call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libflyhip.so')

c_int, c_i64, c_float, c_vp = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
c_u64 = ctypes.c_uint64

# name -> argument ctypes, in the order of include/flyhip.h
SIGNATURES = {
    'flyhip_version': [],
    'flyhip_sb_plan': [c_int] * 5 + [ctypes.POINTER(c_int)] * 3,
    'flyhip_sb_plan_for': [c_int] * 8 + [ctypes.POINTER(c_int)] * 3,
    'flyhip_sb_time_next_fwd': [c_vp, c_vp],
    'flyhip_sb_kv_reduce': [c_vp] * 14 + [c_int] + [c_i64] * 3 + [c_vp] * 2 + [c_int] * 8 + [c_i64] * 6 + [c_float, c_int, c_vp],
    'flyhip_sblocal_fwd': [c_vp] * 13 + [c_vp] * 2 + [c_int] + [c_vp] * 4 + [c_int] * 10 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_sblocal_forward': [c_vp] * 8 + [c_i64] + [c_int] * 9 + [c_i64] * 12 + [c_float, c_int, c_int, c_float, c_u64, c_vp],
    'flyhip_sblocal_fwd_static': [c_vp] * 13 + [c_vp] * 2 + [c_int] + [c_vp] * 3 + [c_int] * 10 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_sblocal_bwd_band': [c_vp] * 12 + [c_int] * 7 + [c_float, c_int, c_vp],
    'flyhip_sblocal_bwd_band_dropout': [c_vp] * 12 + [c_int] * 7 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_sblocal_bwd_band_masked': [c_vp] * 13 + [c_int] * 7 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_sblocal_bwd': [c_vp] * 14 + [c_int] * 7 + [c_float, c_int, c_vp],
    'flyhip_sblocal_bwd_prep': [c_vp] * 18 + [c_i64] + [c_int] * 7 + [c_float, c_vp],
    'flyhip_sblocal_bwd_pieces': [c_vp] * 12 + [c_i64] + [c_int] * 7 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_sbblocksparse_bwd_pieces': [c_vp] * 15 + [c_int] * 2 + [c_vp, c_i64] + [c_int] * 6 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_sbblocksparse_fwd': [c_vp] * 15 + [c_int] * 2 + [c_vp] * 4 + [c_int] * 8 + [c_i64] * 12 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_local_fwd_lse': [c_vp] * 6 + [c_int] * 7 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_local_fwd_dropout': [c_vp] * 6 + [c_int] * 7 + [c_i64] * 12 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_local_fwd_masked': [c_vp] * 7 + [c_int] * 7 + [c_i64] * 12 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_local_fwd': [c_vp] * 5 + [c_int] * 7 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_local_bwd': [c_vp] * 11 + [c_int] * 6 + [c_i64] * 24 + [c_float, c_int, c_vp],
    'flyhip_bs_sdd': [c_vp] * 4 + [c_int] + [c_vp] * 3 + [c_int] * 2 + [c_vp] * 3 + [c_int] * 3 + [c_i64] * 8 + [c_int, c_vp],
    'flyhip_bs_attn_bwd': [c_vp] * 16 + [c_int] * 5 + [c_i64] * 24 + [c_float, c_int, c_float, c_u64, c_vp, c_i64, c_vp, c_i64, c_vp],
    'flyhip_bs_sdd_dsoftmax': [c_vp] * 8 + [c_int] * 6 + [c_i64] * 6 + [c_float, c_int, c_vp],
    'flyhip_bs_sdd_kmajor': [c_vp] * 8 + [c_int] * 8 + [c_i64] * 6 + [c_int, c_vp],
    'flyhip_bs_dsd': [c_vp] * 9 + [c_int] * 6 + [c_i64] * 9 + [c_int, c_vp],
    'flyhip_bs_dds': [c_vp] * 8 + [c_int] * 8 + [c_i64] * 9 + [c_int, c_vp],
    'flyhip_bs_attn_lse': [c_vp] * 8 + [c_int, c_vp, c_i64] + [c_int] * 5 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_bs_attn_masks': [c_vp] * 8 + [c_int, c_vp, c_i64, c_vp, c_i64] + [c_int] * 5 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_bs_sdd_prob_dsoftmax': [c_vp] * 13 + [c_int] * 6 + [c_i64] * 18 + [c_float, c_int, c_vp],
    'flyhip_bs_sdd_prob_dsoftmax_dropout': [c_vp] * 13 + [c_int] * 6 + [c_i64] * 18 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_bs_attn_dropout': [c_vp] * 8 + [c_int, c_vp, c_i64, c_vp, c_i64] + [c_int] * 5 + [c_i64] * 12 + [c_float, c_int, c_float, c_u64, c_vp],
    'flyhip_bs_sdd_prob': [c_vp] * 7 + [c_int] * 6 + [c_i64] * 6 + [c_float, c_int, c_vp],
    'flyhip_bs_attn': [c_vp] * 7 + [c_int, c_vp, c_i64] + [c_int] * 5 + [c_i64] * 12 + [c_float, c_int, c_vp],
    'flyhip_bs_softmax': [c_vp] * 4 + [c_int] * 5 + [c_i64, c_float, c_vp, c_i64, c_int, c_vp, c_i64,
                                                    c_int, c_int, c_vp],
    'flyhip_bs_softmax_bwd': [c_vp] * 5 + [c_int] * 4 + [c_i64, c_float, c_int, c_vp],
    'flyhip_bs_rowreduce': [c_vp] * 4 + [c_int] * 3 + [c_i64, c_int, c_int, c_vp],
}

_lib = None


def load():
    """Load libflyhip.so (once) and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f'{LIB_PATH} is missing: build it with `python -m fly_amd.build` '
                           '(there is no fallback implementation)')
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    lib.flyhip_sb_workspace_bytes.argtypes = [c_int] * 9
    lib.flyhip_sb_workspace_bytes.restype = c_i64
    lib.flyhip_sblocal_bwd_prep_scratch.argtypes = [c_int] * 5
    lib.flyhip_sblocal_bwd_prep_scratch.restype = c_i64
    lib.flyhip_sblocal_bwd_image_bytes.argtypes = [c_int] * 4
    lib.flyhip_sblocal_bwd_image_bytes.restype = c_i64
    lib.flyhip_sblocal_bwd_parts_floats.argtypes = [c_int] * 6
    lib.flyhip_sblocal_bwd_parts_floats.restype = c_i64
    lib.flyhip_sbblocksparse_bwd_parts_floats.argtypes = [c_int] * 6
    lib.flyhip_sbblocksparse_bwd_parts_floats.restype = c_i64
    lib.flyhip_last_error.argtypes = []
    lib.flyhip_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


def call(name, *args):
    """Invoke an entry point; a negative return code becomes a RuntimeError with the library's
    message."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f'{name} failed ({rc}): {lib.flyhip_last_error().decode()}')


DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
SB_EXACT_FP32 = 1          # flag of flyhip_sblocal_forward / flyhip_sb_workspace_bytes (FLYHIP_SB_EXACT_FP32)


def table_ptr(t):
    """Address of an index table that the kernels only read through the ranges of another one: an empty table (a
    layout without blocks) has no storage, so a one-element stand-in is passed; no range points into it."""
    if t.numel() == 0:
        t = torch.zeros(1, dtype=t.dtype, device=t.device)
        _KEEP_ALIVE.append(t)
        del _KEEP_ALIVE[:-8]
    return t.data_ptr()


_KEEP_ALIVE = []


def dtype_code(t):
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError(f'unsupported dtype {t.dtype}; expected float32, bfloat16 or float16') from None


def ptr(t):
    """Device pointer of a tensor, or NULL for None."""
    return None if t is None else t.data_ptr()


def stream_ptr(device):
    """The hipStream_t PyTorch currently enqueues on for `device`."""
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError('the HIP kernels only accept GPU tensors (no CPU implementation is shipped)')
    dev = {t.device for t in tensors if t is not None}
    if len(dev) > 1:
        raise ValueError(f'tensors live on different devices: {sorted(map(str, dev))}')
