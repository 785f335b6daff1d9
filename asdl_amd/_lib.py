"""ctypes binding of libasdl_amd.so (the C ABI declared in include/asdl_amd.h).

The library is loaded from asdl_amd/lib/ next to this file.  There is no fallback: if the
library has not been built the import of any kernel wrapper raises.
"""
import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libasdl_amd.so')
HEADER_PATH = os.path.join(os.path.dirname(_HERE), 'include', 'asdl_amd.h')

_lib = None

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_f32 = ctypes.c_float
c_ptr = ctypes.c_void_p
c_size = ctypes.c_size_t

_SIGNATURES = {
    'ak_version': (c_int, []),
    'ak_error_string': (ctypes.c_char_p, [c_int]),
    'ak_syrk_tn_ws_bytes': (c_size, [c_i64, c_i64]),
    'ak_syrk_tn': (c_int, [c_ptr, c_int, c_i64, c_i64, c_i64, c_f32, c_f32, c_ptr, c_i64, c_ptr, c_size, c_ptr]),
    'ak_conv_syrk_ws_bytes': (c_size, [c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_int, c_int, c_int]),
    'ak_conv_syrk': (c_int, [c_ptr, c_int, c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_f32, c_f32, c_ptr, c_i64, c_ptr, c_size, c_ptr]),
    'ak_conv_syrk_nhwc_ws_bytes': (c_size, [c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_int, c_int, c_int]),
    'ak_conv_syrk_nhwc': (c_int, [c_ptr, c_int, c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_f32, c_f32, c_ptr, c_i64, c_ptr, c_size, c_ptr]),
    'ak_syrk_group_eligible': (c_int, [c_ptr]),
    'ak_syrk_group_sizes': (c_int, [c_ptr, c_int, c_ptr, c_ptr]),
    'ak_syrk_group_launch': (c_int, [c_ptr, c_int, c_ptr, c_ptr, c_size, c_ptr, c_size, c_ptr]),
    'ak_kron_damping': (c_int, [c_ptr, c_ptr, c_ptr, c_int, c_f32, c_f32, c_ptr, c_ptr, c_ptr]),
    'ak_chol_inv_ws_bytes': (c_size, [c_i64, c_int]),
    'ak_chol_inv_batched': (c_int, [c_ptr, c_ptr, c_i64, c_int, c_ptr, c_int, c_ptr, c_int, c_ptr, c_ptr, c_size, c_ptr]),
    'ak_chol_group_plan_bytes': (c_size, [c_ptr, c_int]),
    'ak_chol_group_ws_bytes': (c_size, [c_ptr, c_int]),
    'ak_chol_group_plan': (c_int, [c_ptr, c_int, c_ptr, c_size]),
    'ak_chol_group_plan_launches': (c_int, [c_ptr]),
    'ak_chol_inv_grouped': (c_int, [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_ptr, c_int, c_ptr, c_ptr, c_size, c_ptr]),
    'ak_unit_wise_ws_bytes': (c_size, [c_i64, c_i64, c_i64]),
    'ak_unit_wise_stats': (c_int, [c_ptr, c_int, c_i64, c_i64, c_i64, c_ptr, c_int, c_i64, c_i64, c_i64, c_ptr, c_ptr,
                                   c_i64, c_i64, c_i64, c_f32, c_f32, c_ptr, c_ptr, c_size, c_ptr]),
    'ak_unit_wise_inv': (c_int, [c_ptr, c_i64, c_f32, c_ptr, c_ptr, c_ptr]),
    'ak_unit_wise_mvp': (c_int, [c_ptr, c_i64, c_ptr, c_ptr, c_f32, c_ptr]),
    'ak_unit_wise_mvp_grouped': (c_int, [c_ptr, c_int, c_i64, c_f32, c_ptr]),
    'ak_unit_wise_inv_grouped': (c_int, [c_ptr, c_int, c_i64, c_ptr]),
    'ak_identity_where_zero': (c_int, [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_ptr]),
    'ak_conv_patch_sum': (c_int, [c_ptr, c_int, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_int,
                                  c_int, c_int, c_int, c_int, c_f32, c_f32, c_ptr, c_i64, c_ptr]),
    'ak_kron_damping_swift': (c_int, [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_f32, c_f32, c_ptr, c_ptr, c_ptr]),
    'ak_smw_inv_ws_bytes': (c_size, [c_i64, c_i64]),
    'ak_smw_inv': (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_ptr, c_i64, c_ptr, c_ptr, c_size, c_ptr]),
    'ak_smw_finish': (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_ptr]),
    'ak_event_create': (c_int, [ctypes.POINTER(ctypes.c_void_p), c_int]),
    'ak_event_destroy': (c_int, [c_ptr]),
    'ak_event_record': (c_int, [c_ptr, c_ptr]),
    'ak_stream_order': (c_int, [c_ptr, c_ptr, c_ptr]),
    'ak_event_elapsed_ms': (c_int, [c_ptr, c_ptr, ctypes.POINTER(ctypes.c_float)]),
    'ak_copy_bytes': (c_int, [c_ptr, c_ptr, c_i64, c_ptr]),
    'ak_absmax_block': (c_i64, []),
    'ak_absmax_grouped': (c_int, [c_ptr, c_int, c_i64, c_ptr]),
    'ak_tril_pack': (c_int, [c_ptr, c_i64, c_i64, c_ptr, c_ptr]),
    'ak_tril_unpack': (c_int, [c_ptr, c_i64, c_ptr, c_i64, c_ptr]),
    'ak_gemm_f32': (c_int, [c_int, c_int, c_i64, c_i64, c_i64, c_f32, c_ptr, c_i64, c_ptr, c_i64, c_f32,
                            c_ptr, c_i64, c_int, c_i64, c_i64, c_i64, c_ptr]),
    'ak_gemm_f32_split': (c_int, [c_int, c_int, c_int, c_i64, c_i64, c_i64, c_f32, c_ptr, c_i64, c_ptr, c_i64, c_f32,
                                  c_ptr, c_i64, c_int, c_i64, c_i64, c_i64, c_ptr]),
    'ak_gemm_f32_grouped': (c_int, [c_int, c_ptr, c_int, c_i64, c_ptr]),
    'ak_gemv_f32_grouped': (c_int, [c_ptr, c_int, c_i64, c_f32, c_ptr]),
    'ak_weight_layout_max_row': (c_i64, []),
    'ak_weight_layout_grouped': (c_int, [c_ptr, c_int, c_i64, c_int, c_ptr]),
    'ak_kron_precond_ws_bytes': (c_size, [c_i64, c_i64]),
    'ak_kron_precond': (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_ptr, c_f32, c_ptr, c_size, c_ptr]),
    'ak_kron_precond_static_max_floats': (c_i64, []),
    'ak_kron_precond_static': (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_ptr, c_f32, c_ptr]),
    'ak_inv_root_ws_bytes': (c_size, [c_i64, c_int]),
    'ak_inv_root_newton': (c_int, [c_ptr, c_i64, c_int, c_i64, c_int, c_f32, c_ptr, c_int, c_f32, c_int, c_f32,
                                   c_ptr, c_i64, c_ptr, c_ptr, c_size, c_ptr]),
    'ak_inv_root_active_offset': (c_size, [c_i64, c_int]),
    'ak_inv_root_plane_format': (c_int, [c_i64, c_int, c_f32]),
    'ak_inv_root_newton_part': (c_int, [c_int, c_int, c_ptr, c_i64, c_int, c_i64, c_int, c_f32, c_ptr, c_int, c_f32,
                                        c_int, c_f32, c_ptr, c_i64, c_ptr, c_ptr, c_size, c_ptr]),
}


def declared_symbols():
    """Names of every function declared in include/asdl_amd.h."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ak_[a-z0-9_]+)\s*\(', text)))


def load():
    """Loads the library (once) and sets argument / result types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f'{LIB_PATH} is missing: build it with `python -m asdl_amd.build` (hipcc, gfx950). '
            'asdl_amd has no CPU or PyTorch fallback for its kernels.')
    import torch  # noqa: F401  (makes the process use the HIP runtime PyTorch ships)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class KernelError(RuntimeError):
    pass


def check(code, what):
    if code != 0:
        msg = load().ak_error_string(code)
        raise KernelError(f'{what} failed: {msg.decode() if msg else code}')
