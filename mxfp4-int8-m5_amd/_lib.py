"""ctypes binding of libscmx.so (the C ABI declared in include/scmx.h).  There is no fallback: a missing or
incomplete library raises, and so does every call that returns a negative status."""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libscmx.so")


class CFormat(C.Structure):
    _fields_ = [("block", C.c_int32), ("bc_bits", C.c_int32), ("n_mult", C.c_int32), ("code_mag", C.c_int32 * 8),
                ("mult", C.c_int32 * 16)]


_P, _I, _L, _F, _Z = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
_FMT = C.POINTER(CFormat)

# symbol -> (restype, argtypes): mirrors include/scmx.h line by line
SIGNATURES = {
    "scmx_version": (C.c_char_p, []),
    "scmx_last_error": (C.c_char_p, []),
    "scmx_init": (_I, []),
    "scmx_default_format": (None, [_FMT]),
    "scmx_mxfp4_format": (None, [_FMT]),
    "scmx_unpack_i8": (_I, [_FMT, _P, _P, _P, _L, _L, _P]),
    "scmx_act_quant": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "scmx_act_quant_blocked": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "scmx_mm_i8_i32": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "scmx_mm_epi": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_mm_w4a8": (_I, [_FMT, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_mm_w4a8_blocked": (_I, [_FMT, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_mm_w4a8_prefers_blocked": (_I, [_I, _I, _I]),
    "scmx_linear_w4a8_workspace": (_Z, [_I, _I]),
    "scmx_linear_w4a8": (_I, [_FMT, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P]),
    "scmx_linear_w4a8_static_max_elements": (_Z, []),
    "scmx_linear_w4a8_static_max_rows": (_I, []),
    "scmx_linear_w4a8_static": (_I, [_FMT, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_rmsnorm_quant": (_I, [_P, _P, _F, _P, _P, _P, _I, _I, _I, _P]),
    "scmx_rmsnorm_quant_blocked": (_I, [_P, _P, _F, _P, _P, _P, _I, _I, _I, _P]),
    "scmx_res_norm_quant": (_I, [_P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _P]),
    "scmx_swiglu_quant": (_I, [_P, _P, _P, _P, _P, _I, _I, _P]),
    "scmx_qkv_headnorm": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_attn_decode": (_I, [_P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _F, _P, _I, _P]),
    "scmx_attn_prefill": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P]),
    "scmx_attn_decode_qkv": (_I, [_P, _P, _P, _F, _P, _P, _L, _P, _P, _P, _I, _I, _I, _I, _F, _P, _I, _P]),
    "scmx_qkv_headnorm_rope": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _I, _P, _P, _L, _I, _I, _P]),
    "scmx_qkv_fullnorm": (_I, [_P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _P]),
    "scmx_gemv": (_I, [_FMT, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P, _F, _I, _I, _I, _P, _I, _I, _I, _P]),
    "scmx_route_topk": (_I, [_P, _P, _I, _I, _I, _I, _P, _P, _P]),
    "scmx_route_sort": (_I, [_P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "scmx_moe_mm": (_I, [_FMT, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P]),
    "scmx_moe_mm_i8": (_I, [_P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P]),
    "scmx_moe_combine": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _I, _P]),
    "scmx_rot_quant": (_I, [_P, _P, _P, _P, _I, _I, _I, _P]),
    "scmx_mxfp4_to_sc": (_I, [_P, _P, _P, _P, _L, _L, _P]),
    "scmx_quantize_family": (_I, [_FMT, _P, _I, _L, _I, _P, _P, _P, _P]),
    "scmx_quantize_sc": (_I, [_P, _I, _L, _I, _I, _P, _P, _P, _P]),
}

_lib = None


def load():
    """The loaded library with typed entry points; raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python {os.path.join(HERE, 'build.py')}` "
                               "(there is no CPU or PyTorch fallback for these kernels)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)       # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def call(name, *args):
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.scmx_last_error().decode()
        raise (ValueError if rc in (-1, -2, -4) else RuntimeError)(f"{name} failed ({rc}): {msg}")


def ptr(t):
    """Device pointer of a contiguous CUDA tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("scmx kernels take CUDA (ROCm) tensors; got a CPU tensor")
    if not t.is_contiguous():
        raise ValueError("scmx kernels take contiguous tensors")
    return t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream
