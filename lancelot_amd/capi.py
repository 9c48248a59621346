"""ctypes view of libcahel_hip.so (the C-ABI declared in include/cahel_hip.h).

For callers that own their device buffers (torch tensors, the benchmark, the parity tests): every
function takes raw device pointers as integers.  `check(rc)` turns a non-zero status into RuntimeError.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libcahel_hip.so")

u64 = C.c_uint64
u32 = C.c_uint32
vp = C.c_void_p

# name -> (restype, argtypes); one entry per declaration in include/cahel_hip.h
SIGNATURES = {
    "he_error_string": (C.c_char_p, [C.c_int]),
    "he_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "he_malloc": (C.c_int, [C.POINTER(vp), C.c_size_t]),
    "he_free": (C.c_int, [vp]),
    "he_memcpy_h2d": (C.c_int, [vp, vp, C.c_size_t, vp]),
    "he_host_malloc": (C.c_int, [C.POINTER(vp), C.c_size_t]),
    "he_host_free": (C.c_int, [vp]),
    "he_memcpy_h2d_async": (C.c_int, [vp, vp, C.c_size_t, vp]),
    "he_memcpy_d2h": (C.c_int, [vp, vp, C.c_size_t, vp]),
    "he_memcpy_d2d": (C.c_int, [vp, vp, C.c_size_t, vp]),
    "he_memcpy2d_d2d": (C.c_int, [vp, C.c_size_t, vp, C.c_size_t, C.c_size_t, C.c_size_t, vp]),
    "he_memset_zero": (C.c_int, [vp, C.c_size_t, vp]),
    "he_stream_create": (C.c_int, [C.POINTER(vp)]),
    "he_stream_destroy": (C.c_int, [vp]),
    "he_stream_synchronize": (C.c_int, [vp]),
    "he_event_create": (C.c_int, [C.POINTER(vp)]),
    "he_event_destroy": (C.c_int, [vp]),
    "he_event_record": (C.c_int, [vp, vp]),
    "he_event_synchronize": (C.c_int, [vp]),
    "he_stream_wait_event": (C.c_int, [vp, vp]),
    "he_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "he_context_create": (C.c_int, [vp, C.POINTER(vp)]),
    "he_context_set_level": (C.c_int, [vp, vp]),
    "he_context_destroy": (C.c_int, [vp]),
    "he_ntt_forward": (C.c_int, [vp, vp, u32, u32, u32, u32, u32, u32, vp]),
    "he_ntt_inverse": (C.c_int, [vp, vp, u32, u32, u32, u32, u32, u32, vp]),
    "he_add": (C.c_int, [vp, vp, vp, vp, u32, u32, u32, vp]),
    "he_sub": (C.c_int, [vp, vp, vp, vp, u32, u32, u32, vp]),
    "he_negate": (C.c_int, [vp, vp, vp, u32, u32, u32, vp]),
    "he_multiply": (C.c_int, [vp, vp, vp, vp, u32, u32, u32, vp]),
    "he_multiply_add": (C.c_int, [vp, vp, vp, vp, vp, u32, u32, u32, C.c_int, vp]),
    "he_add_p_multiple": (C.c_int, [vp, vp, vp, vp, u32, u32, vp]),
    "he_tensor": (C.c_int, [vp, vp, vp, vp, u32, vp]),
    "he_tensor_square": (C.c_int, [vp, vp, vp, u32, vp]),
    "he_tensor_mxn": (C.c_int, [vp, vp, u32, vp, u32, vp, u32, vp]),
    "he_galois_ntt": (C.c_int, [vp, vp, vp, u32, u32, vp]),
    "he_rescale": (C.c_int, [vp, vp, vp, u32, u32, vp, vp]),
    "he_rescale_static": (C.c_int, [vp, vp, vp, u32, u32, vp]),
    "he_modup": (C.c_int, [vp, u32, vp, vp, vp, vp]),
    "he_ks_inner_product": (C.c_int, [vp, u32, vp, C.POINTER(vp), vp, u32, C.c_int, vp]),
    "he_moddown": (C.c_int, [vp, u32, vp, vp, u32, C.c_int, vp, vp]),
    "he_keyswitch_workspace_words": (C.c_size_t, [vp, u32]),
    "he_keyswitch": (C.c_int, [vp, u32, vp, C.POINTER(vp), vp, u32, vp, vp]),
    "he_rotate": (C.c_int, [vp, u32, vp, C.POINTER(vp), vp, u32, vp, vp]),
    "he_hoisted_rotations": (C.c_int, [vp, u32, vp, C.POINTER(vp), C.POINTER(u32), u32, vp, vp, vp]),
    "he_keyswitch_batch_workspace_words": (C.c_size_t, [vp, u32, u32]),
    "he_hoisted_rotations_batch": (C.c_int, [vp, u32, u32, vp, C.POINTER(vp), C.POINTER(u32), u32, C.c_int, vp, vp, vp]),
    "he_keyswitch_rescale_batch": (C.c_int, [vp, u32, u32, vp, u32, C.POINTER(vp), vp, vp, u32, vp, vp]),
    "he_pair_square_sum": (C.c_int, [vp, u32, u32, u32, vp, vp, vp, vp]),
    "he_keyswitch_rescale": (C.c_int, [vp, u32, vp, C.POINTER(vp), vp, vp, u32, vp, vp]),
    "he_multiply_relin_rescale_workspace_words": (C.c_size_t, [vp, u32]),
    "he_multiply_relin_rescale": (C.c_int, [vp, u32, vp, vp, C.POINTER(vp), vp, vp, vp]),
    "he_multiply_relin_rescale_batch_workspace_words": (C.c_size_t, [vp, u32, u32]),
    "he_multiply_relin_rescale_batch": (C.c_int, [vp, u32, u32, vp, vp, C.POINTER(vp), vp, vp, vp]),
    "he_decompose_real": (C.c_int, [vp, vp, vp, u32, u32, vp]),
    "he_ckks_encode": (C.c_int, [vp, vp, vp, u32, u32, C.c_double, u32, vp, vp, vp]),
    "he_ckks_decode": (C.c_int, [vp, vp, u32, u32, C.c_double, vp, vp, vp]),
    "he_ckks_workspace_words": (C.c_size_t, [vp, u32]),
    "he_sample": (C.c_int, [vp, C.c_int, C.POINTER(u32), u64, vp, u32, u32, u32, u32, vp, u32, vp]),
    "he_ckks_encode_batch_workspace_words": (C.c_size_t, [vp, u32]),
    "he_ckks_encode_batch": (C.c_int, [vp, vp, vp, u32, u32, C.c_double, u32, u32, C.c_size_t, vp, u32, vp, vp]),
    "he_encrypt_batch_workspace_words": (C.c_size_t, [vp, u32, u32]),
    "he_encrypt_batch": (C.c_int, [vp, u32, u32, vp, C.POINTER(u32), u64, vp, vp, vp]),
    "he_sample_batch": (C.c_int, [vp, C.c_int, C.POINTER(u32), u64, vp, u32, u32, u32, u32, vp, u32, u32, vp]),
    "he_decrypt_decode_batch_workspace_words": (C.c_size_t, [vp, u32, u32, u32]),
    "he_decrypt_decode_batch": (C.c_int, [vp, vp, u32, u32, vp, vp, u32, C.c_double, u32, vp, vp, vp]),
}

# the measurement library beside it (include/cahel_probe.h)
PROBE_LIB_PATH = os.path.join(_PKG, "libcahel_probe.so")
PROBE_SIGNATURES = {
    "he_probe_fp64_issue_rate": (C.c_int, [u32, u32, C.POINTER(C.c_double), vp]),
    "he_probe_issue_rate": (C.c_int, [u32, u32, u32, C.POINTER(C.c_double), vp]),
}

_lib = None
_probe_lib = None


def lib():
    """Loads libcahel_hip.so; raises if it has not been built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libcahel_hip.so is missing: run `python -m lancelot_amd.build`")
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _lib


def probe_lib():
    """Loads libcahel_probe.so (issue-rate micro-benchmarks for bench.py); raises if it has not been built."""
    global _probe_lib
    if _probe_lib is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError("libcahel_probe.so is missing: run `python -m lancelot_amd.build`")
        _probe_lib = C.CDLL(PROBE_LIB_PATH)
        for name, (res, args) in PROBE_SIGNATURES.items():
            fn = getattr(_probe_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _probe_lib


def check(rc: int, what: str = "libcahel_hip"):
    if rc != 0:
        raise RuntimeError("%s failed: %s" % (what, lib().he_error_string(rc).decode()))


def evk_array(ptrs):
    """Host array of device pointers for he_ks_inner_product / he_keyswitch."""
    return (vp * len(ptrs))(*ptrs)
