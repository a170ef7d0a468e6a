"""ctypes binding of the C ABI declared in include/hyc_abi.h.

The library is built in-tree by build.py (hipcc, gfx950).  There is no CPU fallback: if the shared
library is missing, loading fails with an error that says how to build it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libhyc_gfx950.so")

MODE_CHANNEL, MODE_THRESHOLD, MODE_DENSE = 0, 1, 2
DTYPE_BF16, DTYPE_F32 = 0, 1
ACT_SILU, ACT_GELU_TANH = 0, 1
SCALE_RANGE, SCALE_ABSMAX = 0, 1
ABI_VERSION = 3
RMSNORM_BWD_STATIC_MAX_FLOATS = 4 * 1024 * 1024
EINVAL, EFAULT, ENOTSUP, ELAUNCH = -22, -14, -95, -5

c_i32, c_i64, c_f32, c_ptr = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class HycDesc(ctypes.Structure):
    """struct hyc_desc"""
    _fields_ = [
        ("mode", c_i32), ("bits", c_i32), ("group", c_i32), ("k", c_i32),
        ("chan_plan", c_ptr),
        ("threshold", c_f32),
        ("scale", c_ptr),
        ("scale_stride_token", c_i64), ("scale_stride_channel", c_i64), ("S", c_i64),
        ("L", c_ptr), ("R", c_ptr),
        ("rank", c_i32), ("scale_rule", c_i32),
        ("csr_row_ptr", c_ptr), ("csr_cols", c_ptr), ("csr_vals", c_ptr),
        ("chan_idx", c_ptr),
    ]


# name -> (restype, argtypes); one line per declaration in include/hyc_abi.h
SIGNATURES = {
    "hyc_abi_version": (c_i32, []),
    "hyc_last_error": (ctypes.c_char_p, []),
    "hyc_check_shape": (c_i32, [c_i64, c_i32, c_i32, c_i32]),
    "hyc_stored_row_bytes": (c_i64, [c_i64, c_i32]),
    "hyc_rmsnorm_bwd_partials": (c_i64, [c_i64, c_i64]),
    "hyc_rmsnorm_bwd_partial_rows": (c_i64, [c_i64, c_i64, ctypes.POINTER(HycDesc)]),
    "hyc_channel_absmax": (c_i32, [c_ptr, c_i64, c_i64, c_ptr, c_ptr]),
    "hyc_select_channels": (c_i32, [c_ptr, c_i64, c_i32, c_ptr, c_ptr, c_ptr]),
    "hyc_compress": (c_i32, [c_ptr, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_compress_rows": (c_i32, [c_ptr, c_i64, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_decompress": (c_i32, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr]),
    "hyc_ref_outlier_count": (c_i32, [c_ptr, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr]),
    "hyc_ref_outlier_fill": (c_i32, [c_ptr, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_rmsnorm_fwd_compress": (c_i32, [c_ptr, c_ptr, c_i32, c_f32, c_i64, c_i64, ctypes.POINTER(HycDesc),
                                         c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_layernorm_fwd_compress": (c_i32, [c_ptr, c_ptr, c_ptr, c_i32, c_f32, c_i64, c_i64, ctypes.POINTER(HycDesc),
                                           c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_rmsnorm_bwd": (c_i32, [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i32, c_ptr, c_i64, c_i64,
                                ctypes.POINTER(HycDesc), c_i32, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_rmsnorm_bwd_static": (c_i32, [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i32, c_ptr, c_i64, c_i64,
                                       ctypes.POINTER(HycDesc), c_i32, c_ptr, c_ptr, c_ptr]),
    "hyc_layernorm_bwd": (c_i32, [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i32, c_ptr, c_ptr, c_i64, c_i64,
                                  ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_act_bwd": (c_i32, [c_i32, c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr]),
    "hyc_hadamard_bwd": (c_i32, [c_ptr, c_ptr, c_ptr, c_ptr, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr,
                                 ctypes.POINTER(HycDesc), c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_gated_act_bwd": (c_i32, [c_i32, c_ptr, c_ptr, c_ptr, c_ptr, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, ctypes.POINTER(HycDesc),
                                  c_ptr, c_ptr, c_ptr, ctypes.POINTER(HycDesc), c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_gated_act_fwd": (c_i32, [c_i32, c_ptr, c_i64, c_ptr, c_i64, c_i64, c_i64, ctypes.POINTER(HycDesc), ctypes.POINTER(HycDesc),
                                  ctypes.POINTER(HycDesc), c_ptr] + [c_ptr] * 9 + [c_ptr]),
    "hyc_act_fwd_compress": (c_i32, [c_i32, c_ptr, c_i64, c_i64, c_i64, ctypes.POINTER(HycDesc), c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_hadamard_fwd_compress": (c_i32, [c_ptr, c_i64, c_ptr, c_i64, c_i64, c_i64, ctypes.POINTER(HycDesc), ctypes.POINTER(HycDesc),
                                          c_ptr] + [c_ptr] * 6 + [c_ptr]),
    "hyc_softmax_fwd": (c_i32, [c_ptr, c_i64, c_i64, c_f32, c_ptr, c_ptr, c_ptr]),
    "hyc_softmax_causal_fwd": (c_i32, [c_ptr, c_i64, c_i64, c_i64, c_f32, c_ptr, c_ptr, c_ptr]),
    "hyc_csr_offsets": (c_i32, [c_ptr, c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_softmax_fill": (c_i32, [c_ptr, c_i64, c_i64, c_f32, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_softmax_bwd": (c_i32, [c_ptr, c_i64, c_i64, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_softmax_dense": (c_i32, [c_i64, c_i64, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "hyc_gradw_workspace_bytes": (c_i64, [c_i64, c_i64, c_i64]),
    "hyc_gradw_gemm": (c_i32, [c_ptr, c_i64, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, ctypes.POINTER(HycDesc),
                               c_f32, c_f32, c_ptr, c_i32, c_ptr, c_ptr]),
    "hyc_low_rank_update": (c_i32, [c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i32, c_i32, c_ptr]),
    "hyc_kth_value_workspace_bytes": (c_i64, []),
    "hyc_kth_value": (c_i32, [c_ptr, c_i32, c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_rope_to_heads": (c_i32, [c_ptr, c_i64, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_rope_from_heads": (c_i32, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_ptr]),
    "hyc_dropout": (c_i32, [c_ptr, c_ptr, c_i64, c_f32, ctypes.c_uint64, c_i32, c_ptr]),
    "hyc_nf4_quantize": (c_i32, [c_ptr, c_i64, c_ptr, c_ptr, c_ptr]),
    "hyc_nf4_dequantize": (c_i32, [c_ptr, c_ptr, c_i64, c_ptr, c_ptr]),
}

_lib = None


def load():
    """dlopen the library once and attach the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    # torch first: it ships its own HIP runtime (same soname as the system one); the library must bind to the
    # runtime instance that owns the caller's streams and allocations, so torch's has to be resident already.
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "HIP library %s is missing: build it with `python hyc-lora_amd/build.py` "
            "(there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)           # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if lib.hyc_abi_version() != ABI_VERSION:
        raise RuntimeError("libhyc ABI version %d, expected %d: rebuild it with `python hyc-lora_amd/build.py`"
                           % (lib.hyc_abi_version(), ABI_VERSION))
    _lib = lib
    return lib


class HycError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("hyc error %d: %s" % (code, msg))
        self.code = code


def check(rc):
    """raise the Python exception that corresponds to a negative return code"""
    if rc == 0:
        return
    msg = load().hyc_last_error().decode("utf-8", "replace")
    if rc == ENOTSUP:
        raise NotImplementedError("hyc: " + msg)
    if rc in (EINVAL, EFAULT):
        raise ValueError("hyc: " + msg)
    raise HycError(rc, msg)
