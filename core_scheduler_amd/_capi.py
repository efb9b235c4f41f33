"""ctypes binding of the C ABI declared in include/cs_hip_kernels.h.

Loads core_scheduler_amd/lib/libcs_hip_kernels.so, which
core_scheduler_amd/csrc/Makefile builds.  There is no fallback: if the
library is missing, loading raises, and every op in this package goes through
it.
"""
import ctypes
import os
from ctypes import c_double, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcs_hip_kernels.so")

# enum cs_dtype / cs_itype / cs_reduction / cs_gelu_mode
F32, F64, F16, BF16 = 0, 1, 2, 3
I32, I64 = 0, 1
REDUCTION_NONE, REDUCTION_MEAN, REDUCTION_SUM = 0, 1, 2
GELU_ERF, GELU_TANH = 0, 1

OK = 0
ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_MISALIGNED, ERR_WORKSPACE, ERR_TOO_LARGE = -1, -2, -3, -4, -5
ERR_STATIC_LIMIT = -6


class AdamWTensor(ctypes.Structure):
    """struct cs_adamw_tensor"""

    _fields_ = [
        ("w", c_void_p),
        ("dw", c_void_p),
        ("m", c_void_p),
        ("v", c_void_p),
        ("v_max", c_void_p),
        ("n", c_int64),
    ]


# name -> (restype, argtypes); one entry per declaration in the header
SIGNATURES = {
    "cs_hip_abi_version": (c_int, []),
    "cs_hip_error_string": (ctypes.c_char_p, [c_int]),
    "cs_stream_copy": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "cs_stream_read_out_words": (c_int64, [c_int64]),
    "cs_stream_read": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "cs_stream_fill": (c_int, [c_void_p, c_int64, ctypes.c_uint32, c_void_p]),
    "cs_stream_fill_shape": (c_int, [c_void_p, c_int64, ctypes.c_uint32] + [c_int] * 5 + [c_void_p]),
    "cs_stream_update4": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "cs_adamw_step": (c_int, [c_void_p] * 5 + [c_int64, c_int] + [c_double] * 5 + [c_int64, c_void_p]),
    "cs_adamw_multi_table_bytes": (c_size_t, [c_int64]),
    "cs_adamw_multi_build_table": (
        c_int,
        [ctypes.POINTER(AdamWTensor), c_int64, c_int, c_void_p, c_size_t, ctypes.POINTER(c_int64)],
    ),
    "cs_adamw_multi_step": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_int] + [c_double] * 5 + [c_int64, c_void_p],
    ),
    "cs_grad_norm_multi_workspace_bytes": (c_size_t, [c_int64]),
    "cs_grad_norm_multi": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_double, c_double, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p],
    ),
    "cs_grad_scale_multi": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p]),
    "cs_adamw_multi_step_clipped": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_int] + [c_double] * 5 + [c_int64, c_void_p, c_void_p],
    ),
    "cs_gelu_forward": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "cs_gelu_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "cs_layernorm_forward": (
        c_int,
        [c_void_p] * 6 + [c_int64, c_int64, c_double, c_int, c_int, c_int, c_void_p],
    ),
    "cs_add_layernorm_forward": (
        c_int,
        [c_void_p] * 8 + [c_int64, c_int64, c_double, c_int, c_int, c_int, c_void_p],
    ),
    "cs_layernorm_backward_add": (
        c_int,
        [c_void_p] * 10 + [c_size_t, c_int64, c_int64] + [c_int] * 5 + [c_void_p],
    ),
    "cs_layernorm_backward_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "cs_layernorm_backward_partial_rows": (c_int64, [c_int64, c_int64, c_int]),
    "cs_layernorm_backward_rows": (
        c_int,
        [c_void_p] * 8 + [c_size_t, c_int64, c_int64] + [c_int] * 4 + [c_void_p],
    ),
    "cs_layernorm_backward_finalize": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p],
    ),
    "cs_layernorm_backward_rows_pending": (
        c_int,
        [c_void_p] * 8 + [c_size_t, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int64] + [c_int] * 4
        + [c_void_p],
    ),
    "cs_layernorm_backward": (
        c_int,
        [c_void_p] * 9 + [c_size_t, c_int64, c_int64] + [c_int] * 5 + [c_void_p],
    ),
    "cs_embedding_forward": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
    ),
    "cs_embedding_forward_add": (
        c_int,
        [c_void_p] * 4 + [c_int64] * 4 + [c_int, c_int, c_void_p],
    ),
    "cs_embedding_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "cs_embedding_backward": (
        c_int,
        [c_void_p] * 4 + [c_size_t] + [c_int64] * 4 + [c_int, c_int, c_int, c_void_p],
    ),
    "cs_embedding_backward_scaled": (
        c_int,
        [c_void_p] * 4 + [c_size_t] + [c_int64] * 4 + [c_int, c_int, c_int, c_void_p],
    ),
    "cs_embedding_backward_fused": (
        c_int,
        [c_void_p] * 5 + [c_size_t] + [c_int64] * 4 + [c_int, c_int, c_int, c_void_p],
    ),
    "cs_embedding_backward_positions": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
    ),
    "cs_fused_classifier_workspace_bytes": (c_size_t, [c_int64]),
    "cs_fused_classifier": (
        c_int,
        [c_void_p] * 7 + [c_size_t] + [c_int64] * 4 + [c_int, c_float, c_int, c_int, c_void_p],
    ),
    "cs_fused_classifier_weighted": (
        c_int,
        [c_void_p] * 8 + [c_size_t] + [c_int64] * 4 + [c_int, c_float, c_int, c_int, c_void_p],
    ),
    "cs_fused_classifier_static_max_rows": (c_int64, []),
    "cs_fused_classifier_static": (
        c_int,
        [c_void_p] * 6 + [c_int64] * 4 + [c_int, c_float, c_int, c_int, c_void_p],
    ),
    "cs_fused_classifier_phases": (
        c_int,
        [c_void_p] * 7 + [c_size_t] + [c_int64] * 4 + [c_int, c_float, c_int, c_int, c_int, c_void_p],
    ),
}

_lib = None


class KernelLibraryMissing(RuntimeError):
    pass


class KernelError(RuntimeError):
    def __init__(self, fn, code, text):
        super().__init__(f"{fn} failed: {code} ({text})")
        self.code = code


def load():
    """Returns the loaded library with argtypes set; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KernelLibraryMissing(
            f"{LIB_PATH} is not built. Run `make -C core_scheduler_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "There is no CPU fallback for these ops."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.cs_hip_abi_version() != 1:
        raise KernelLibraryMissing(f"{LIB_PATH}: ABI version {lib.cs_hip_abi_version()}, expected 1")
    _lib = lib
    return lib


def check(fn_name, code):
    """Raises KernelError for a non-zero return of a C-ABI call."""
    if code != OK:
        text = load().cs_hip_error_string(code)
        raise KernelError(fn_name, code, text.decode() if text else "?")
