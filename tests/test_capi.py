"""The C-ABI library builds, loads and exports what include/cs_hip_kernels.h declares.

No kernel is launched here: the only calls made are ones the library rejects
on argument checks before it touches the HIP runtime.
"""
import ctypes
import os
import re

import pytest

from core_scheduler_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cs_hip_kernels.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cs_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for op in ("cs_adamw_step", "cs_adamw_multi_step", "cs_gelu_forward", "cs_gelu_backward",
               "cs_layernorm_forward", "cs_layernorm_backward", "cs_embedding_forward",
               "cs_embedding_forward_add", "cs_embedding_backward", "cs_embedding_backward_fused",
               "cs_fused_classifier"):
        assert op in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_capi.LIB_PATH), "run `make -C core_scheduler_amd/csrc` first"
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_binding_covers_the_header_exactly():
    assert sorted(_capi.SIGNATURES) == declared_functions()
    assert _capi.load().cs_hip_abi_version() == 1


def test_error_strings():
    lib = _capi.load()
    assert lib.cs_hip_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert len(lib.cs_hip_error_string(code)) > 4


def test_argument_checks_reject_before_launch():
    lib = _capi.load()
    p = ctypes.c_void_p(4096)  # never dereferenced: every call below fails its checks first
    h = (1e-3, 0.9, 0.999, 1e-8, 1e-2)
    assert lib.cs_adamw_step(p, p, p, p, None, -1, _capi.F32, *h, 1, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_adamw_step(p, p, p, p, None, 8, 17, *h, 1, None) == _capi.ERR_UNSUPPORTED
    assert lib.cs_adamw_step(None, p, p, p, None, 8, _capi.F32, *h, 1, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_adamw_step(ctypes.c_void_p(4097), p, p, p, None, 8, _capi.F32, *h, 1, None) == _capi.ERR_MISALIGNED
    assert lib.cs_adamw_step(p, p, p, p, None, 0, _capi.F32, *h, 1, None) == _capi.OK  # empty tensor: nothing to do
    assert lib.cs_gelu_forward(p, p, 8, _capi.BF16, 7, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_gelu_backward(None, p, p, 8, _capi.BF16, 0, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_layernorm_forward(p, p, p, p, p, p, 4, 0, 1e-5, 0, 0, 0, None) == _capi.ERR_INVALID_ARGUMENT
    # y may only be x's dtype or fp32
    assert lib.cs_layernorm_forward(p, p, p, p, p, p, 4, 8, 1e-5, _capi.F32, _capi.BF16, _capi.F32,
                                    None) == _capi.ERR_UNSUPPORTED
    assert lib.cs_layernorm_backward(p, p, p, p, p, p, p, p, None, 0, 4, 768, _capi.BF16, _capi.BF16, _capi.BF16,
                                     _capi.F32, 0, None) == _capi.ERR_WORKSPACE
    assert lib.cs_embedding_forward(p, p, p, 4, 8, 10, _capi.F32, 5, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_embedding_backward(p, p, p, None, 0, 4, 8, 10, -1, _capi.F32, _capi.I64, 0,
                                     None) == _capi.ERR_WORKSPACE
    # an empty table cannot be gathered from; a position table longer than 2^31 - 1 rows is refused
    assert lib.cs_embedding_forward(p, p, p, 4, 8, 0, _capi.F32, _capi.I64, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_embedding_forward(p, p, p, 0, 8, 0, _capi.F32, _capi.I64, None) == _capi.OK  # nothing to gather
    assert lib.cs_embedding_forward_add(p, p, p, p, 1, 1 << 31, 8, 10, _capi.F32, _capi.I64, None) == _capi.ERR_TOO_LARGE
    # the pending partial rows of cs_layernorm_backward_rows_pending may not be this call's own
    assert lib.cs_layernorm_backward_rows_pending(p, p, p, p, p, None, p, p, 1 << 20, p, 4, p, p, 0, 64, 768, _capi.BF16,
                                                  _capi.BF16, _capi.BF16, _capi.F32, None) == _capi.ERR_INVALID_ARGUMENT
    assert lib.cs_layernorm_backward_rows_pending(p, p, p, p, p, None, p, p, 1 << 20, ctypes.c_void_p(1 << 30), 100000, p, p,
                                                  0, 64, 768, _capi.BF16, _capi.BF16, _capi.BF16, _capi.F32,
                                                  None) == _capi.ERR_INVALID_ARGUMENT  # more rows than any plan leaves
    assert lib.cs_fused_classifier(p, p, p, p, p, p, p, 1 << 20, 4, 100, 50, -100, 1, 1.0, _capi.BF16, _capi.BF16,
                                   None) == _capi.ERR_INVALID_ARGUMENT  # stride < V
    assert lib.cs_fused_classifier(p, p, p, p, p, p, None, 0, 4, 100, 128, -100, 1, 1.0, _capi.BF16, _capi.BF16,
                                   None) == _capi.ERR_WORKSPACE
    assert lib.cs_fused_classifier(p, p, p, p, p, p, p, 1 << 20, 4, 100, 128, -100, 1, 1.0, _capi.F32, _capi.BF16,
                                   None) == _capi.ERR_UNSUPPORTED


def test_workspace_sizes():
    lib = _capi.load()
    assert lib.cs_fused_classifier_workspace_bytes(8192) >= 256 + 4 * 8192
    assert lib.cs_layernorm_backward_workspace_bytes(8192, 768) >= 2 * 768 * 4
    assert lib.cs_layernorm_backward_workspace_bytes(0, 768) == 0
    small = lib.cs_embedding_backward_workspace_bytes(8192, 768, 50257)
    big = lib.cs_embedding_backward_workspace_bytes(16384, 1600, 50257)
    assert 0 < small < big
    assert lib.cs_adamw_multi_table_bytes(148) >= 148 * 64 + 149 * 8


def test_multi_tensor_table_layout():
    # the table is built on the host, so its layout can be checked without a GPU
    lib = _capi.load()
    n = 3
    arr = (_capi.AdamWTensor * n)()
    sizes = [4096 * 4 + 1, 5, 8192]
    for i, s in enumerate(sizes):
        base = 0x10000 * (i + 1)
        arr[i].w, arr[i].dw, arr[i].m, arr[i].v, arr[i].v_max, arr[i].n = base, base + 0x1000, base + 0x2000, base + 0x3000, None, s
    nbytes = lib.cs_adamw_multi_table_bytes(n)
    buf = (ctypes.c_uint8 * nbytes)()
    slots = ctypes.c_int64()
    assert lib.cs_adamw_multi_build_table(arr, n, _capi.F32, buf, nbytes, ctypes.byref(slots)) == 0
    assert slots.value == 5 + 1 + 2  # one workgroup slot per 4096 fp32 elements (256 lanes x 4 vectors)
    first = (ctypes.c_int64 * 8).from_buffer(buf)
    assert list(first[:4]) == [0, 5, 6, 8]
    assert lib.cs_adamw_multi_build_table(arr, n, _capi.F32, buf, nbytes - 1, ctypes.byref(slots)) == _capi.ERR_WORKSPACE
    arr[1].w = 0x20002  # not 4-byte aligned
    assert lib.cs_adamw_multi_build_table(arr, n, _capi.F32, buf, nbytes, ctypes.byref(slots)) == _capi.ERR_MISALIGNED


def test_ops_refuse_cpu_tensors():
    import torch

    from core_scheduler_amd import ops

    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.gelu_forward(torch.zeros(8))


def test_static_scratch_entry_point_rejects_sizes_beyond_its_array():
    lib = _capi.load()
    limit = lib.cs_fused_classifier_static_max_rows()
    assert limit == ((1 << 20) - 256) // 4
    p = ctypes.c_void_p(4096)  # never dereferenced: rejected before the HIP runtime is touched
    code = lib.cs_fused_classifier_static(p, p, p, None, p, None, limit + 1, 8, 8, -100, _capi.REDUCTION_MEAN, 1.0,
                                          _capi.F32, _capi.F32, None)
    assert code == _capi.ERR_STATIC_LIMIT
