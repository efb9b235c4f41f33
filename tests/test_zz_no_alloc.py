"""cs_fused_classifier_static: the fused classifier for callers that cannot allocate.

It takes its workspace from an array the library keeps in device memory, so it must give what
cs_fused_classifier gives with a caller-owned workspace - bit for bit, the launches are the
same - on the first call on a device and on a later, smaller call that finds the previous
call's contents in the array.
"""
import ctypes

import pytest
import torch

from core_scheduler_amd import _capi
from tests._util import assert_bit_exact, randint, randn

pytestmark = pytest.mark.gpu

P = ctypes.c_void_p
DT = {torch.float32: _capi.F32, torch.bfloat16: _capi.BF16, torch.float16: _capi.F16}


def _ptr(t):
    return P(t.data_ptr()) if t is not None else None


def _run(lib, static, logits, targets, V, keep_rows, reduction, ignore_index=-100):
    """One call through the C ABI; returns (loss, total_weight, dlogits, row_loss or None)."""
    dev = logits.device
    N, stride = logits.shape
    row_loss = torch.full((N,), -7.0, dtype=torch.float32, device=dev) if keep_rows else None
    loss = torch.full((), -7.0, dtype=torch.float32, device=dev)
    tw = torch.full((), -7.0, dtype=torch.float32, device=dev)
    dlogits = torch.empty_like(logits)
    stream = P(torch.cuda.current_stream(dev).cuda_stream)
    tail = (N, V, stride, ignore_index, reduction, 1.0, DT[logits.dtype], DT[logits.dtype], stream)
    if static:
        code = lib.cs_fused_classifier_static(_ptr(logits), _ptr(dlogits), _ptr(targets), _ptr(row_loss), _ptr(loss),
                                              _ptr(tw), *tail)
        _capi.check("cs_fused_classifier_static", code)
    else:
        ws_bytes = lib.cs_fused_classifier_workspace_bytes(N)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        code = lib.cs_fused_classifier(_ptr(logits), _ptr(dlogits), _ptr(targets), _ptr(row_loss), _ptr(loss),
                                       _ptr(tw), _ptr(ws), ws_bytes, *tail)
        _capi.check("cs_fused_classifier", code)
    torch.cuda.synchronize()
    return loss, tw, dlogits, row_loss


def _same(a, b, what):
    for x, y, name in zip(a, b, ("loss", "total_weight", "dlogits", "row_loss")):
        if x is None:
            assert y is None
            continue
        assert_bit_exact(x, y, f"{what}: {name}")


def test_static_scratch_matches_workspace_call_twice_in_a_row():
    lib = _capi.load()
    dev = torch.device("cuda:0")
    # first call: the GPT-2 vocabulary, row losses kept in the library's array (row_loss NULL)
    N, V, stride = 1024, 50257, 50304
    x = randn((N, stride), 11, std=2.0, dtype=torch.bfloat16).to(dev)
    t = randint(0, V, (N,), 12)
    t[::7] = -100  # ignored rows: the count in the array's header differs from N
    t = t.to(dev)
    want = _run(lib, False, x, t, V, keep_rows=False, reduction=_capi.REDUCTION_MEAN)
    got = _run(lib, True, x, t, V, keep_rows=False, reduction=_capi.REDUCTION_MEAN)
    _same(got, want, "first call")
    assert float(got[1]) == float((t != -100).sum())

    # second call, smaller and of another type: it finds the first call's count and row losses
    # in the array and must not be affected by them
    N2, V2 = 300, 1000
    x2 = randn((N2, V2), 13, std=3.0, dtype=torch.float32).to(dev)
    t2 = randint(0, V2, (N2,), 14).to(dev)
    want2 = _run(lib, False, x2, t2, V2, keep_rows=False, reduction=_capi.REDUCTION_SUM)
    got2 = _run(lib, True, x2, t2, V2, keep_rows=False, reduction=_capi.REDUCTION_SUM)
    _same(got2, want2, "second, smaller call")
    assert float(got2[1]) == N2

    # and with the caller keeping the row losses
    want3 = _run(lib, False, x2, t2, V2, keep_rows=True, reduction=_capi.REDUCTION_MEAN)
    got3 = _run(lib, True, x2, t2, V2, keep_rows=True, reduction=_capi.REDUCTION_MEAN)
    _same(got3, want3, "third call, caller's row losses")


def test_static_scratch_rejects_more_rows_than_it_holds():
    lib = _capi.load()
    limit = lib.cs_fused_classifier_static_max_rows()
    assert limit == ((1 << 20) - 256) // 4
    p = P(4096)  # never dereferenced: the call is rejected before anything is launched
    code = lib.cs_fused_classifier_static(p, p, p, None, p, None, limit + 1, 8, 8, -100, _capi.REDUCTION_MEAN, 1.0,
                                          _capi.F32, _capi.F32, None)
    assert code == _capi.ERR_STATIC_LIMIT
    assert b"scratch" in lib.cs_hip_error_string(code)


def test_static_scratch_at_its_row_limit():
    """The largest call the array takes: its row losses end exactly at the array's last byte."""
    lib = _capi.load()
    dev = torch.device("cuda:0")
    N, V = lib.cs_fused_classifier_static_max_rows(), 8
    x = randn((N, V), 15, std=2.0, dtype=torch.float32).to(dev)
    t = randint(0, V, (N,), 16)
    t[::5] = -100
    t = t.to(dev)
    want = _run(lib, False, x, t, V, keep_rows=False, reduction=_capi.REDUCTION_MEAN)
    got = _run(lib, True, x, t, V, keep_rows=False, reduction=_capi.REDUCTION_MEAN)
    _same(got, want, "row limit")
    # and a small call right after it still finds nothing of it
    x2 = randn((64, 32), 17, dtype=torch.float32).to(dev)
    t2 = randint(0, 32, (64,), 18).to(dev)
    _same(_run(lib, True, x2, t2, 32, keep_rows=False, reduction=_capi.REDUCTION_MEAN),
          _run(lib, False, x2, t2, 32, keep_rows=False, reduction=_capi.REDUCTION_MEAN), "small call after the largest")
