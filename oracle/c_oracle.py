"""TEST INFRASTRUCTURE ONLY: ctypes front end of the C oracle.

Functions take and return CPU torch tensors.  Storage rule: float16 /
bfloat16 inputs are widened to float32, the float32 oracle runs, and the
result is rounded to the storage type once (ATen's opmath rule); float64
inputs use the float64 oracle.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libcs_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        assert _lib.oracle_abi_version() == 1
    return _lib


def _wide(t):
    """(contiguous f32/f64 copy, suffix)"""
    if t.dtype == torch.float64:
        return t.detach().contiguous().clone(), "f64"
    return t.detach().to(torch.float32).contiguous().clone(), "f32"


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _ids(ids):
    return ids.detach().to(torch.int64).contiguous()


def _call(name, sfx, *args):
    fn = getattr(lib(), f"{name}_{sfx}")
    fn.restype = None
    fn(*args)


I64, DBL, INT = ctypes.c_int64, ctypes.c_double, ctypes.c_int


def adamw_step(w, dw, m, v, *, lr, beta1, beta2, eps, weight_decay, t, v_max=None):
    """Returns updated (w, m, v, v_max) in the inputs' dtype; inputs are not modified."""
    dt = w.dtype
    ww, sfx = _wide(w)
    gw, mw, vw = _wide(dw)[0], _wide(m)[0], _wide(v)[0]
    xw = _wide(v_max)[0] if v_max is not None else None
    _call("oracle_adamw_step", sfx, _p(ww), _p(gw), _p(mw), _p(vw), _p(xw), I64(ww.numel()), DBL(lr),
          DBL(beta1), DBL(beta2), DBL(eps), DBL(weight_decay), I64(t))
    return ww.to(dt), mw.to(dt), vw.to(dt), (xw.to(dt) if xw is not None else None)


def clip_grad_norm(grads, max_norm, norm_type=2.0):
    """(scaled gradients in their dtype, total_norm, clip_coef); the inputs are not modified.
    16-bit gradients are widened, scaled in float and rounded once, as an in-place multiply does."""
    wide = [_wide(g) for g in grads]
    sfx = wide[0][1]
    bufs = [w for w, _ in wide]
    n = len(bufs)
    ptrs = (ctypes.c_void_p * n)(*[b.data_ptr() for b in bufs])
    sizes = (ctypes.c_int64 * n)(*[b.numel() for b in bufs])
    real = ctypes.c_double if sfx == "f64" else ctypes.c_float
    total, coef = real(0), real(0)
    _call("oracle_clip_grad_norm", sfx, ptrs, sizes, I64(n), INT(1 if norm_type == float("inf") else 0),
          DBL(max_norm), INT(1), ctypes.byref(total), ctypes.byref(coef))
    return [b.to(g.dtype).reshape(g.shape) for b, g in zip(bufs, grads)], total.value, coef.value


def gelu_forward(x, approximate="none"):
    xw, sfx = _wide(x)
    y = torch.empty_like(xw)
    _call("oracle_gelu_forward", sfx, _p(xw), _p(y), I64(xw.numel()), INT(0 if approximate == "none" else 1))
    return y.to(x.dtype)


def gelu_backward(dy, x, approximate="none"):
    xw, sfx = _wide(x)
    dw = _wide(dy)[0].to(xw.dtype)
    dx = torch.empty_like(xw)
    _call("oracle_gelu_backward", sfx, _p(dw), _p(xw), _p(dx), I64(xw.numel()),
          INT(0 if approximate == "none" else 1))
    return dx.to(x.dtype)


def layernorm_forward(x, gamma, beta=None, eps=1e-5, out_dtype=None):
    """(y, mean, rstd); statistics stay wide (f32, or f64 for f64 x)."""
    xw, sfx = _wide(x)
    C = x.shape[-1]
    rows = x.numel() // C
    gw = gamma.detach().to(xw.dtype).contiguous()
    bw = beta.detach().to(xw.dtype).contiguous() if beta is not None else None
    y = torch.empty_like(xw)
    mean = torch.empty(rows, dtype=xw.dtype)
    rstd = torch.empty(rows, dtype=xw.dtype)
    _call("oracle_layernorm_forward", sfx, _p(xw), _p(gw), _p(bw), _p(y), _p(mean), _p(rstd), I64(rows),
          I64(C), DBL(eps))
    return y.to(out_dtype or x.dtype), mean, rstd


def layernorm_backward(dy, x, mean, rstd, gamma, dgamma=None, dbeta=None, out_dtype=None):
    """(dx, dgamma, dbeta); dgamma/dbeta given are accumulated into (copies)."""
    xw, sfx = _wide(x)
    C = x.shape[-1]
    rows = x.numel() // C
    dw = dy.detach().to(xw.dtype).contiguous()
    gw = gamma.detach().to(xw.dtype).contiguous()
    mw, rw = mean.detach().to(xw.dtype).contiguous(), rstd.detach().to(xw.dtype).contiguous()
    dx = torch.empty_like(xw)
    acc = dgamma is not None
    dg = dgamma.detach().to(xw.dtype).contiguous().clone() if acc else torch.empty(C, dtype=xw.dtype)
    db = dbeta.detach().to(xw.dtype).contiguous().clone() if dbeta is not None else torch.zeros(C, dtype=xw.dtype)
    _call("oracle_layernorm_backward", sfx, _p(dw), _p(xw), _p(mw), _p(rw), _p(gw), _p(dx), _p(dg), _p(db),
          I64(rows), I64(C), INT(int(acc)))
    return dx.to(out_dtype or x.dtype), dg.to(gamma.dtype), db.to(gamma.dtype)


def embedding_forward(weight, ids):
    ww, sfx = _wide(weight)
    V, C = weight.shape
    idx = _ids(ids)
    out = torch.empty(idx.numel(), C, dtype=ww.dtype)
    _call("oracle_embedding_forward", sfx, _p(ww), _p(idx), _p(out), I64(idx.numel()), I64(C), I64(V))
    return out.to(weight.dtype).reshape(*ids.shape, C)


def embedding_forward_add(wte, wpe, ids):
    ww, sfx = _wide(wte)
    pw = _wide(wpe)[0]
    V, C = wte.shape
    B, T = ids.shape
    idx = _ids(ids)
    out = torch.empty(B, T, C, dtype=ww.dtype)
    _call("oracle_embedding_forward_add", sfx, _p(ww), _p(pw), _p(idx), _p(out), I64(B), I64(T), I64(C), I64(V))
    return out.to(wte.dtype)


def embedding_backward(dout, ids, num_weights, padding_idx=-1, dweight=None, scale_grad_by_freq=False):
    dw, sfx = _wide(dout)
    C = dout.shape[-1]
    idx = _ids(ids)
    acc = dweight is not None
    g = _wide(dweight)[0] if acc else torch.empty(num_weights, C, dtype=dw.dtype)
    _call("oracle_embedding_backward", sfx, _p(dw), _p(idx), _p(g), I64(idx.numel()), I64(C), I64(num_weights),
          I64(padding_idx), INT(int(acc)), INT(int(scale_grad_by_freq)))
    return g.to(dout.dtype)


def embedding_backward_positions(dout, dwpe=None):
    dw, sfx = _wide(dout)
    B, T, C = dout.shape
    acc = dwpe is not None
    g = _wide(dwpe)[0] if acc else torch.empty(T, C, dtype=dw.dtype)
    _call("oracle_embedding_backward_positions", sfx, _p(dw), _p(g), I64(B), I64(T), I64(C), INT(int(acc)))
    return g.to(dout.dtype)


def cross_entropy(logits, targets, num_classes=None, *, ignore_index=-100, reduction="mean", dloss=1.0,
                  dlogits_dtype=None, class_weight=None):
    """(loss, row_loss, dlogits, total_weight); loss/row_loss stay wide, dlogits is rounded once."""
    xw, sfx = _wide(logits)
    N, stride = logits.shape
    V = stride if num_classes is None else num_classes
    t = _ids(targets)
    row = torch.empty(N, dtype=xw.dtype)
    loss = torch.zeros((), dtype=xw.dtype)
    tw = torch.zeros((), dtype=xw.dtype)
    d = torch.empty_like(xw)
    red = {"none": 0, "mean": 1, "sum": 2}[reduction]
    cw = None if class_weight is None else class_weight.to(xw.dtype).contiguous()
    _call("oracle_cross_entropy", sfx, _p(xw), _p(t), _p(row), _p(loss), _p(tw), _p(d), I64(N), I64(V),
          I64(stride), I64(ignore_index), INT(red), DBL(dloss), _p(cw) if cw is not None else None)
    return (row if reduction == "none" else loss), row, d.to(dlogits_dtype or logits.dtype), tw
