"""The GPT-2 training ops on torch tensors, through the C ABI.

torch supplies device memory and the current stream; every computation is a
call into libcs_hip_kernels.so.  Tensors must live on a ROCm device and be
contiguous; there is no CPU path.
"""
import ctypes

import torch

from . import _capi

_DTYPES = {
    torch.float32: _capi.F32,
    torch.float64: _capi.F64,
    torch.float16: _capi.F16,
    torch.bfloat16: _capi.BF16,
}
_ITYPES = {torch.int32: _capi.I32, torch.int64: _capi.I64}
_REDUCTIONS = {"none": _capi.REDUCTION_NONE, "mean": _capi.REDUCTION_MEAN, "sum": _capi.REDUCTION_SUM}
_GELU = {"none": _capi.GELU_ERF, "tanh": _capi.GELU_TANH}


def _dt(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}") from None


def _dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("core_scheduler_amd ops need tensors on a ROCm device; there is no CPU path")
        if not t.is_contiguous():
            raise RuntimeError("core_scheduler_amd ops need contiguous tensors")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("tensors on different devices")
    return dev


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _workspace(nbytes, dev):
    # torch's allocator hands out 512-byte aligned blocks
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)


# ------------------------------------------------------------------ AdamW
def _check_adamw_tensors(w, dw, m, v, v_max=None):
    """The kernels take one element type and one count for the parameter, its gradient and its
    state; a mismatch would read or write past the end of the smaller tensor."""
    for name, t in (("gradient", dw), ("m", m), ("v", v), ("v_max", v_max)):
        if t is None:
            continue
        if t.dtype != w.dtype or t.numel() != w.numel():
            raise ValueError(f"AdamW: {name} is {t.dtype} x {t.numel()}, the parameter {w.dtype} x {w.numel()}")
        if not t.is_contiguous():
            raise ValueError(f"AdamW: {name} must be contiguous")
    if not w.is_contiguous():
        raise ValueError("AdamW: the parameter must be contiguous")


def adamw_step(w, dw, m, v, *, lr, beta1, beta2, eps, weight_decay, t, v_max=None):
    """One AdamW step on one tensor, in place (cs::optimizer::AdamW::step).  `t` >= 1."""
    _check_adamw_tensors(w, dw, m, v, v_max)
    dev = _dev(w, dw, m, v, v_max)
    lib = _capi.load()
    with torch.cuda.device(dev):
        code = lib.cs_adamw_step(_ptr(w), _ptr(dw), _ptr(m), _ptr(v), _ptr(v_max), w.numel(), _dt(w),
                                 lr, beta1, beta2, eps, weight_decay, t, _stream(dev))
    _capi.check("cs_adamw_step", code)


class MultiTensorAdamW:
    """All parameters of a model in one launch per step.

    The descriptor table is laid out by the library in pinned host memory and
    copied to the device on the op's stream whenever `refresh` is called (at
    construction, and again if gradients were re-allocated).
    """

    def __init__(self, params, grads, *, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
                 weight_decay=1e-2, amsgrad=False, t=0):
        self.params = list(params)
        self.lr, self.beta1, self.beta2, self.eps, self.weight_decay = lr, beta1, beta2, eps, weight_decay
        self.amsgrad, self.t = amsgrad, t
        self.dtype = self.params[0].dtype
        for p in self.params:
            if p.dtype != self.dtype or not p.is_contiguous():
                raise ValueError("MultiTensorAdamW needs contiguous parameters of one dtype")
        self.dev = _dev(*self.params)
        self.m = [torch.zeros_like(p) for p in self.params]
        self.v = [torch.zeros_like(p) for p in self.params]
        self.v_max = [torch.zeros_like(p) for p in self.params] if amsgrad else None
        lib = _capi.load()
        self._bytes = lib.cs_adamw_multi_table_bytes(len(self.params))
        self._table = torch.empty(self._bytes, dtype=torch.uint8, device=self.dev)
        self._slots = 0
        self.refresh(grads)

    def refresh(self, grads):
        grads = list(grads)
        n = len(self.params)
        if len(grads) != n:
            raise ValueError("one gradient per parameter")
        for p, g in zip(self.params, grads):
            if g.numel() != p.numel() or g.dtype != p.dtype or not g.is_contiguous():
                raise ValueError("gradient does not match its parameter")
        _dev(*grads)
        lib = _capi.load()
        arr = (_capi.AdamWTensor * n)()
        for i, (p, g) in enumerate(zip(self.params, grads)):
            arr[i].w, arr[i].dw = p.data_ptr(), g.data_ptr()
            arr[i].m, arr[i].v = self.m[i].data_ptr(), self.v[i].data_ptr()
            arr[i].v_max = self.v_max[i].data_ptr() if self.amsgrad else None
            arr[i].n = p.numel()
        slots = ctypes.c_int64(0)
        # A new pinned block for every refresh: the copy below reads it when the stream gets
        # there, not now, and the host may be a step ahead of the device; rewriting one shared
        # block would hand the step still queued the next step's gradient addresses.  The block
        # goes back to torch's pinned allocator, which reuses it only after the copy has run.
        host = torch.empty(self._bytes, dtype=torch.uint8, pin_memory=True)
        code = lib.cs_adamw_multi_build_table(arr, n, _DTYPES[self.dtype], ctypes.c_void_p(host.data_ptr()),
                                              self._bytes, ctypes.byref(slots))
        _capi.check("cs_adamw_multi_build_table", code)
        self._slots = slots.value
        self._grads = grads  # keep them alive: the table holds their addresses
        with torch.cuda.device(self.dev):
            self._table.copy_(host, non_blocking=True)

    def step(self, max_grad_norm=None, norm_type=2.0):
        """One launch for every parameter.  With `max_grad_norm`, the global gradient norm is
        taken first (two small launches) and the step applies the clipping coefficient to the
        gradients as it reads them; returns the norm as a 0-d device tensor then."""
        self.t += 1
        lib = _capi.load()
        n = len(self.params)
        with torch.cuda.device(self.dev):
            if max_grad_norm is None:
                code = lib.cs_adamw_multi_step(_ptr(self._table), n, self._slots, _DTYPES[self.dtype],
                                               int(self.amsgrad), self.lr, self.beta1, self.beta2, self.eps,
                                               self.weight_decay, self.t, _stream(self.dev))
                _capi.check("cs_adamw_multi_step", code)
                return None
            norm = self.grad_norm(max_grad_norm, norm_type)
            code = lib.cs_adamw_multi_step_clipped(_ptr(self._table), n, self._slots, _DTYPES[self.dtype],
                                                   int(self.amsgrad), self.lr, self.beta1, self.beta2, self.eps,
                                                   self.weight_decay, self.t, _ptr(self._clip), _stream(self.dev))
            _capi.check("cs_adamw_multi_step_clipped", code)
            return norm

    def grad_norm(self, max_norm, norm_type=2.0):
        """Global norm of all gradients; leaves the clipping coefficient in `self._clip`."""
        lib = _capi.load()
        nbytes = lib.cs_grad_norm_multi_workspace_bytes(self._slots)
        if getattr(self, "_norm_ws", None) is None or self._norm_ws.numel() < nbytes:
            self._norm_ws = torch.empty(nbytes, dtype=torch.uint8, device=self.dev)
            self._clip = torch.empty((), dtype=torch.float32, device=self.dev)
        norm = torch.empty((), dtype=torch.float32, device=self.dev)
        with torch.cuda.device(self.dev):
            code = lib.cs_grad_norm_multi(_ptr(self._table), len(self.params), self._slots, _DTYPES[self.dtype],
                                          float(norm_type), float(max_norm), _ptr(self._norm_ws), nbytes,
                                          _ptr(norm), _ptr(self._clip), _stream(self.dev))
        _capi.check("cs_grad_norm_multi", code)
        return norm

    def clip_grad_norm_(self, max_norm, norm_type=2.0):
        """The reference's Utils::clip_grad_norm_: scales the gradients in place, returns the norm."""
        norm = self.grad_norm(max_norm, norm_type)
        with torch.cuda.device(self.dev):
            code = _capi.load().cs_grad_scale_multi(_ptr(self._table), len(self.params), self._slots,
                                                    _DTYPES[self.dtype], _ptr(self._clip), _stream(self.dev))
        _capi.check("cs_grad_scale_multi", code)
        return norm


# ------------------------------------------------------------------- GeLU
def gelu_forward(x, approximate="none"):
    dev = _dev(x)
    y = torch.empty_like(x)
    with torch.cuda.device(dev):
        code = _capi.load().cs_gelu_forward(_ptr(x), _ptr(y), x.numel(), _dt(x), _GELU[approximate],
                                            _stream(dev))
    _capi.check("cs_gelu_forward", code)
    return y


def gelu_backward(dy, x, approximate="none"):
    dev = _dev(dy, x)
    if dy.dtype != x.dtype or dy.numel() != x.numel():
        raise ValueError("dy and x must match")
    dx = torch.empty_like(x)
    with torch.cuda.device(dev):
        code = _capi.load().cs_gelu_backward(_ptr(dy), _ptr(x), _ptr(dx), x.numel(), _dt(x),
                                             _GELU[approximate], _stream(dev))
    _capi.check("cs_gelu_backward", code)
    return dx


# -------------------------------------------------------------- LayerNorm
def add_layernorm_forward(x, residual, gamma, beta=None, eps=1e-5, out_dtype=None, inplace=False):
    """s = x + residual; returns (s, LayerNorm(s), mean, rstd) from one pass.  `inplace` writes s over x."""
    dev = _dev(x, residual, gamma, beta)
    if residual.shape != x.shape or residual.dtype != x.dtype:
        raise ValueError("residual must match x")
    C = x.shape[-1]
    rows = x.numel() // C
    if gamma.numel() != C or (beta is not None and (beta.numel() != C or beta.dtype != gamma.dtype)):
        raise ValueError("gamma/beta must be [C] of one dtype")
    total = x if inplace else torch.empty_like(x)
    y = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=dev)
    stat = torch.float64 if x.dtype == torch.float64 else torch.float32
    mean = torch.empty(rows, dtype=stat, device=dev)
    rstd = torch.empty(rows, dtype=stat, device=dev)
    with torch.cuda.device(dev):
        code = _capi.load().cs_add_layernorm_forward(_ptr(x), _ptr(residual), _ptr(total), _ptr(gamma), _ptr(beta),
                                                     _ptr(y), _ptr(mean), _ptr(rstd), rows, C, eps, _dt(x),
                                                     _dt(y), _dt(gamma), _stream(dev))
    _capi.check("cs_add_layernorm_forward", code)
    return total, y, mean, rstd


def layernorm_forward(x, gamma, beta=None, eps=1e-5, out_dtype=None):
    """Returns (y, mean, rstd); mean and rstd are [rows] fp32 (fp64 for fp64 x)."""
    dev = _dev(x, gamma, beta)
    C = x.shape[-1]
    rows = x.numel() // C
    if gamma.numel() != C or (beta is not None and (beta.numel() != C or beta.dtype != gamma.dtype)):
        raise ValueError("gamma/beta must be [C] of one dtype")
    y = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=dev)
    stat = torch.float64 if x.dtype == torch.float64 else torch.float32
    mean = torch.empty(rows, dtype=stat, device=dev)
    rstd = torch.empty(rows, dtype=stat, device=dev)
    with torch.cuda.device(dev):
        code = _capi.load().cs_layernorm_forward(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(mean),
                                                 _ptr(rstd), rows, C, eps, _dt(x), _dt(y), _dt(gamma),
                                                 _stream(dev))
    _capi.check("cs_layernorm_forward", code)
    return y, mean, rstd


def layernorm_backward(dy, x, mean, rstd, gamma, *, need_dx=True, need_dgamma=True, need_dbeta=True,
                       dgamma=None, dbeta=None, dx_dtype=None, dresidual=None):
    """Returns (dx, dgamma, dbeta).  Passing dgamma / dbeta accumulates into them; `dresidual`
    (same shape and dtype as dx) is added to dx in the same pass."""
    dev = _dev(dy, x, mean, rstd, gamma, dgamma, dbeta, dresidual)
    if dresidual is not None and (not need_dx or dresidual.shape != x.shape
                                  or dresidual.dtype != (dx_dtype or x.dtype)):
        raise ValueError("dresidual must match dx")
    C = x.shape[-1]
    rows = x.numel() // C
    accumulate = dgamma is not None or dbeta is not None
    if accumulate and ((need_dgamma and dgamma is None) or (need_dbeta and dbeta is None)):
        raise ValueError("accumulating needs every requested parameter gradient passed in")
    dx = torch.empty(x.shape, dtype=dx_dtype or x.dtype, device=dev) if need_dx else None
    if need_dgamma and dgamma is None:
        dgamma = torch.empty(C, dtype=gamma.dtype, device=dev)
    if need_dbeta and dbeta is None:
        dbeta = torch.empty(C, dtype=gamma.dtype, device=dev)
    if not need_dgamma:
        dgamma = None
    if not need_dbeta:
        dbeta = None
    lib = _capi.load()
    ws_bytes = lib.cs_layernorm_backward_workspace_bytes(rows, C) if (need_dgamma or need_dbeta) else 0
    ws = _workspace(ws_bytes, dev) if ws_bytes else None
    with torch.cuda.device(dev):
        if dresidual is not None:
            code = lib.cs_layernorm_backward_add(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma),
                                                 _ptr(dresidual), _ptr(dx), _ptr(dgamma), _ptr(dbeta), _ptr(ws),
                                                 ws_bytes, rows, C, _dt(dy), _dt(x), _dt(dx), _dt(gamma),
                                                 int(accumulate), _stream(dev))
        else:
            code = lib.cs_layernorm_backward(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma), _ptr(dx),
                                             _ptr(dgamma), _ptr(dbeta), _ptr(ws), ws_bytes, rows, C, _dt(dy),
                                             _dt(x), _dt(dx) if dx is not None else _dt(dy), _dt(gamma),
                                             int(accumulate), _stream(dev))
    _capi.check("cs_layernorm_backward", code)
    return dx, dgamma, dbeta


def layernorm_backward_rows(dy, x, mean, rstd, gamma, *, need_dx=True, dx_dtype=None, dresidual=None):
    """First half of the backward pass as two tasks (main stream): returns (dx, partials).

    `partials` is a new fp32 tensor [partial_rows, 2, C] for `layernorm_backward_finalize`, which
    may run on another stream once this call's work is done.  Raises ValueError for shapes that
    have no split form (use `layernorm_backward`).
    """
    dev = _dev(dy, x, mean, rstd, gamma, dresidual)
    if dresidual is not None and (not need_dx or dresidual.shape != x.shape
                                  or dresidual.dtype != (dx_dtype or x.dtype)):
        raise ValueError("dresidual must match dx")
    C = x.shape[-1]
    rows = x.numel() // C
    lib = _capi.load()
    n = lib.cs_layernorm_backward_partial_rows(rows, C, _dt(x))
    if n == 0:
        raise ValueError(f"no split form for rows of {C} {x.dtype} elements")
    dx = torch.empty(x.shape, dtype=dx_dtype or x.dtype, device=dev) if need_dx else None
    partials = torch.empty((n, 2, C), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        code = lib.cs_layernorm_backward_rows(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma),
                                              _ptr(dresidual), _ptr(dx), _ptr(partials), partials.numel() * 4,
                                              rows, C, _dt(dy), _dt(x), _dt(dx) if dx is not None else _dt(dy),
                                              _dt(gamma), _stream(dev))
    _capi.check("cs_layernorm_backward_rows", code)
    return dx, partials


def layernorm_backward_finalize(partials, x_dtype, param_dtype, *, need_dgamma=True, need_dbeta=True,
                                dgamma=None, dbeta=None):
    """Second half: (dgamma, dbeta) from the partial rows, added in a fixed order.  Passing
    dgamma / dbeta accumulates into them.  `x_dtype` is the dtype of the x the rows call read."""
    dev = _dev(partials, dgamma, dbeta)
    n, two, C = partials.shape
    if two != 2 or partials.dtype != torch.float32 or not partials.is_contiguous():
        raise ValueError("partials must be the contiguous fp32 [n, 2, C] tensor of layernorm_backward_rows")
    accumulate = dgamma is not None or dbeta is not None
    if accumulate and ((need_dgamma and dgamma is None) or (need_dbeta and dbeta is None)):
        raise ValueError("accumulating needs every requested parameter gradient passed in")
    for g in (dgamma, dbeta):
        if g is not None and (g.dtype != param_dtype or g.numel() != C):
            raise ValueError("dgamma / dbeta must be [C] of the parameter dtype")
    if need_dgamma and dgamma is None:
        dgamma = torch.empty(C, dtype=param_dtype, device=dev)
    if need_dbeta and dbeta is None:
        dbeta = torch.empty(C, dtype=param_dtype, device=dev)
    if not need_dgamma:
        dgamma = None
    if not need_dbeta:
        dbeta = None
    with torch.cuda.device(dev):
        code = _capi.load().cs_layernorm_backward_finalize(_ptr(partials), n, _ptr(dgamma), _ptr(dbeta), C,
                                                           _DTYPES[x_dtype], _DTYPES[param_dtype], int(accumulate),
                                                           _stream(dev))
    _capi.check("cs_layernorm_backward_finalize", code)
    return dgamma, dbeta


class LayerNormBackwardChain:
    """LayerNorm backward calls run one after another on one stream, as a training step runs them
    (one per norm): each call's launch also adds up the partial rows the PREVIOUS call left, so
    only the last norm of the chain needs a launch for its column sums (`flush`).

    `backward` returns (dx, dgamma, dbeta) at once; dgamma / dbeta hold their values once the next
    `backward` of the chain, or `flush`, has run.  The bits are those of `layernorm_backward`.
    Shapes without partial rows (see `layernorm_backward_rows`) go through `layernorm_backward`.
    """

    def __init__(self):
        self._pending = None  # (partials, dgamma, dbeta, accumulate, C, x dtype, parameter dtype)

    def backward(self, dy, x, mean, rstd, gamma, *, dresidual=None, dgamma=None, dbeta=None, dx_dtype=None):
        dev = _dev(dy, x, mean, rstd, gamma, dgamma, dbeta, dresidual)
        C = x.shape[-1]
        rows = x.numel() // C
        if dresidual is not None and (dresidual.shape != x.shape or dresidual.dtype != (dx_dtype or x.dtype)):
            raise ValueError("dresidual must match dx")
        accumulate = dgamma is not None or dbeta is not None
        if accumulate and (dgamma is None or dbeta is None):
            raise ValueError("accumulating needs both parameter gradients passed in")
        for g in (dgamma, dbeta):
            if g is not None and (g.dtype != gamma.dtype or g.numel() != C):
                raise ValueError("dgamma / dbeta must be [C] of the parameter dtype")
        lib = _capi.load()
        n = lib.cs_layernorm_backward_partial_rows(rows, C, _dt(x))
        if n == 0:
            self.flush()
            return layernorm_backward(dy, x, mean, rstd, gamma, dgamma=dgamma, dbeta=dbeta, dx_dtype=dx_dtype,
                                      dresidual=dresidual)
        pend = self._pending
        if pend is not None and (pend[4], pend[5], pend[6]) != (C, x.dtype, gamma.dtype):
            self.flush()  # another width or type: its sums cannot ride in this launch
            pend = None
        dx = torch.empty(x.shape, dtype=dx_dtype or x.dtype, device=dev)
        if dgamma is None:
            dgamma = torch.empty(C, dtype=gamma.dtype, device=dev)
            dbeta = torch.empty(C, dtype=gamma.dtype, device=dev)
        partials = torch.empty((n, 2, C), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            code = lib.cs_layernorm_backward_rows_pending(
                _ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma), _ptr(dresidual), _ptr(dx), _ptr(partials),
                partials.numel() * 4, _ptr(pend[0]) if pend else None, pend[0].shape[0] if pend else 0,
                _ptr(pend[1]) if pend else None, _ptr(pend[2]) if pend else None, int(pend[3]) if pend else 0,
                rows, C, _dt(dy), _dt(x), _dt(dx), _dt(gamma), _stream(dev))
        _capi.check("cs_layernorm_backward_rows_pending", code)
        self._pending = (partials, dgamma, dbeta, accumulate, C, x.dtype, gamma.dtype)
        return dx, dgamma, dbeta

    def flush(self):
        """Column sums of the last call of the chain, as a launch of their own."""
        pend, self._pending = self._pending, None
        if pend is None:
            return
        partials, dgamma, dbeta, accumulate, C, x_dtype, p_dtype = pend
        with torch.cuda.device(partials.device):
            code = _capi.load().cs_layernorm_backward_finalize(_ptr(partials), partials.shape[0], _ptr(dgamma),
                                                               _ptr(dbeta), C, _DTYPES[x_dtype], _DTYPES[p_dtype],
                                                               int(accumulate), _stream(partials.device))
        _capi.check("cs_layernorm_backward_finalize", code)


# -------------------------------------------------------------- Embedding
def embedding_forward(weight, indices):
    """out[..., :] = weight[indices[...], :] (cs::compute::Embedding::forward)."""
    dev = _dev(weight, indices)
    V, C = weight.shape
    out = torch.empty(*indices.shape, C, dtype=weight.dtype, device=dev)
    with torch.cuda.device(dev):
        code = _capi.load().cs_embedding_forward(_ptr(weight), _ptr(indices), _ptr(out), indices.numel(), C,
                                                 V, _dt(weight), _ITYPES[indices.dtype], _stream(dev))
    _capi.check("cs_embedding_forward", code)
    return out


def embedding_forward_add(wte, wpe, indices):
    """out[b,t,:] = wte[indices[b,t],:] + wpe[t,:]."""
    dev = _dev(wte, wpe, indices)
    V, C = wte.shape
    B, T = indices.shape
    if wpe.shape[0] < T or wpe.shape[1] != C or wpe.dtype != wte.dtype:
        raise ValueError("wpe must be [>=T, C] of wte's dtype")
    out = torch.empty(B, T, C, dtype=wte.dtype, device=dev)
    with torch.cuda.device(dev):
        code = _capi.load().cs_embedding_forward_add(_ptr(wte), _ptr(wpe), _ptr(indices), _ptr(out), B, T, C,
                                                     V, _dt(wte), _ITYPES[indices.dtype], _stream(dev))
    _capi.check("cs_embedding_forward_add", code)
    return out


def _check_table_gradient(t, rows, C, dtype, name):
    """An existing gradient is added to with dout's element type and row length."""
    if t.dtype != dtype or tuple(t.shape) != (rows, C) or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous [{rows}, {C}] tensor of {dtype}, got {tuple(t.shape)} {t.dtype}")


def embedding_backward(dout, indices, num_weights, padding_idx=-1, dweight=None, scale_grad_by_freq=False):
    """Dense dweight [num_weights, C]; passing dweight accumulates into it.  `scale_grad_by_freq`
    divides a row's sum by the number of indices that name it."""
    C = dout.shape[-1]
    n = indices.numel()
    accumulate = dweight is not None
    if accumulate:
        _check_table_gradient(dweight, num_weights, C, dout.dtype, "dweight")
    dev = _dev(dout, indices, dweight)
    if dweight is None:
        dweight = torch.empty(num_weights, C, dtype=dout.dtype, device=dev)
    lib = _capi.load()
    ws_bytes = lib.cs_embedding_backward_workspace_bytes(n, C, num_weights)
    ws = _workspace(ws_bytes, dev)
    with torch.cuda.device(dev):
        call = lib.cs_embedding_backward_scaled if scale_grad_by_freq else lib.cs_embedding_backward
        code = call(_ptr(dout), _ptr(indices), _ptr(dweight), _ptr(ws), ws_bytes, n, C, num_weights, padding_idx,
                    _dt(dout), _ITYPES[indices.dtype], int(accumulate), _stream(dev))
    _capi.check("cs_embedding_backward", code)
    return dweight


def embedding_backward_fused(dout, indices, num_weights, dwte=None, dwpe=None):
    """(dwte, dwpe) of out = wte[ids] + wpe[pos] from dout [B,T,C]."""
    B, T, C = dout.shape
    accumulate = dwte is not None
    if (dwte is None) != (dwpe is None):
        raise ValueError("pass both gradients to accumulate, or neither")
    if accumulate:
        _check_table_gradient(dwte, num_weights, C, dout.dtype, "dwte")
        _check_table_gradient(dwpe, T, C, dout.dtype, "dwpe")
    dev = _dev(dout, indices, dwte, dwpe)
    if dwte is None:
        dwte = torch.empty(num_weights, C, dtype=dout.dtype, device=dev)
        dwpe = torch.empty(T, C, dtype=dout.dtype, device=dev)
    lib = _capi.load()
    ws_bytes = lib.cs_embedding_backward_workspace_bytes(B * T, C, num_weights)
    ws = _workspace(ws_bytes, dev)
    with torch.cuda.device(dev):
        code = lib.cs_embedding_backward_fused(_ptr(dout), _ptr(indices), _ptr(dwte), _ptr(dwpe), _ptr(ws),
                                               ws_bytes, B, T, C, num_weights, _dt(dout),
                                               _ITYPES[indices.dtype], int(accumulate), _stream(dev))
    _capi.check("cs_embedding_backward_fused", code)
    return dwte, dwpe


def embedding_backward_positions(dout, dwpe=None):
    B, T, C = dout.shape
    accumulate = dwpe is not None
    if accumulate:
        _check_table_gradient(dwpe, T, C, dout.dtype, "dwpe")
    dev = _dev(dout, dwpe)
    if dwpe is None:
        dwpe = torch.empty(T, C, dtype=dout.dtype, device=dev)
    with torch.cuda.device(dev):
        code = _capi.load().cs_embedding_backward_positions(_ptr(dout), _ptr(dwpe), B, T, C, _dt(dout),
                                                            int(accumulate), _stream(dev))
    _capi.check("cs_embedding_backward_positions", code)
    return dwpe


# ------------------------------------------------------- fused classifier
def fused_classifier(logits, targets, num_classes=None, *, ignore_index=-100, reduction="mean", dloss=1.0,
                     want_dlogits=True, inplace=False, dlogits_dtype=None, class_weight=None):
    """Softmax cross entropy with its gradient in one pass.

    logits [N, stride]; classes are columns [0, num_classes).  Returns
    (loss, row_loss, dlogits, total_weight): loss is 0-d for mean/sum and
    row_loss itself for "none"; dlogits is None unless wanted and is `logits`
    when inplace.  `class_weight` ([num_classes] fp32) weighs every row by its
    target's class, as nll_loss's `weight`.
    """
    dev = _dev(logits, targets, class_weight)
    N, stride = logits.shape
    V = stride if num_classes is None else num_classes
    if targets.dtype != torch.int64 or targets.numel() != N:
        raise ValueError("targets must be int64 [N]")
    if class_weight is not None and (class_weight.dtype != torch.float32 or class_weight.numel() != V):
        raise ValueError("class_weight must be fp32 [num_classes]")
    row_loss = torch.empty(N, dtype=torch.float32, device=dev)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    total_weight = torch.empty((), dtype=torch.float32, device=dev)
    dlogits = None
    if want_dlogits:
        if inplace:
            dlogits = logits
        else:
            dlogits = torch.empty(logits.shape, dtype=dlogits_dtype or logits.dtype, device=dev)
    lib = _capi.load()
    ws_bytes = lib.cs_fused_classifier_workspace_bytes(N)
    ws = _workspace(ws_bytes, dev)
    tail = (_ptr(ws), ws_bytes, N, V, stride, ignore_index, _REDUCTIONS[reduction], dloss, _dt(logits),
            _dt(dlogits) if dlogits is not None else _dt(logits), _stream(dev))
    with torch.cuda.device(dev):
        if class_weight is None:
            code = lib.cs_fused_classifier(_ptr(logits), _ptr(dlogits), _ptr(targets), _ptr(row_loss), _ptr(loss),
                                           _ptr(total_weight), *tail)
        else:
            code = lib.cs_fused_classifier_weighted(_ptr(logits), _ptr(dlogits), _ptr(targets), _ptr(class_weight),
                                                    _ptr(row_loss), _ptr(loss), _ptr(total_weight), *tail)
    _capi.check("cs_fused_classifier", code)
    return (row_loss if reduction == "none" else loss), row_loss, dlogits, total_weight
