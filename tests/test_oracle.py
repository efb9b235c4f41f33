"""Pins the CPU oracle (oracle/cs_oracle.c) before anything is judged by it.

Each op of the oracle is checked against
  * the ATen CPU kernels issued in the reference's own call order
    (oracle/aten_port.py) - the library routine the reference task body calls,
  * the closed form the reference's test writes out (AdamW,
    test/test_adamw.cpp:94-99) and torch.optim.AdamW (test/test_adamw.cpp:145-176),
  * what the mathematics fixes: special values, invariants, finite differences
    and brute force in float64 on tiny inputs,
chosen so that a dropped term, a wrong sign or a transposed index fails one of
them.  No GPU is used here.
"""
import math

import pytest
import torch

from _util import assert_bit_exact, assert_close, randint, randn, zipf_ids
from oracle import aten_port as ap
from oracle import c_oracle as co


# ------------------------------------------------------------------ AdamW
HYPER = dict(lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


def test_adamw_reference_test_closed_form():
    # test/test_adamw.cpp:63-103: lr 1, betas (0.9, 0.999), wd 1e-2, one step from m = v = 0
    for size in (128, 512, 1024):
        x = torch.rand(size, generator=torch.Generator().manual_seed(1))
        dx = torch.rand(size, generator=torch.Generator().manual_seed(2))
        lr, b1, b2, eps, wd, t = 1.0, 0.9, 0.999, 1e-8, 1e-2, 0
        w, m, v, _ = co.adamw_step(x, dx, torch.zeros(size), torch.zeros(size), lr=lr, beta1=b1, beta2=b2,
                                   eps=eps, weight_decay=wd, t=t + 1)
        xt = x - lr * wd * x
        mt = (1 - b1) * dx
        vt = (1 - b2) * dx.square()
        m_hat = mt / (1 - math.pow(b1, t + 1))
        v_hat = vt / (1 - math.pow(b2, t + 1))
        xt = xt - lr * m_hat / (v_hat.sqrt() + eps)
        assert torch.allclose(w, xt, 1e-4, 1e-5) and torch.allclose(m, mt, 1e-4, 1e-5)
        assert torch.allclose(v, vt, 1e-4, 1e-5)
        # The kernel narrows the hyper-parameters to float before using them (adamw.cu:45-59:
        # `one - cast_higher<UpT>(beta2)` is 1 - float(0.999), 1.3e-5 away from 0.001), which is
        # why the reference's bar above is loose.  With the same narrowing applied, the closed
        # form in float64 must agree to float rounding.
        f = lambda a: float(torch.tensor(a, dtype=torch.float32))
        lrf, b1f, b2f, epsf, wdf = f(lr), f(b1), f(b2), f(eps), f(wd)
        ibc1, ibc2 = f(1 / (1 - math.pow(b1, t + 1))), f(1 / (1 - math.pow(b2, t + 1)))
        xd, gd = x.double(), dx.double()
        md = (1 - b1f) * gd
        vd = (1 - b2f) * gd * gd
        wd_ = (xd - lrf * wdf * xd) - lrf * (md * ibc1) / ((vd * ibc2).sqrt() + epsf)
        assert_close(w.double(), wd_, atol=1e-6, rtol=1e-6, name="w (narrowed closed form)")
        assert_close(m.double(), md, atol=1e-9, rtol=1e-6, name="m")
        assert_close(v.double(), vd, atol=1e-12, rtol=1e-6, name="v")


def test_adamw_first_step_sign_form():
    # from m = v = 0: w1 = w0 (1 - lr wd) - lr g / (|g| + eps), whatever the betas
    w0 = randn(1000, 3, std=0.02)
    g = randn(1000, 4, std=1e-3)
    w, m, v, _ = co.adamw_step(w0, g, torch.zeros(1000), torch.zeros(1000), t=1, **HYPER)
    want = w0.double() * (1 - HYPER["lr"] * HYPER["weight_decay"]) - HYPER["lr"] * g.double() / (
        g.double().abs() + HYPER["eps"])
    assert_close(w.double(), want, atol=1e-9, name="w1")


@pytest.mark.parametrize("amsgrad", [False, True])
def test_adamw_ten_steps_match_torch_optim(amsgrad):
    # test/test_adamw.cpp:145-176 compares with torch::optim::AdamW
    n = 4096
    w0 = randn(n, 10, std=0.02)
    p = torch.nn.Parameter(w0.clone())
    opt = torch.optim.AdamW([p], lr=HYPER["lr"], betas=(HYPER["beta1"], HYPER["beta2"]), eps=HYPER["eps"],
                            weight_decay=HYPER["weight_decay"], amsgrad=amsgrad, foreach=False)
    w, m, v = w0.clone(), torch.zeros(n), torch.zeros(n)
    vmax = torch.zeros(n) if amsgrad else None
    for t in range(1, 11):
        g = randn(n, 100 + t, std=1e-3)
        p.grad = g.clone()
        opt.step()
        w, m, v, vmax = co.adamw_step(w, g, m, v, t=t, v_max=vmax, **HYPER)
    if amsgrad:
        # torch keeps max(v) and divides by sqrt(max_v)/sqrt(bc2); the reference keeps max(v_hat)
        # (adamw.cu:82-84).  They differ by design, so only the plain path is compared to torch.
        return
    assert_close(w, p.detach(), atol=1e-7, name="w after 10 steps")
    assert_close(m, opt.state[p]["exp_avg"], atol=1e-9, name="m")
    assert_close(v, opt.state[p]["exp_avg_sq"], atol=1e-12, name="v")


def test_adamw_amsgrad_keeps_running_max_of_v_hat():
    n = 64
    w, m, v, vmax = randn(n, 1), torch.zeros(n), torch.zeros(n), torch.zeros(n)
    seen = torch.zeros(n, dtype=torch.float64)
    for t in range(1, 6):
        g = randn(n, 20 + t) * (1.0 if t != 3 else 10.0)  # a spike at step 3 must stick
        w, m, v, vmax = co.adamw_step(w, g, m, v, t=t, v_max=vmax, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
                                      weight_decay=0.0)
        v_hat = v.double() / (1 - 0.999 ** t)
        seen = torch.maximum(seen, v_hat)
        assert_close(vmax.double(), seen, atol=1e-12, rtol=1e-5, name=f"vmax t={t}")


def test_adamw_f64_agrees_with_f32_and_with_double_brute_force():
    n = 257
    w0, g = randn(n, 5, std=0.02), randn(n, 6, std=1e-3)
    w32, *_ = co.adamw_step(w0, g, torch.zeros(n), torch.zeros(n), t=7, **HYPER)
    w64, m64, v64, _ = co.adamw_step(w0.double(), g.double(), torch.zeros(n).double(), torch.zeros(n).double(),
                                     t=7, **HYPER)
    assert_close(w32.double(), w64, atol=1e-9, name="f32 vs f64")
    b1, b2 = HYPER["beta1"], HYPER["beta2"]
    mm, vv = (1 - b1) * g.double(), (1 - b2) * g.double() ** 2
    want = w0.double() * (1 - HYPER["lr"] * HYPER["weight_decay"]) - HYPER["lr"] * (mm / (1 - b1 ** 7)) / (
        (vv / (1 - b2 ** 7)).sqrt() + HYPER["eps"])
    assert_close(w64, want, atol=1e-15, rtol=1e-12, name="f64 brute force")


# ------------------------------------------------------------------- GeLU
@pytest.mark.parametrize("norm_type", [2.0, float("inf")])
def test_clip_grad_norm_matches_torch_and_closed_forms(norm_type):
    # Utils::clip_grad_norm_ (src/compute/utils.cpp:700-746) restates torch.nn.utils.clip_grad_norm_
    g = [randn((1000,), 1), randn((37, 5), 2), randn((1,), 3)]
    ps = [torch.nn.Parameter(torch.zeros_like(x)) for x in g]
    for p, x in zip(ps, g):
        p.grad = x.clone()
    ref = torch.nn.utils.clip_grad_norm_(ps, 0.5, norm_type=norm_type, foreach=False)
    out, total, coef = co.clip_grad_norm(g, 0.5, norm_type)
    assert abs(total - ref.item()) <= 1e-6 * ref.item()
    for p, o in zip(ps, out):
        assert torch.allclose(p.grad, o, rtol=1e-6, atol=0)
    # closed forms: n copies of c have 2-norm c sqrt(n) and largest magnitude c; the coefficient is
    # max_norm / (total + 1e-6), and 1 (gradients untouched, bit for bit) when total <= max_norm
    ones = [torch.full((50,), 2.0), torch.full((14,), -2.0)]
    out, total, coef = co.clip_grad_norm(ones, 4.0, norm_type)
    want = 16.0 if norm_type == 2.0 else 2.0
    assert total == want and abs(coef - min(1.0, 4.0 / (want + 1e-6))) < 1e-7
    if norm_type == 2.0:
        assert all(torch.allclose(o, x * 0.25, rtol=1e-6) for o, x in zip(out, ones))
    out, total, coef = co.clip_grad_norm(g, 1e6, norm_type)
    assert coef == 1.0 and all(torch.equal(o, x) for o, x in zip(out, g))
    # a sign error or a dropped tensor would show here: the norm of the concatenation
    brute = torch.cat([x.flatten().double() for x in g])
    want = brute.abs().max().item() if norm_type != 2.0 else brute.square().sum().sqrt().item()
    assert abs(co.clip_grad_norm(g, 1.0, norm_type)[1] - want) <= 1e-6 * want


@pytest.mark.parametrize("mode", ["none", "tanh"])
def test_gelu_matches_aten_cpu(mode):
    x = randn(20000, 11, std=1.5)
    dy = randn(20000, 12)
    # atol 1e-6: the expression 1 + erf(.) / 1 + tanh(.) cancels for x << 0, so fp32
    # results are only defined to ~6e-8 * |x| there, whichever library evaluates them
    assert_close(co.gelu_forward(x, mode), ap.gelu_forward(x, mode), atol=1e-6, name="fwd")
    # backward multiplies that floor by |dy| (up to ~4 here) and by terms of order |x|
    assert_close(co.gelu_backward(dy, x, mode), ap.gelu_backward(dy, x, mode), atol=5e-6, name="bwd")
    xd, dyd = x.double(), dy.double()
    assert_close(co.gelu_forward(xd, mode), ap.gelu_forward(xd, mode), atol=1e-14, name="fwd f64")
    assert_close(co.gelu_backward(dyd, xd, mode), ap.gelu_backward(dyd, xd, mode), atol=1e-14, name="bwd f64")


@pytest.mark.parametrize("mode", ["none", "tanh"])
def test_gelu_special_values_and_derivative(mode):
    x = torch.tensor([0.0, 30.0, -30.0, 1.0], dtype=torch.float64)
    y = co.gelu_forward(x, mode)
    assert y[0] == 0 and y[1] == 30.0 and abs(y[2]) < 1e-30
    if mode == "none":
        assert abs(y[3].item() - 0.5 * (1 + math.erf(1 / math.sqrt(2)))) < 1e-15
    else:
        assert abs(y[3].item() - 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715))) < 1e-15
    one = torch.ones(4, dtype=torch.float64)
    d = co.gelu_backward(one, x, mode)
    assert abs(d[0].item() - 0.5) < 1e-15 and abs(d[1].item() - 1) < 1e-12 and abs(d[2].item()) < 1e-12
    # central differences pin the derivative (a wrong sign or a dropped term is O(1) off)
    xs = torch.linspace(-4, 4, 161, dtype=torch.float64)
    h = 1e-6
    fd = (co.gelu_forward(xs + h, mode) - co.gelu_forward(xs - h, mode)) / (2 * h)
    assert_close(co.gelu_backward(torch.ones_like(xs), xs, mode), fd, atol=1e-8, name="d/dx")
    # dy scales linearly
    assert_close(co.gelu_backward(3 * torch.ones_like(xs), xs, mode), 3 * fd, atol=1e-7, name="3 d/dx")


def test_gelu_bf16_storage_rule():
    x = randn(4096, 13, std=1.5, dtype=torch.bfloat16)
    want = ap.gelu_forward(x.float(), "tanh").to(torch.bfloat16)
    assert_close(co.gelu_forward(x, "tanh"), want, atol=1e-6, name="bf16 fwd")


# -------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("rows,C", [(64, 768), (7, 384), (3, 50)])
def test_layernorm_matches_aten_cpu(rows, C):
    x = randn((rows, C), 21)
    gamma, beta = randn(C, 22, std=0.02, mean=1.0), randn(C, 23, std=0.02)
    dy = randn((rows, C), 24)
    y, mean, rstd = co.layernorm_forward(x, gamma, beta, 1e-5)
    y2, mean2, rstd2 = ap.layernorm_forward(x, gamma, beta, 1e-5)
    assert_close(y, y2, atol=2e-6, name="y")
    assert_close(mean, mean2.flatten(), atol=1e-7, name="mean")
    assert_close(rstd, rstd2.flatten(), atol=1e-6, name="rstd")
    dx, dg, db = co.layernorm_backward(dy, x, mean, rstd, gamma)
    dx2, dg2, db2 = ap.layernorm_backward(dy, x, mean2, rstd2, gamma, beta)
    # ATen's CPU backward uses a form with more cancellation (a*dy*g + b*x + c); ~1e-6 abs on O(1) data
    assert_close(dx, dx2, atol=5e-6, name="dx")
    assert_close(dg, dg2, atol=2e-5, name="dgamma")
    assert_close(db, db2, atol=2e-5, name="dbeta")
    # no-bias path (src/compute/layer_norm.cpp:198-204)
    y3, _, _ = co.layernorm_forward(x, gamma, None, 1e-5)
    assert_close(y3, ap.layernorm_forward(x, gamma, None, 1e-5)[0], atol=2e-6, name="y no bias")


def test_layernorm_invariants_and_brute_force():
    rows, C = 5, 32
    x = randn((rows, C), 31).double()
    gamma, beta = torch.ones(C, dtype=torch.float64), torch.zeros(C, dtype=torch.float64)
    y, mean, rstd = co.layernorm_forward(x, gamma, beta, 1e-5)
    assert_close(y.mean(1), torch.zeros(rows, dtype=torch.float64), atol=1e-14, name="row mean 0")
    var = x.var(1, unbiased=False)
    assert_close(rstd, 1 / (var + 1e-5).sqrt(), atol=1e-14, name="rstd")
    assert_close(y.var(1, unbiased=False), var / (var + 1e-5), atol=1e-13, name="row var")
    # constant row -> y = beta
    yc, _, _ = co.layernorm_forward(torch.full((1, C), 3.0, dtype=torch.float64), randn(C, 1).double(),
                                    randn(C, 2).double(), 1e-5)
    assert_close(yc[0], randn(C, 2).double(), atol=1e-12, name="constant row")
    # autograd of the textbook formula in float64
    g2, b2 = randn(C, 32).double(), randn(C, 33).double()
    xa, ga, ba = x.clone().requires_grad_(), g2.clone().requires_grad_(), b2.clone().requires_grad_()
    mu = xa.mean(1, keepdim=True)
    yy = (xa - mu) / ((xa - mu).pow(2).mean(1, keepdim=True) + 1e-5).sqrt() * ga + ba
    dy = randn((rows, C), 34).double()
    yy.backward(dy)
    _, mean, rstd = co.layernorm_forward(x, g2, b2, 1e-5)
    dx, dg, db = co.layernorm_backward(dy, x, mean, rstd, g2)
    assert_close(dx, xa.grad, atol=1e-12, name="dx")
    assert_close(dg, ga.grad, atol=1e-12, name="dgamma")
    assert_close(db, ba.grad, atol=1e-12, name="dbeta")
    assert dx.sum(1).abs().max() < 1e-10  # each dx row sums to 0 when gamma is applied before centring
    # accumulate (+= into an existing gradient, layer_norm.cpp:325-334)
    _, dg2, db2 = co.layernorm_backward(dy, x, mean, rstd, g2, dgamma=dg, dbeta=db)
    assert_close(dg2, 2 * dg, atol=1e-12, name="dgamma +=")
    assert_close(db2, 2 * db, atol=1e-12, name="dbeta +=")


def test_layernorm_bf16_storage_rule():
    x = randn((16, 768), 41, dtype=torch.bfloat16)
    gamma, beta = randn(768, 42, std=0.02, mean=1.0), randn(768, 43, std=0.02)
    y, mean, rstd = co.layernorm_forward(x, gamma, beta, 1e-5)
    y2, mean2, rstd2 = ap.layernorm_forward(x, gamma, beta, 1e-5)  # mixed call: fp32 statistics, bf16 y
    assert y.dtype == torch.bfloat16 and mean2.dtype == torch.float32
    assert_close(y, y2, atol=1e-6, name="y bf16")
    assert_close(mean, mean2.flatten(), atol=1e-7, name="mean")
    assert_close(rstd, rstd2.flatten(), atol=1e-6, name="rstd")


# -------------------------------------------------------------- Embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("idx_dtype", [torch.int32, torch.int64])
def test_embedding_forward_is_atens_gather(dtype, idx_dtype):
    w = randn((97, 24), 51, dtype=dtype)
    ids = randint(0, 97, (3, 11), 52, dtype=idx_dtype)
    assert_bit_exact(co.embedding_forward(w, ids), ap.embedding_forward(w, ids.long()).reshape(3, 11, 24), "gather")
    wpe = randn((11, 24), 53, dtype=dtype)
    assert_bit_exact(co.embedding_forward_add(w, wpe, ids), ap.token_position_forward(w, wpe, ids.long()),
                     "gather-add")


def test_cross_entropy_with_class_weights():
    """at::nll_loss's `weight` (src/compute/cross_entropy.cpp:52-63, 97-105): the C restatement against
    the reference's ATen op sequence called with a weight, and against the closed form in float64."""
    g = torch.Generator().manual_seed(31)
    N, V = 37, 11
    x = torch.randn((N, V), generator=g) * 2
    t = torch.randint(0, V, (N,), generator=g)
    t[::6] = -100
    w = torch.rand(V, generator=g) + 0.1
    for reduction, code in (("mean", 1), ("sum", 2), ("none", 0)):
        loss, row, d, tw = co.cross_entropy(x, t, reduction=reduction, class_weight=w)
        a_loss, a_grad, a_tw = ap.cross_entropy(x, t, reduction=code, weight=w)
        if reduction != "none":
            assert_close(loss, a_loss, atol=1e-6, name=f"{reduction}: loss vs ATen")
            assert_close(d, a_grad, atol=1e-8, name=f"{reduction}: gradient vs ATen")
            assert_close(tw, a_tw, atol=1e-6, name=f"{reduction}: total weight vs ATen")
        else:
            assert_close(row, a_loss, atol=1e-6, name="none: row losses vs ATen")
    live = t != -100
    lp = torch.log_softmax(x.double(), 1)
    wt = torch.where(live, w.double()[t.clamp(min=0)], torch.zeros((), dtype=torch.float64))
    nll = -lp[torch.arange(N), t.clamp(min=0)] * wt
    loss, row, d, tw = co.cross_entropy(x, t, class_weight=w)
    assert_close(tw.double(), wt.sum(), atol=1e-6, name="total weight = sum of the targets' weights")
    assert_close(loss.double(), nll.sum() / wt.sum(), atol=1e-6, name="weighted mean")
    onehot = torch.zeros((N, V), dtype=torch.float64)
    onehot[torch.arange(N)[live], t[live]] = 1
    want = (lp.exp() - onehot) * (wt / wt.sum())[:, None]
    assert_close(d.double(), want, atol=1e-8, name="(softmax - onehot) w_t / sum w")
    # all weights 1 is the unweighted call
    same = co.cross_entropy(x, t, class_weight=torch.ones(V))
    plain = co.cross_entropy(x, t)
    for a, b in zip(same, plain):
        assert torch.equal(a, b)


def test_embedding_backward_matches_aten_and_brute_force():
    # the reference's own case: 2048 contributions over 3 rows (test/test_embedding.cpp:70-72), scaled down
    V, C = 40, 16
    ids = randint(0, 3, (2, 128), 61)
    dout = randn((2, 128, C), 62)
    got = co.embedding_backward(dout, ids, V)
    assert_close(got, ap.embedding_backward(dout, ids, V), atol=2e-5, name="hot rows")
    want = torch.zeros(V, C, dtype=torch.float64)
    for i, k in enumerate(ids.flatten().tolist()):
        want[k] += dout.reshape(-1, C)[i].double()
    assert_close(got.double(), want, atol=1e-6, name="loop")
    assert (got[3:] == 0).all()  # untouched rows are exactly zero
    assert_close(got.sum(0), dout.reshape(-1, C).sum(0), atol=1e-4, name="column sums")
    # padding row gets nothing; accumulate adds to what is there
    got_pad = co.embedding_backward(dout, ids, V, padding_idx=1)
    assert (got_pad[1] == 0).all() and torch.equal(got_pad[0], got[0])
    assert_close(co.embedding_backward(dout, ids, V, dweight=got), 2 * got, atol=1e-6, name="+=")
    assert_close(got_pad, ap.embedding_backward(dout, ids, V, 1), atol=2e-5, name="padding_idx")


def test_embedding_backward_scaled_by_frequency():
    """scale_grad_by_freq: against the ATen CPU op the reference calls with that option, and against
    the closed form (a row's mean over the entries that name it) in float64."""
    g = torch.Generator().manual_seed(77)
    V, C = 23, 12
    ids = torch.randint(0, 6, (5, 40), generator=g)  # few ids, many repeats
    ids[0, :3] = 20
    dout = torch.randn((5, 40, C), generator=g)
    got = co.embedding_backward(dout, ids, V, scale_grad_by_freq=True)
    assert_close(got, ap.embedding_backward(dout, ids, V, scale_grad_by_freq=True), atol=2e-6, name="ATen, scaled")
    flat, d = ids.reshape(-1), dout.reshape(-1, C).double()
    for k in range(V):
        rows = d[flat == k]
        want = rows.mean(0) if len(rows) else torch.zeros(C, dtype=torch.float64)
        assert_close(got[k], want.float(), atol=1e-6, name=f"row {k}: mean of its entries")
    assert not torch.allclose(got, co.embedding_backward(dout, ids, V))  # the option does something
    # with a padding row, and added to an existing gradient (only the new part is scaled)
    pad = co.embedding_backward(dout, ids, V, padding_idx=2, scale_grad_by_freq=True)
    assert_close(pad, ap.embedding_backward(dout, ids, V, 2, True), atol=2e-6, name="ATen, scaled, padding row")
    assert pad[2].abs().max() == 0
    base = torch.randn((V, C), generator=g)
    assert_close(co.embedding_backward(dout, ids, V, dweight=base.clone(), scale_grad_by_freq=True), base + got, atol=1e-6,
                 name="+= of the scaled sums")


def test_embedding_backward_bf16_uses_fp32_accumulation():
    V, C = 30, 8
    ids = randint(0, 3, (4, 256), 63)
    dout = randn((4, 256, C), 64, dtype=torch.bfloat16)
    got = co.embedding_backward(dout, ids, V)
    want = ap.embedding_backward(dout.float(), ids, V).to(torch.bfloat16)  # widen first, round once
    assert_close(got, want, atol=1e-6, name="bf16")


def test_embedding_positions_and_zipf():
    B, T, C, V = 4, 16, 8, 50
    dout = randn((B, T, C), 65)
    ids = zipf_ids(B * T, V, 66).reshape(B, T)
    dwte, dwpe = ap.token_position_backward(dout, ids, V)
    assert_close(co.embedding_backward_positions(dout), dwpe, atol=1e-6, name="dwpe")
    assert_close(co.embedding_backward(dout, ids, V), dwte, atol=1e-5, name="dwte zipf")


# ---------------------------------------------------------- Cross entropy
@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_cross_entropy_matches_aten_cpu(reduction):
    N, V = 64, 384  # test/test_cross_entropy.cpp:69-99 uses [128*256, 384]
    x = torch.rand((N, V), generator=torch.Generator().manual_seed(71))
    t = randint(0, V, (N,), 72)
    red = {"none": 0, "mean": 1, "sum": 2}[reduction]
    loss, row, d, tw = co.cross_entropy(x, t, reduction=reduction)
    loss2, d2, tw2 = ap.cross_entropy(x, t, reduction=red)
    assert_close(loss, loss2, atol=1e-6, name="loss")
    assert_close(d, d2, atol=1e-9, name="dlogits")
    want = torch.nn.functional.cross_entropy(x, t, reduction=reduction)
    assert_close(loss, want, atol=1e-6, name="cross_entropy_loss")


def test_cross_entropy_ignore_index_and_padding():
    N, V, stride = 32, 50, 64
    x = randn((N, stride), 73, std=2.0)
    t = randint(0, V, (N,), 74)
    t[::5] = -100
    loss, row, d, tw = co.cross_entropy(x, t, num_classes=V)
    xs = x[:, :V].contiguous()
    loss2, d2, tw2 = ap.cross_entropy(xs, t)
    assert tw.item() == tw2.item() == (t != -100).sum().item()
    assert_close(loss, loss2, atol=1e-6, name="loss")
    assert_close(d[:, :V].contiguous(), d2, atol=1e-9, name="dlogits")
    assert (d[:, V:] == 0).all() and (d[::5] == 0).all() and (row[::5] == 0).all()
    # V == stride reduces to the reference's case (it softmaxes over all 50304 columns)
    loss3, _, d3, _ = co.cross_entropy(x, t, num_classes=stride)
    loss4, d4, _ = ap.cross_entropy(x, t)
    assert_close(loss3, loss4, atol=1e-6, name="loss V==stride")
    assert_close(d3, d4, atol=1e-9, name="dlogits V==stride")


def test_cross_entropy_closed_forms():
    N, V = 6, 11
    t = randint(0, V, (N,), 75)
    # equal logits -> log V, softmax 1/V
    loss, row, d, _ = co.cross_entropy(torch.full((N, V), 0.7, dtype=torch.float64), t)
    assert_close(row, torch.full((N,), math.log(V), dtype=torch.float64), atol=1e-14, name="log V")
    want = torch.full((N, V), 1.0 / V, dtype=torch.float64)
    want[torch.arange(N), t] -= 1
    assert_close(d, want / N, atol=1e-15, name="uniform softmax")
    # brute force in float64 + shift invariance + rows sum to zero + dloss scales
    x = randn((N, V), 76, std=2.0).double()
    loss, row, d, _ = co.cross_entropy(x, t)
    lse = torch.logsumexp(x, 1)
    assert_close(row, lse - x[torch.arange(N), t], atol=1e-13, name="lse - x_t")
    assert abs(loss.item() - row.mean().item()) < 1e-14
    assert d.sum(1).abs().max() < 1e-15
    loss_s, _, d_s, _ = co.cross_entropy(x + 123.0, t)
    assert_close(d_s, d, atol=1e-13, name="shift")
    _, _, d2, _ = co.cross_entropy(x, t, dloss=-2.5)
    assert_close(d2, -2.5 * d, atol=1e-15, name="dloss")
    # finite differences of the mean loss
    h = 1e-6
    xp, xm = x.clone(), x.clone()
    xp[2, 3] += h
    xm[2, 3] -= h
    fd = (co.cross_entropy(xp, t)[0] - co.cross_entropy(xm, t)[0]) / (2 * h)
    assert abs(fd.item() - d[2, 3].item()) < 1e-8


def test_cross_entropy_amp_rule():
    # test/test_cross_entropy.cpp:102-139: bf16 logits, fp32 math, fp32 gradient
    N, V = 16, 384
    x = randn((N, V), 77, std=2.0, dtype=torch.bfloat16)
    t = randint(0, V, (N,), 78)
    loss, _, d, _ = co.cross_entropy(x, t, dlogits_dtype=torch.float32)
    loss2, d2, _ = ap.cross_entropy(x.float(), t)
    assert_close(loss, loss2, atol=1e-6, name="loss")
    assert_close(d, d2, atol=1e-9, name="dlogits fp32")
    _, _, d16, _ = co.cross_entropy(x, t)
    assert_close(d16, d2.to(torch.bfloat16), atol=1e-9, name="dlogits bf16")
