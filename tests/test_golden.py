"""The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the
ATen CPU kernels in the reference's call order) against the C oracle (no GPU needed) and against the
HIP kernels through the C ABI (marked gpu).  Same bar as everywhere else: tests/_util.py."""
import os

import numpy as np
import pytest
import torch

from _util import assert_bit_exact, assert_close

HERE = os.path.dirname(os.path.abspath(__file__))


def load(name):
    out = {}
    with np.load(os.path.join(HERE, "golden", name + ".npz"), allow_pickle=False) as z:
        for k in z.files:
            a = z[k]
            if a.dtype == np.uint16:  # bfloat16 bit patterns
                out[k] = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
            elif a.shape == ():
                out[k] = torch.tensor(a.item()) if a.dtype.kind == "f" else int(a)
            else:
                out[k] = torch.from_numpy(a.copy())
    return out


def backends():
    from oracle import c_oracle

    yield pytest.param(("oracle", c_oracle, lambda t: t), id="oracle")
    yield pytest.param(("hip", None, lambda t: None if t is None else t.to("cuda:0")), id="hip",
                       marks=pytest.mark.gpu)


@pytest.fixture(params=list(backends()))
def be(request):
    kind, mod, to = request.param
    if kind == "hip":
        from core_scheduler_amd import ops

        mod = ops
    return kind, mod, to


def test_cross_entropy_vectors(be):
    kind, m, to = be
    f = load("cross_entropy_f32")
    ce = m.cross_entropy if kind == "oracle" else m.fused_classifier
    loss, row, d, tw = ce(to(f["logits"]), to(f["targets"]), f["num_classes"])
    assert_close(loss.float(), f["loss"], atol=1e-6, name="loss")
    assert_close(d[:, :f["num_classes"]].contiguous(), f["dlogits"], atol=1e-9, name="dlogits")
    assert (d[:, f["num_classes"]:] == 0).all() and tw.item() == f["total_weight"].item()
    b = load("cross_entropy_bf16")
    loss, row, d, tw = ce(to(b["logits"]), to(b["targets"]), b["num_classes"], dlogits_dtype=torch.float32)
    assert_close(loss.float(), b["loss"], atol=1e-6, name="loss bf16")
    assert_close(d[:, :b["num_classes"]].contiguous(), b["dlogits_f32"], atol=1e-9, name="dlogits fp32 from bf16")
    _, _, d16, _ = ce(to(b["logits"]), to(b["targets"]), b["num_classes"])
    assert_close(d16[:, :b["num_classes"]].contiguous(), b["dlogits_bf16"], atol=1e-9, name="dlogits bf16")


@pytest.mark.parametrize("name", ["layernorm_f32", "layernorm_bf16"])
def test_layernorm_vectors(be, name):
    kind, m, to = be
    f = load(name)
    y, mean, rstd = m.layernorm_forward(to(f["x"]), to(f["gamma"]), to(f["beta"]), 1e-5)
    assert_close(y, f["y"], atol=2e-6, name="y")
    assert_close(mean.float(), f["mean"], atol=1e-7, name="mean")
    assert_close(rstd.float(), f["rstd"], atol=1e-6, name="rstd")
    dx, dg, db = m.layernorm_backward(to(f["dy"]), to(f["x"]), to(f["mean"]), to(f["rstd"]), to(f["gamma"]))
    assert_close(dx, f["dx"], atol=5e-6, name="dx")
    assert_close(dg, f["dgamma"], atol=5e-6, name="dgamma")
    assert_close(db, f["dbeta"], atol=5e-6, name="dbeta")


@pytest.mark.parametrize("mode", ["none", "tanh"])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_gelu_vectors(be, mode, dt):
    kind, m, to = be
    f = load(f"gelu_{mode}_{dt}")
    assert_close(m.gelu_forward(to(f["x"]), mode), f["y"], atol=1e-6, name="y")
    assert_close(m.gelu_backward(to(f["dy"]), to(f["x"]), mode), f["dx"], atol=5e-6, name="dx")


@pytest.mark.parametrize("tag", ["hot", "spread"])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_embedding_vectors(be, tag, dt):
    kind, m, to = be
    f = load(f"embedding_{tag}_{dt}")
    V = f["wte"].shape[0]
    assert_bit_exact(m.embedding_forward_add(to(f["wte"]), to(f["wpe"]), to(f["ids"])), f["out"], "gather-add")
    if "gather" in f:
        assert_bit_exact(m.embedding_forward(to(f["wte"]), to(f["ids"])), f["gather"], "gather")
    atol = 1e-5 if dt == "f32" else 1e-6
    assert_close(m.embedding_backward(to(f["dout"]), to(f["ids"]), V), f["dwte"], atol=atol, name="dwte")
    assert_close(m.embedding_backward_positions(to(f["dout"])), f["dwpe"], atol=atol, name="dwpe")
    if kind == "hip":
        dwte, dwpe = m.embedding_backward_fused(to(f["dout"]), to(f["ids"]), V)
        assert_close(dwte, f["dwte"], atol=atol, name="dwte fused")
        assert_close(dwpe, f["dwpe"], atol=atol, name="dwpe fused")


def test_adamw_vectors(be):
    kind, m, to = be
    f = load("adamw_f32")
    lr, b1, b2, eps, wd = [float(x) for x in f["hyper"]]
    w = to(f["w0"].clone())
    mm, vv = to(torch.zeros_like(f["w0"])), to(torch.zeros_like(f["w0"]))
    for t in range(5):
        g = to(f["grads"][t].contiguous())
        if kind == "oracle":
            w, mm, vv, _ = m.adamw_step(w, g, mm, vv, lr=lr, beta1=b1, beta2=b2, eps=eps, weight_decay=wd, t=t + 1)
        else:
            m.adamw_step(w, g, mm, vv, lr=lr, beta1=b1, beta2=b2, eps=eps, weight_decay=wd, t=t + 1)
        assert_close(w, f["w"][t], atol=1e-7, name=f"w step {t + 1}")
    assert_close(mm, f["m"], atol=1e-9, name="m")
    assert_close(vv, f["v"], atol=1e-12, name="v")
