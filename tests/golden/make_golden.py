"""Writes tests/golden/*.npz: small input/output vectors for every op of the hot path.

The expected outputs come from the installed ATen CPU kernels, called in the
reference's own order (oracle/aten_port.py), and for AdamW from
torch.optim.AdamW (what test/test_adamw.cpp:145-176 compares with).  16-bit
cases follow the reference's AMP rule: widen to fp32, compute, round once.
The fixtures are data only; rerun this script to regenerate them:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import aten_port as ap  # noqa: E402


def g(seed):
    return torch.Generator().manual_seed(seed)


def bits(t):
    """bf16 tensors are stored as their uint16 bit patterns (numpy has no bfloat16)."""
    return t.contiguous().view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.numpy()


def save(name, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **{k: bits(v) if torch.is_tensor(v) else v
                                                              for k, v in arrays.items()})


def main():
    torch.set_num_threads(1)
    # ---- cross entropy: fp32, and bf16 logits with fp32 gradient (the AMP rule), one ignored row
    N, V, stride = 24, 203, 208
    x = torch.randn((N, stride), generator=g(1)) * 2
    t = torch.randint(0, V, (N,), generator=g(2))
    t[5] = -100
    loss, d, tw = ap.cross_entropy(x[:, :V].contiguous(), t)
    save("cross_entropy_f32", logits=x, targets=t, num_classes=np.int64(V), loss=loss, dlogits=d, total_weight=tw)
    xb = x.to(torch.bfloat16)
    loss, d, tw = ap.cross_entropy(xb.float()[:, :V].contiguous(), t)
    save("cross_entropy_bf16", logits=xb, targets=t, num_classes=np.int64(V), loss=loss, dlogits_f32=d,
         dlogits_bf16=d.to(torch.bfloat16), total_weight=tw)
    # ---- layer norm: fp32 and bf16 x with fp32 parameters
    rows, C = 20, 96
    x = torch.randn((rows, C), generator=g(3))
    gamma, beta = torch.randn(C, generator=g(4)) * 0.02 + 1, torch.randn(C, generator=g(5)) * 0.02
    dy = torch.randn((rows, C), generator=g(6))
    y, mean, rstd = ap.layernorm_forward(x, gamma, beta)
    dx, dg, db = ap.layernorm_backward(dy, x, mean, rstd, gamma, beta)
    save("layernorm_f32", x=x, gamma=gamma, beta=beta, dy=dy, y=y, mean=mean.flatten(), rstd=rstd.flatten(), dx=dx,
         dgamma=dg, dbeta=db)
    xb, dyb = x.to(torch.bfloat16), dy.to(torch.bfloat16)
    y, mean, rstd = ap.layernorm_forward(xb.float(), gamma, beta)
    dx, dg, db = ap.layernorm_backward(dyb.float(), xb.float(), mean, rstd, gamma, beta)
    save("layernorm_bf16", x=xb, gamma=gamma, beta=beta, dy=dyb, y=y.to(torch.bfloat16), mean=mean.flatten(),
         rstd=rstd.flatten(), dx=dx.to(torch.bfloat16), dgamma=dg, dbeta=db)
    # ---- gelu, both forms
    x = torch.cat([torch.randn(500, generator=g(7)) * 1.5, torch.tensor([0.0, -6.0, 6.0, -0.5, 0.5])])
    dy = torch.randn(x.numel(), generator=g(8))
    for mode in ("none", "tanh"):
        save(f"gelu_{mode}_f32", x=x, dy=dy, y=ap.gelu_forward(x, mode), dx=ap.gelu_backward(dy, x, mode))
        xb, dyb = x.to(torch.bfloat16), dy.to(torch.bfloat16)
        save(f"gelu_{mode}_bf16", x=xb, dy=dyb, y=ap.gelu_forward(xb.float(), mode).to(torch.bfloat16),
             dx=ap.gelu_backward(dyb.float(), xb.float(), mode).to(torch.bfloat16))
    # ---- embedding: token + position, hot rows (ids in [0, 3)) and spread ids
    B, T, C, V = 3, 40, 16, 50
    wte, wpe = torch.randn((V, C), generator=g(9)), torch.randn((T, C), generator=g(10))
    dout = torch.randn((B, T, C), generator=g(11))
    for tag, ids in (("hot", torch.randint(0, 3, (B, T), generator=g(12))),
                     ("spread", torch.randint(0, V, (B, T), generator=g(13)))):
        dwte, dwpe = ap.token_position_backward(dout, ids, V)
        save(f"embedding_{tag}_f32", wte=wte, wpe=wpe, ids=ids, dout=dout, out=ap.token_position_forward(wte, wpe, ids),
             gather=ap.embedding_forward(wte, ids).reshape(B, T, C), dwte=dwte, dwpe=dwpe)
        wb, pb, db_ = wte.to(torch.bfloat16), wpe.to(torch.bfloat16), dout.to(torch.bfloat16)
        dwte, dwpe = ap.token_position_backward(db_.float(), ids, V)
        save(f"embedding_{tag}_bf16", wte=wb, wpe=pb, ids=ids, dout=db_, out=ap.token_position_forward(wb, pb, ids),
             dwte=dwte.to(torch.bfloat16), dwpe=dwpe.to(torch.bfloat16))
    # ---- AdamW: five steps of torch.optim.AdamW
    n = 300
    w0 = torch.randn(n, generator=g(14)) * 0.02
    grads = torch.stack([torch.randn(n, generator=g(20 + i)) * 1e-3 for i in range(5)])
    p = torch.nn.Parameter(w0.clone())
    opt = torch.optim.AdamW([p], lr=6e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, foreach=False)
    ws = []
    for i in range(5):
        p.grad = grads[i].clone()
        opt.step()
        ws.append(p.detach().clone())
    save("adamw_f32", w0=w0, grads=grads, w=torch.stack(ws), m=opt.state[p]["exp_avg"], v=opt.state[p]["exp_avg_sq"],
         hyper=np.array([6e-4, 0.9, 0.95, 1e-8, 0.1]))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
