"""The C++ host API (cs::compute / cs::optimizer over the C ABI), driven the way the reference's
gtest suites drive theirs: a DynamicScheduler, op states, forward / backward, wait, compare.

Cases follow test/test_gelu.cpp, test_embedding.cpp, test_cross_entropy.cpp, test_layer_norm.cpp,
test_adamw.cpp and test_autocast.cpp of the reference; expected values come from the CPU oracle.
The error-convention tests at the bottom need no GPU.
"""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

from _util import assert_bit_exact, assert_close, randint, randn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


@pytest.fixture(scope="module")
def host():
    from core_scheduler_amd import _cs_host

    return _cs_host


@pytest.fixture(scope="module")
def sched(host):
    return host.DynamicScheduler(0)


@pytest.fixture(scope="module")
def co():
    from oracle import c_oracle

    return c_oracle


def up(host, sched, t):
    return host.from_torch(sched, t.to(DEV))


def down(host, sched, handle):
    return host.to_torch(sched, handle).cpu()


# ---------------------------------------------------------------------------- GeLU
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("T", [128, 512, 1024])
def test_gelu_routine(host, sched, co, dtype, T):
    # test/test_gelu.cpp:59-102: B 2, d 512 (smaller here), randn input, randn grad_output
    x = randn((2, T, 256), 1, dtype=dtype)
    dy = randn((2, T, 256), 2, dtype=dtype)
    state = host.GeLU.init(sched)
    y = host.GeLU.forward(sched, state, up(host, sched, x))
    dx = host.GeLU.backward(sched, state, up(host, sched, dy))
    y.wait()
    assert_close(down(host, sched, y), co.gelu_forward(x), atol=1e-6, name="y")
    assert_close(down(host, sched, dx), co.gelu_backward(dy, x), atol=5e-6, name="dx")
    # the tanh form is an option the reference does not have
    state = host.GeLU.init(sched, approximate=1)
    y = host.GeLU.forward(sched, state, up(host, sched, x))
    assert_close(down(host, sched, y), co.gelu_forward(x, "tanh"), atol=1e-6, name="y tanh")


# ----------------------------------------------------------------------- Embedding
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_embedding_routine(host, sched, co, dtype):
    # test/test_embedding.cpp:58-97: B 2, T 1024, vocab 4095, d 512, int32 ids in [0, 3)
    B, T, V, d = 2, 1024, 4095, 512
    tdt = getattr(torch, dtype)
    ids = randint(0, 3, (B, T), 3, dtype=torch.int32)
    state = host.Embedding.init(sched, V, d, dtype=dtype)
    w = down(host, sched, state.weight)
    assert w.shape == (V, d) and w.dtype == tdt and abs(w.float().std().item() - 1) < 0.05  # N(0, 1) init
    out = host.Embedding.forward(sched, state, up(host, sched, ids))
    out.wait()
    got = down(host, sched, out)
    assert got.shape == (B, T, d)
    assert_bit_exact(got, co.embedding_forward(w, ids), "forward")
    dout = randn((B, T, d), 4, dtype=tdt)
    assert not state.grad_weight.defined()
    host.Embedding.backward(sched, state, up(host, sched, dout))
    want = co.embedding_backward(dout, ids, V)
    assert state.grad_weight.priority() == 1  # produced on the assist stream, as in the reference
    assert_close(down(host, sched, state.grad_weight), want, atol=2e-5 if dtype == "float32" else 1e-6, name="grad")
    # a second backward accumulates (`+=`), zero_grad drops the gradient
    host.Embedding.forward(sched, state, up(host, sched, ids))
    host.Embedding.backward(sched, state, up(host, sched, dout))
    assert_close(down(host, sched, state.grad_weight), co.embedding_backward(dout, ids, V, dweight=want),
                 atol=4e-5 if dtype == "float32" else 1e-6, name="grad +=")
    state.zero_grad()
    assert not state.grad_weight.defined()


@pytest.mark.gpu
def test_embedding_scale_grad_by_freq(host, sched, co):
    # Embedding::Options::scale_grad_by_freq reaches at::embedding_backward in the reference
    # (src/compute/embedding.cpp:147-157): a row's gradient is the mean over the entries that name it
    B, T, V, d = 2, 512, 300, 256
    ids = randint(0, 40, (B, T), 33, dtype=torch.int64)
    state = host.Embedding.init(sched, V, d, dtype="float32", scale_grad_by_freq=True)
    host.Embedding.forward(sched, state, up(host, sched, ids))
    dout = randn((B, T, d), 34)
    host.Embedding.backward(sched, state, up(host, sched, dout))
    want = co.embedding_backward(dout, ids, V, scale_grad_by_freq=True)
    assert_close(down(host, sched, state.grad_weight), want, atol=2e-6, name="scaled grad")
    host.Embedding.forward(sched, state, up(host, sched, ids))
    host.Embedding.backward(sched, state, up(host, sched, dout))
    assert_close(down(host, sched, state.grad_weight), 2 * want, atol=4e-6, name="scaled grad +=")


@pytest.mark.gpu
def test_embedding_inside_autocast_guard(host, sched, co):
    # test/test_autocast.cpp:158-204: fp32 table and fp32 upstream gradient, guard set to bf16;
    # a gather is not an autocast op, so output and gradient stay fp32
    B, T, V, d = 2, 1024, 4095, 512
    ids = randint(0, 3, (B, T), 30, dtype=torch.int32)
    state = host.Embedding.init(sched, V, d, dtype="float32")
    w = down(host, sched, state.weight)
    scope = host.autocast()
    scope.enter(sched, "bfloat16")
    try:
        out = host.Embedding.forward(sched, state, up(host, sched, ids))
        out.wait()
    finally:
        scope.exit()
    got = down(host, sched, out)
    assert got.dtype == torch.float32
    assert_bit_exact(got, co.embedding_forward(w, ids), "forward")
    dout = randn((B, T, d), 31)
    host.Embedding.backward(sched, state, up(host, sched, dout))
    grad = down(host, sched, state.grad_weight)
    assert grad.dtype == torch.float32
    assert_close(grad, co.embedding_backward(dout, ids, V), atol=2e-5, name="grad")


@pytest.mark.gpu
def test_embedding_with_positions(host, sched, co):
    B, T, V, C = 4, 64, 500, 128
    tok = host.Embedding.init(sched, V, C, dtype="bfloat16")
    pos = host.Embedding.init(sched, T, C, dtype="bfloat16")
    wte, wpe = down(host, sched, tok.weight), down(host, sched, pos.weight)
    ids = randint(0, V, (B, T), 5)
    out = host.Embedding.forward_with_positions(sched, tok, pos, up(host, sched, ids))
    assert_bit_exact(down(host, sched, out), co.embedding_forward_add(wte, wpe, ids), "gather-add")
    dout = randn((B, T, C), 6, dtype=torch.bfloat16)
    host.Embedding.backward_with_positions(sched, tok, pos, up(host, sched, dout))
    assert_close(down(host, sched, tok.grad_weight), co.embedding_backward(dout, ids, V), atol=1e-6, name="dwte")
    assert_close(down(host, sched, pos.grad_weight), co.embedding_backward_positions(dout), atol=1e-6, name="dwpe")


# ------------------------------------------------------------------- CrossEntropy
@pytest.mark.gpu
def test_cross_entropy_with_class_weights(host, sched, co):
    # state->forward.weight goes to nll_loss_forward / backward in the reference
    # (src/compute/cross_entropy.cpp:52-63,97-105)
    N, V = 512, 384
    x = randn((N, V), 40)
    t = randint(0, V, (N,), 41)
    t[::9] = -100
    w = torch.rand(V, generator=torch.Generator().manual_seed(42)) + 0.25
    state = host.CrossEntropy.init(sched)
    state.set_weight(up(host, sched, w))
    loss = host.CrossEntropy.forward(sched, state, up(host, sched, x), up(host, sched, t))
    dx = host.CrossEntropy.backward(sched, state)
    loss.wait()
    want_loss, _, want_dx, want_tw = co.cross_entropy(x, t, class_weight=w)
    assert_close(down(host, sched, loss).double(), want_loss.double(), atol=1e-5, name="weighted loss")
    assert_close(down(host, sched, dx), want_dx, atol=1e-9, name="weighted dx")



@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_cross_entropy_routine(host, sched, co, dtype):
    # test/test_cross_entropy.cpp:69-99: x = rand [B*256, 384] (B smaller here), int64 targets
    N, V = 8 * 256, 384
    x = torch.rand((N, V), generator=torch.Generator().manual_seed(1)).to(dtype)
    t = randint(0, V, (N,), 7)
    state = host.CrossEntropy.init(sched)
    loss = host.CrossEntropy.forward(sched, state, up(host, sched, x), up(host, sched, t))
    dx = host.CrossEntropy.backward(sched, state)
    loss.wait()
    want_loss, _, want_dx, _ = co.cross_entropy(x, t)
    assert_close(down(host, sched, loss).double(), want_loss.double(), atol=1e-5, name="loss")
    assert_close(down(host, sched, dx), want_dx, atol=1e-9, name="dx")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_cross_entropy_amp(host, sched, co, dtype):
    # test/test_cross_entropy.cpp:102-139: 16-bit logits inside the autocast guard, fp32 gradient
    N, V = 1024, 384
    x = torch.rand((N, V), generator=torch.Generator().manual_seed(1)).to(getattr(torch, dtype))
    t = randint(0, V, (N,), 8)
    scope = host.autocast()
    scope.enter(sched, dtype)
    try:
        state = host.CrossEntropy.init(sched)
        loss = host.CrossEntropy.forward(sched, state, up(host, sched, x), up(host, sched, t))
        dx = host.CrossEntropy.backward(sched, state)
    finally:
        scope.exit()
    got = down(host, sched, dx)
    assert got.dtype == torch.float32
    want_loss, _, want_dx, _ = co.cross_entropy(x, t, dlogits_dtype=torch.float32)
    assert_close(down(host, sched, loss), want_loss, atol=1e-5, name="loss")
    assert_close(got, want_dx, atol=1e-9, name="dx fp32")
    # outside the guard the gradient keeps the logits' dtype; padded vocabulary via num_classes
    state = host.CrossEntropy.init(sched, num_classes=300)
    loss16 = host.CrossEntropy.forward(sched, state, up(host, sched, x), up(host, sched, t % 300))
    got = down(host, sched, host.CrossEntropy.backward(sched, state))
    assert got.dtype == x.dtype and (got[:, 300:] == 0).all()
    # ... and so does the loss, as nll_loss_forward's does (cross_entropy.cpp:57-66)
    loss16 = down(host, sched, loss16)
    want16, _, _, _ = co.cross_entropy(x[:, :300], t % 300)
    assert loss16.dtype == x.dtype
    assert loss16 == want16.to(x.dtype) or abs(float(loss16) - float(want16)) <= 2.0 ** -7 * float(want16)


@pytest.mark.gpu
def test_host_reads_see_finished_main_lane_work(host, sched):
    # Main-lane tasks share an event that is recorded only when somebody asks for it.  The asking
    # is what is tested here: the host reads the output of a long task the moment it is submitted,
    # with more main-lane work queued behind it, then an assist-lane task (the optimizer) consumes a
    # main-lane result, and a main-lane task consumes what the optimizer wrote.
    from core_scheduler_amd import ops

    n = 1 << 25  # 32M elements: ~100 us of kernel time, far longer than the submission
    state = host.GeLU.init(sched, 1)
    for seed in (1, 2, 3):
        x = randn((n,), seed, dtype=torch.bfloat16).to(DEV)
        y = host.GeLU.forward(sched, state, host.from_torch(sched, x))
        later = [host.GeLU.forward(sched, state, y) for _ in range(3)]  # queued behind it
        assert_bit_exact(host.to_torch(sched, y).cpu(), ops.gelu_forward(x, approximate="tanh").cpu(), f"y[{seed}]")
        assert later[2].defined()
    # main -> assist -> main
    w0 = torch.zeros(n // 8, device=DEV)
    g_src = randn((n // 8,), 9).to(DEV)
    w = host.from_torch(sched, w0.clone())
    opt = host.AdamW.init(sched, w, lr=1.0, beta1=0.0, beta2=0.0, eps=1.0, weight_decay=0.0, t=0)
    gel = host.GeLU.init(sched, 1)
    grad = host.GeLU.forward(sched, gel, host.from_torch(sched, g_src))   # main lane
    host.AdamW.step(sched, opt, w, grad)                                  # assist lane, reads grad
    out = host.GeLU.forward(sched, gel, w)                                # main lane, reads the updated w
    gref = ops.gelu_forward(g_src, approximate="tanh")
    wref = w0 - gref / (gref.abs() + 1.0)  # beta1 = beta2 = 0, eps = 1, lr = 1: w -= g / (|g| + 1)
    assert_close(host.to_torch(sched, w).cpu(), wref.cpu(), atol=1e-6, name="w after the step")
    assert_close(host.to_torch(sched, out).cpu(), ops.gelu_forward(wref, approximate="tanh").cpu(), atol=1e-6,
                 name="main-lane task after the step")


# ---------------------------------------------------------------------- LayerNorm
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_layer_norm_routine(host, sched, co, dtype):
    # test/test_layer_norm.cpp:63-134: x = rand [.., 384], weight 1, bias 0
    tdt = getattr(torch, dtype)
    x = torch.rand((16, 64, 384), generator=torch.Generator().manual_seed(1)).to(tdt)
    dy = torch.rand((16, 64, 384), generator=torch.Generator().manual_seed(2)).to(tdt)
    state = host.LayerNorm.init(sched, [384], dtype=dtype)
    assert list(state.parameter_names()) == ["weight", "bias"]
    w, b = down(host, sched, state.weight), down(host, sched, state.bias)
    assert (w == 1).all() and (b == 0).all()
    y = host.LayerNorm.forward(sched, state, up(host, sched, x))
    dx = host.LayerNorm.backward(sched, state, up(host, sched, dy))
    y2, mean, rstd = co.layernorm_forward(x.reshape(-1, 384), w, b)
    dx2, dg2, db2 = co.layernorm_backward(dy.reshape(-1, 384), x.reshape(-1, 384), mean, rstd, w)
    tight = dtype == "float64"
    assert_close(down(host, sched, y).reshape(-1, 384), y2, atol=1e-13 if tight else 2e-6, name="y")
    assert_close(down(host, sched, dx).reshape(-1, 384), dx2, atol=1e-13 if tight else 5e-6, name="dx")
    # column sums of 1024 terms of size ~0.5: fp32 rounding of the running sum allows about
    # 2 * 6e-8 * (sum of the terms' magnitudes) = 1e-4 in absolute terms
    assert_close(down(host, sched, state.grad_weight), dg2, atol=1e-10 if tight else 1e-4, name="dgamma")
    assert_close(down(host, sched, state.grad_bias), db2, atol=1e-10 if tight else 1e-4, name="dbeta")
    # second backward accumulates into the existing gradients (src/compute/layer_norm.cpp:325-334)
    host.LayerNorm.forward(sched, state, up(host, sched, x))
    host.LayerNorm.backward(sched, state, up(host, sched, dy))
    assert_close(down(host, sched, state.grad_bias), 2 * db2, atol=1e-9 if tight else 2e-4, name="dbeta +=")
    state.zero_grad()
    assert not state.grad_weight.defined() and not state.grad_bias.defined()


@pytest.mark.gpu
def test_layer_norm_autocast_and_no_bias(host, sched, co):
    # test/test_autocast.cpp:112-156: bf16 x inside the guard, fp32 parameters, fp32 y and dy
    x = randn((8, 64, 768), 9, dtype=torch.bfloat16)
    dy = randn((8, 64, 768), 10)
    state = host.LayerNorm.init(sched, [768], dtype="float32")
    gamma, beta = randn(768, 11, std=0.02, mean=1.0), randn(768, 12, std=0.02)
    state.set_weight(up(host, sched, gamma))
    state.set_bias(up(host, sched, beta))
    scope = host.autocast()
    scope.enter(sched, "bfloat16")
    try:
        y = host.LayerNorm.forward(sched, state, up(host, sched, x))
        dx = host.LayerNorm.backward(sched, state, up(host, sched, dy))
    finally:
        scope.exit()
    got_y = down(host, sched, y)
    assert got_y.dtype == torch.float32
    y2, mean, rstd = co.layernorm_forward(x.reshape(-1, 768), gamma, beta, out_dtype=torch.float32)
    dx2, dg2, db2 = co.layernorm_backward(dy.reshape(-1, 768), x.reshape(-1, 768), mean, rstd, gamma,
                                          out_dtype=torch.float32)
    assert_close(got_y.reshape(-1, 768), y2, atol=2e-6, name="y fp32")
    assert_close(down(host, sched, dx).reshape(-1, 768), dx2, atol=5e-6, name="dx fp32")
    assert_close(down(host, sched, state.grad_weight), dg2, atol=1e-4, name="dgamma")  # 512 terms of size ~1
    assert_close(down(host, sched, state.grad_bias), db2, atol=1e-4, name="dbeta")
    # bias=false path (src/compute/layer_norm.cpp:198-204)
    nb = host.LayerNorm.init(sched, [768], bias=False, dtype="float32")
    assert list(nb.parameter_names()) == ["weight"]
    xs = randn((32, 768), 13)
    y = host.LayerNorm.forward(sched, nb, up(host, sched, xs))
    assert_close(down(host, sched, y), co.layernorm_forward(xs, torch.ones(768), None)[0], atol=2e-6, name="no bias")
    host.LayerNorm.backward(sched, nb, up(host, sched, xs))
    assert nb.grad_weight.defined() and not nb.grad_bias.defined()


@pytest.mark.gpu
def test_layer_norm_backward_sums_ride_in_the_next_backward(host, sched):
    # a step's backward pass: one LayerNorm backward per norm, back to back on the main stream, with
    # other tasks between them.  Each call leaves its column sums to the next call's launch; the
    # gradients must hold the bits of the one-call kernel path whenever and however they are read.
    from core_scheduler_amd import ops

    widths = [768, 768, 1600, 768, 768]  # the width change makes one record settle on its own
    rows = 2048
    states, xs, dys, dxs = [], [], [], []
    for i, C in enumerate(widths):
        st = host.LayerNorm.init(sched, [C], bias=(i != 3), dtype="float32")
        st.set_weight(up(host, sched, randn(C, 100 + i, std=0.02, mean=1.0)))
        if i != 3:
            st.set_bias(up(host, sched, randn(C, 120 + i, std=0.02)))
        states.append(st)
        xs.append(randn((rows, C), 140 + i, dtype=torch.bfloat16))
        dys.append(randn((rows, C), 160 + i, dtype=torch.bfloat16))

    def want(i, times=1):
        x, dy = xs[i].to(DEV), dys[i].to(DEV)
        gamma = down(host, sched, states[i].weight).to(DEV)
        beta = torch.zeros_like(gamma)
        _, mean, rstd = ops.layernorm_forward(x, gamma, beta)
        dx, dg, db = ops.layernorm_backward(dy, x, mean, rstd, gamma)
        for _ in range(times - 1):
            ops.layernorm_backward(dy, x, mean, rstd, gamma, dgamma=dg, dbeta=db)
        return dx.cpu(), dg.cpu(), db.cpu()

    def backward_all():
        out = []
        for i, st in enumerate(states):
            host.LayerNorm.forward(sched, st, up(host, sched, xs[i]))
        gelu = host.GeLU.init(sched)
        for i, st in enumerate(states):
            out.append(host.LayerNorm.backward(sched, st, up(host, sched, dys[i])))
            host.GeLU.forward(sched, gelu, out[-1])  # an unrelated task between two norms
        return out

    dxs = backward_all()
    # read in an order that is not the order of the launches; the last norm's sums had no successor
    for i in (4, 0, 2, 1, 3):
        dx2, dg2, db2 = want(i)
        assert_bit_exact(down(host, sched, states[i].grad_weight), dg2, f"dgamma[{i}]")
        if i != 3:
            assert_bit_exact(down(host, sched, states[i].grad_bias), db2, f"dbeta[{i}]")
        assert_bit_exact(down(host, sched, dxs[i]), dx2, f"dx[{i}]")
    # a second pass adds to the gradients that exist (micro-batches), again through the chain
    backward_all()
    for i in (1, 2, 4):
        _, dg2, db2 = want(i, times=2)
        assert_bit_exact(down(host, sched, states[i].grad_weight), dg2, f"dgamma[{i}] +=")
        assert_bit_exact(down(host, sched, states[i].grad_bias), db2, f"dbeta[{i}] +=")
    # a task that takes the gradient as its input gets the finished sums without any host read
    for st in states:
        st.zero_grad()
    backward_all()
    w = up(host, sched, torch.zeros(768))
    opt = host.AdamW.init(sched, w, lr=1.0, beta1=0.0, beta2=0.0, eps=1.0, weight_decay=0.0, t=0)
    host.AdamW.step(sched, opt, w, states[4].grad_weight)  # m = g with beta1 = 0
    assert_bit_exact(down(host, sched, opt.m), want(4)[1], "gradient seen by the optimizer task")
    # gradients nobody reads are dropped with their sums still outstanding
    for st in states:
        st.zero_grad()
    backward_all()
    for st in states:
        st.zero_grad()
    assert_bit_exact(down(host, sched, backward_all()[0]), want(0)[0], "dx after dropped gradients")


@pytest.mark.gpu
@pytest.mark.parametrize("C,rows", [(768, 1024), (1600, 512), (250, 33)])
def test_layer_norm_with_the_residual_stream(host, sched, C, rows):
    # example/gpt2/gpt2_single_device.cpp:459-460 (res1 = add(x, attn_out); ln2->forward(res1)) and
    # :468-469 (dx_ln2 = ln2->backward(dx_mlp); dx_res1 = add(dx_ln2, dx)) as one task each way:
    # the bits of the separate add and norm tasks
    x = randn((rows, C), 300, dtype=torch.bfloat16)
    res = randn((rows, C), 301, dtype=torch.bfloat16)
    dy = randn((rows, C), 302, dtype=torch.bfloat16)
    dres = randn((rows, C), 303, dtype=torch.bfloat16)
    gamma, beta = randn(C, 304, std=0.02, mean=1.0), randn(C, 305, std=0.02)

    def state():
        st = host.LayerNorm.init(sched, [C], dtype="float32")
        st.set_weight(up(host, sched, gamma))
        st.set_bias(up(host, sched, beta))
        return st

    fused, plain = state(), state()
    y, new_res = host.LayerNorm.forward_with_residual(sched, fused, up(host, sched, x), up(host, sched, res))
    total = (x.to(DEV) + res.to(DEV))  # one rounding to bf16, as the kernel does
    y2 = host.LayerNorm.forward(sched, plain, host.from_torch(sched, total))
    assert_bit_exact(down(host, sched, new_res), total.cpu(), "x + residual")
    assert_bit_exact(down(host, sched, y), down(host, sched, y2), "y")
    dx = host.LayerNorm.backward_with_residual(sched, fused, up(host, sched, dy), up(host, sched, dres))
    dx2 = host.LayerNorm.backward(sched, plain, up(host, sched, dy))
    # dx + dresidual in fp32, rounded once (the separate tasks round dx first: up to one bf16 ulp apart)
    from core_scheduler_amd import ops

    _, mean, rstd = ops.layernorm_forward(total, gamma.to(DEV), beta.to(DEV))
    want, _, _ = ops.layernorm_backward(dy.to(DEV), total, mean, rstd, gamma.to(DEV), dresidual=dres.to(DEV))
    assert_bit_exact(down(host, sched, dx), want.cpu(), "dx + dresidual")
    two_tasks = down(host, sched, dx2).float() + dres.float()
    assert_close(down(host, sched, dx).float(), two_tasks, atol=0.04, name="against the two tasks")  # bf16 ulp at |v| ~ 4
    assert_bit_exact(down(host, sched, fused.grad_weight), down(host, sched, plain.grad_weight), "dgamma")
    assert_bit_exact(down(host, sched, fused.grad_bias), down(host, sched, plain.grad_bias), "dbeta")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_layer_norm_autocast_with_16_bit_parameters(host, sched, co, dtype):
    # a model whose LayerNorm parameters are 16 bit, run inside the autocast guard: fp32 y, fp32 dy and dx,
    # parameter gradients in the parameters' type, twice (the second backward adds to the first)
    td = getattr(torch, dtype)
    x = randn((4, 32, 768), 21, dtype=td)
    dy = randn((4, 32, 768), 22)
    state = host.LayerNorm.init(sched, [768], dtype=dtype)
    gamma, beta = randn(768, 23, std=0.02, mean=1.0, dtype=td), randn(768, 24, std=0.02, dtype=td)
    state.set_weight(up(host, sched, gamma))
    state.set_bias(up(host, sched, beta))
    scope = host.autocast()
    scope.enter(sched, dtype)
    try:
        y = host.LayerNorm.forward(sched, state, up(host, sched, x))
        dx = host.LayerNorm.backward(sched, state, up(host, sched, dy))
        host.LayerNorm.forward(sched, state, up(host, sched, x))
        host.LayerNorm.backward(sched, state, up(host, sched, dy))
    finally:
        scope.exit()
    x2, g2, b2 = x.reshape(-1, 768), gamma.float(), beta.float()
    y2, mean, rstd = co.layernorm_forward(x2, g2, b2, out_dtype=torch.float32)
    dx2, dg2, db2 = co.layernorm_backward(dy.reshape(-1, 768), x2, mean, rstd, g2, out_dtype=torch.float32)
    assert_close(down(host, sched, y).reshape(-1, 768), y2, atol=2e-6, name="y fp32")
    assert_close(down(host, sched, dx).reshape(-1, 768), dx2, atol=5e-6, name="dx fp32")
    got_dg, got_db = down(host, sched, state.grad_weight), down(host, sched, state.grad_bias)
    assert got_dg.dtype == td and got_db.dtype == td
    # each backward's gradient is rounded to 16 bit, then the two are added and rounded again
    want_dg = (dg2.to(td).float() * 2).to(td)
    want_db = (db2.to(td).float() * 2).to(td)
    assert_close(got_dg, want_dg, atol=1e-4, name="dgamma, two backward passes")
    assert_close(got_db, want_db, atol=1e-4, name="dbeta, two backward passes")


@pytest.mark.gpu
def test_tensor_handles_print_like_at_print(host, sched):
    # include/tensor.h:65-70: print waits for the tensor and hands it to at::print
    t = up(host, sched, torch.tensor([[1.0, 2.5, -3.0], [4.0, 0.0, 6.0]]))
    text = host.tensor_to_string(t)
    assert "2.5" in text and "-3" in text and "{2,3}" in text, text


# -------------------------------------------------------------------------- AdamW
@pytest.mark.gpu
@pytest.mark.parametrize("size", [128, 512, 1024])
def test_adamw_functional_routine(host, sched, size):
    # test/test_adamw.cpp:63-103, with the closed form and the tolerances written there
    lr, b1, b2, eps, wd = 1.0, 0.9, 0.999, 1e-8, 1e-2
    x0 = torch.rand(size, generator=torch.Generator().manual_seed(1))
    dx = torch.rand(size, generator=torch.Generator().manual_seed(2))
    x = up(host, sched, x0)
    state = host.AdamW.init(sched, x, lr=lr, beta1=b1, beta2=b2, eps=eps, weight_decay=wd, t=0)
    host.AdamW.step(sched, state, x, up(host, sched, dx))
    assert state.t == 1
    xt = x0 - lr * wd * x0
    mt = (1 - b1) * dx
    vt = (1 - b2) * dx.square()
    xt = xt - lr * (mt / (1 - b1)) / ((vt / (1 - b2)).sqrt() + eps)
    assert torch.allclose(down(host, sched, x), xt, 1e-4, 1e-5)
    assert torch.allclose(down(host, sched, state.m), mt, 1e-4, 1e-5)
    assert torch.allclose(down(host, sched, state.v), vt, 1e-4, 1e-5)


@pytest.mark.gpu
def test_adamw_all_parameters_in_one_task(host, sched, co):
    # the loop of src/module/adamw.cpp:32-38 as one launch; compared with per-tensor steps and the oracle
    hp = dict(lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    shapes = [(300, 64), (64,), (5000,), (17, 3)]
    ws0 = [randn(s, 20 + i, std=0.02) for i, s in enumerate(shapes)]
    gs = [randn(s, 40 + i, std=1e-3) for i, s in enumerate(shapes)]
    ws = [up(host, sched, w) for w in ws0]
    states = [host.AdamW.init(sched, w, **hp) for w in ws]
    for _ in range(3):
        host.AdamW.step_all(sched, states, ws, [up(host, sched, g) for g in gs])
    states[0].set_lr(1e-3)
    assert states[0].get_lr() == 1e-3
    for i, s in enumerate(shapes):
        w, m, v = ws0[i], torch.zeros(s), torch.zeros(s)
        for t in range(1, 4):
            w, m, v, _ = co.adamw_step(w, gs[i], m, v, t=t, **hp)
        assert_close(down(host, sched, ws[i]), w.reshape(s), atol=1e-8, name=f"w[{i}]")
        assert_close(down(host, sched, states[i].v), v.reshape(s), atol=1e-13, name=f"v[{i}]")
    # an undefined gradient is skipped with a warning and leaves the parameter alone
    before = down(host, sched, ws[1])
    host.AdamW.step(sched, states[1], ws[1], host.Tensor())
    assert_bit_exact(down(host, sched, ws[1]), before, "skipped update")


@pytest.mark.gpu
def test_adamw_descriptor_tables_are_reused_only_when_identical(host, sched, co):
    # the optimizer task keeps its last few descriptor tables on the device and skips the copy when
    # a new table matches one byte for byte; ten different parameter sets stepped in turn (more than
    # are kept) and the first set again must each get their own update
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    sets = []
    for k in range(10):
        w0 = [randn((64 + k, 8), 900 + k, std=0.02), randn((33,), 920 + k, std=0.02)]
        g = [randn((64 + k, 8), 940 + k, std=1e-2), randn((33,), 960 + k, std=1e-2)]
        ws = [up(host, sched, w) for w in w0]
        gs = [up(host, sched, x) for x in g]
        sets.append((w0, g, ws, gs, [host.AdamW.init(sched, w, **hp) for w in ws]))
    for rnd in range(3):
        for w0, g, ws, gs, states in sets:
            host.AdamW.step_all(sched, states, ws, gs)
    for w0, g, ws, gs, states in sets:
        for i in range(2):
            w, m, v = w0[i], torch.zeros_like(w0[i]), torch.zeros_like(w0[i])
            for t in range(1, 4):
                w, m, v, _ = co.adamw_step(w, g[i], m, v, t=t, **hp)
            assert_close(down(host, sched, ws[i]), w.reshape(w0[i].shape), atol=1e-8, name="w")


# ------------------------------------------------------------------- module layer
def build_tree(host, sched, V=211, T=16, C=64):
    """A GPT-2-shaped tree: wte, wpe, h.0.ln_1, h.0.ln_2, ln_f (what the ops here cover)."""
    root = host.Container()
    wte = root.register_module("wte", host.EmbeddingModule(sched, V, C))
    wpe = root.register_module("wpe", host.EmbeddingModule(sched, T, C))
    h = root.register_module("h", host.Container())
    block = h.register_module("0", host.Container())
    ln1 = block.register_module("ln_1", host.LayerNormModule(sched, [C]))
    ln2 = block.register_module("ln_2", host.LayerNormModule(sched, [C], bias=False))
    lnf = root.register_module("ln_f", host.LayerNormModule(sched, [C]))
    return root, dict(wte=wte, wpe=wpe, ln1=ln1, ln2=ln2, lnf=lnf)


@pytest.mark.gpu
def test_module_tree_names_and_zero_grad(host, sched):
    # src/module/module.cpp:33-120: depth-first order, names joined with '.', state name appended
    root, mods = build_tree(host, sched)
    assert root.named_states() == ["wte", "wpe", "h.0.ln_1", "h.0.ln_2", "ln_f"]
    names = [k for k, _ in root.named_parameters()]
    assert names == ["wte.weight", "wpe.weight", "h.0.ln_1.weight", "h.0.ln_1.bias", "h.0.ln_2.weight",
                     "ln_f.weight", "ln_f.bias"]
    assert [k for k, _ in root.named_gradients()] == names
    assert all(not g.defined() for _, g in root.named_gradients())  # nothing has run backward yet
    B, T, C = 2, 16, 64
    ids = randint(0, 211, (B, T), 5, dtype=torch.int64)
    x = mods["wte"].forward(sched, up(host, sched, ids))
    y = mods["ln1"].forward(sched, x)
    dy = up(host, sched, randn((B, T, C), 6))
    dx = mods["ln1"].backward(sched, dy)
    mods["wte"].backward(sched, dx)
    grads = dict(root.named_gradients())
    for k in ("wte.weight", "h.0.ln_1.weight", "h.0.ln_1.bias"):
        grads[k].wait()
        assert grads[k].defined(), k
    assert not grads["ln_f.weight"].defined()
    root.zero_grad()  # set to undefined, as the reference does (src/compute/embedding.cpp:54)
    assert all(not g.defined() for _, g in root.named_gradients())
    root.to("bfloat16")
    assert all(down(host, sched, p).dtype == torch.bfloat16 for _, p in root.named_parameters())


@pytest.mark.gpu
def test_adamw_module_matches_torch_optimizer(host, sched):
    # test/test_adamw.cpp:105-190 checks cs::module::AdamW against torch::optim::AdamW on the same
    # parameters and gradients with tolerance (1e-4, 1e-5); here over a tree and three steps.
    # (amsgrad is left out: the reference keeps the maximum of the bias-corrected second moment,
    # src/optimizer/adamw.cu:80-82, torch.optim the maximum of the raw one.)
    amsgrad = False
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    root, mods = build_tree(host, sched)
    opt = host.AdamWModule(sched, root, amsgrad=amsgrad, **hp)
    names = [k for k, _ in root.named_parameters()]
    assert [k for k, _ in opt.named_states()] == names
    ref_params = {k: torch.nn.Parameter(down(host, sched, p).clone()) for k, p in root.named_parameters()}
    ref = torch.optim.AdamW(ref_params.values(), lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                            weight_decay=hp["weight_decay"], amsgrad=amsgrad, foreach=False)
    B, T, C = 2, 16, 64
    for step in range(3):
        ids = randint(0, 211, (B, T), 50 + step, dtype=torch.int64)
        x = mods["wte"].forward(sched, up(host, sched, ids))
        y = mods["ln1"].forward(sched, x)
        z = mods["lnf"].forward(sched, y)
        dz = up(host, sched, randn((B, T, C), 60 + step))
        dy = mods["lnf"].backward(sched, dz)
        dx = mods["ln1"].backward(sched, dy)
        mods["wte"].backward(sched, dx)
        grads = dict(root.named_gradients())
        for k, p in ref_params.items():  # wpe and h.0.ln_2 were not used: no gradient, no update
            p.grad = down(host, sched, grads[k]).clone() if k in ("wte.weight", "h.0.ln_1.weight", "h.0.ln_1.bias",
                                                                 "ln_f.weight", "ln_f.bias") else None
        opt.step(sched)
        ref.step()
        opt.zero_grad(sched)
    for k, p in root.named_parameters():
        got = down(host, sched, p)
        assert torch.allclose(got, ref_params[k].detach(), 1e-4, 1e-5), k
    states = dict(opt.named_states())
    assert all(s.t == 3 for s in states.values())
    assert torch.allclose(down(host, sched, states["wte.weight"].m), ref.state[ref_params["wte.weight"]]["exp_avg"],
                          1e-4, 1e-6)
    assert torch.allclose(down(host, sched, states["ln_f.bias"].v), ref.state[ref_params["ln_f.bias"]]["exp_avg_sq"],
                          1e-4, 1e-9)
    opt.set_lr(5e-3)
    assert opt.get_lr() == 5e-3 and all(s.get_lr() == 5e-3 for s in states.values())


@pytest.mark.gpu
def test_training_chain_matches_torch_autograd(host, sched):
    """Every op of the path in one chain, gradients flowing from the loss to the tables, five
    optimizer steps: token + position gather -> LayerNorm -> GeLU (tanh) -> LayerNorm -> cross
    entropy over the C columns, AdamW with weight decay.  The same model in torch (float64 on the
    CPU, autograd, torch.optim.AdamW) from the same parameters has to show the same loss at every
    step and end at the same parameters, which pins what the per-op tests cannot: that each
    backward consumes exactly the gradient the next op produces and that the optimizer sees it."""
    B, T, C, V = 4, 32, 128, 300
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    root, mods = build_tree(host, sched, V=V, T=T, C=C)
    opt = host.AdamWModule(sched, root, **hp)
    gelu = host.GeLU.init(sched, 1)
    used = ["wte.weight", "wpe.weight", "h.0.ln_1.weight", "h.0.ln_1.bias", "ln_f.weight", "ln_f.bias"]
    ref = {k: torch.nn.Parameter(down(host, sched, p).double()) for k, p in root.named_parameters() if k in used}
    ref_opt = torch.optim.AdamW(ref.values(), lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                                weight_decay=hp["weight_decay"], foreach=False)
    tok, pos = mods["wte"].state(), mods["wpe"].state()
    losses, ref_losses = [], []

    def reshaped(handle, *shape):  # a view of the same device memory under a new handle
        return host.from_torch(sched, host.to_torch(sched, handle).view(*shape))

    for step in range(5):
        ids = randint(0, V, (B, T), 700)  # the same batch every step, so the loss has to fall
        targets = randint(0, C, (B * T,), 720)
        x = host.Embedding.forward_with_positions(sched, tok, pos, up(host, sched, ids))
        h1 = mods["ln1"].forward(sched, x)
        a = host.GeLU.forward(sched, gelu, h1)
        h2 = mods["lnf"].forward(sched, a)
        ce = host.CrossEntropy.init(sched)
        loss = host.CrossEntropy.forward(sched, ce, reshaped(h2, B * T, C), up(host, sched, targets))
        dlogits = host.CrossEntropy.backward(sched, ce)
        da = mods["lnf"].backward(sched, reshaped(dlogits, B, T, C))
        dh1 = host.GeLU.backward(sched, gelu, da)
        dx = mods["ln1"].backward(sched, dh1)
        host.Embedding.backward_with_positions(sched, tok, pos, dx)
        opt.step(sched)
        opt.zero_grad(sched)
        losses.append(float(down(host, sched, loss)))
        # the same step in torch
        ref_opt.zero_grad()
        rx = ref["wte.weight"][ids] + ref["wpe.weight"][None, :T]
        r1 = torch.nn.functional.layer_norm(rx, (C,), ref["h.0.ln_1.weight"], ref["h.0.ln_1.bias"], 1e-5)
        ra = torch.nn.functional.gelu(r1, approximate="tanh")
        r2 = torch.nn.functional.layer_norm(ra, (C,), ref["ln_f.weight"], ref["ln_f.bias"], 1e-5)
        rl = torch.nn.functional.cross_entropy(r2.reshape(B * T, C), targets)
        rl.backward()
        ref_opt.step()
        ref_losses.append(float(rl.detach()))
    for i, (a, b) in enumerate(zip(losses, ref_losses)):
        assert abs(a - b) <= 2e-5 * abs(b), f"loss at step {i}: {a} vs {b}"
    assert ref_losses[-1] < ref_losses[0]  # the model learns, so the gradients mattered
    for k, p in root.named_parameters():
        if k in used:
            got = down(host, sched, p).double()
            assert torch.allclose(got, ref[k].detach(), rtol=2e-4, atol=2e-5), f"{k}: {(got - ref[k]).abs().max()}"


@pytest.mark.gpu
def test_steps_without_host_waits_match_steps_with_waits(host, sched):
    """The scheduler's stream rules are what keeps a step correct when nothing waits on the host:
    gradients are produced on the assist stream (embedding backward) and on the main stream, the
    optimizer reads both, zero_grad drops them, the next step starts at once.  Every kernel is
    deterministic, so ten steps submitted back to back must give, bit for bit, the parameters of
    the same ten steps with a host wait after every task."""
    B, T, C, V = 4, 64, 256, 2000
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    first = None
    results = []
    for waits in (True, False, False):
        root, mods = build_tree(host, sched, V=V, T=T, C=C)
        if first is None:
            first = {k: down(host, sched, p).clone() for k, p in root.named_parameters()}
        for k, p in root.named_parameters():  # the same start for every run
            host.assign_(sched, p, first[k].to(DEV))
        opt = host.AdamWModule(sched, root, max_grad_norm=1.0, **hp)
        gelu = host.GeLU.init(sched, 1)

        def settle(*handles):
            if waits:
                for h in handles:
                    h.wait()

        # inputs are on the device before the first step, so no copy interrupts the submissions
        inputs = [(randint(0, V, (B, T), 900 + step).to(DEV), randn((B, T, C), 950 + step).to(DEV)) for step in range(10)]
        torch.cuda.synchronize()
        for step in range(10):
            ids = host.from_torch(sched, inputs[step][0])
            x = mods["wte"].forward(sched, ids); settle(x)
            y = mods["ln1"].forward(sched, x); settle(y)
            a = host.GeLU.forward(sched, gelu, y); settle(a)
            z = mods["lnf"].forward(sched, a); settle(z)
            dz = host.from_torch(sched, inputs[step][1])  # upstream gradient of the step
            da = mods["lnf"].backward(sched, dz); settle(da)
            dy = host.GeLU.backward(sched, gelu, da); settle(dy)
            dx = mods["ln1"].backward(sched, dy); settle(dx)
            mods["wte"].backward(sched, dx)
            opt.step(sched)
            opt.zero_grad(sched)
            if waits:
                for _, p in root.named_parameters():
                    p.wait()
        results.append({k: down(host, sched, p) for k, p in root.named_parameters()})
    for k in results[0]:
        assert_bit_exact(results[1][k], results[0][k], f"{k}: no waits vs waits")
        assert_bit_exact(results[2][k], results[0][k], f"{k}: no waits, again")
    assert not torch.equal(results[0]["wte.weight"], first["wte.weight"])  # the steps did something


@pytest.mark.gpu
def test_clip_grad_norm_task_and_clipped_optimizer(host, sched, co):
    # Utils::clip_grad_norm_ (src/compute/utils.cpp:700-746) against torch.nn.utils.clip_grad_norm_,
    # then the module optimizer with max_grad_norm against clip + torch.optim.AdamW
    shapes = [(300, 64), (64,), (5000,), (17, 3)]
    gs = [randn(s, 70 + i, std=0.1) for i, s in enumerate(shapes)]
    handles = [up(host, sched, g.clone()) for g in gs]
    norm = host.clip_grad_norm_(sched, handles, 0.5, 2.0)
    ps = [torch.nn.Parameter(torch.zeros(s)) for s in shapes]
    for p, g in zip(ps, gs):
        p.grad = g.clone()
    want = torch.nn.utils.clip_grad_norm_(ps, 0.5, foreach=False)
    assert abs(down(host, sched, norm).item() - want.item()) <= 1e-5 * want.item()
    for h, p in zip(handles, ps):
        assert torch.allclose(down(host, sched, h), p.grad, rtol=1e-5, atol=1e-9)

    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    root, mods = build_tree(host, sched)
    opt = host.AdamWModule(sched, root, max_grad_norm=0.05, **hp)
    assert not opt.last_grad_norm().defined()
    ref_params = {k: torch.nn.Parameter(down(host, sched, p).clone()) for k, p in root.named_parameters()}
    ref = torch.optim.AdamW(ref_params.values(), lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                            weight_decay=hp["weight_decay"], foreach=False)
    B, T, C = 2, 16, 64
    used = ("wte.weight", "h.0.ln_1.weight", "h.0.ln_1.bias")
    for step in range(2):
        ids = randint(0, 211, (B, T), 80 + step, dtype=torch.int64)
        y = mods["ln1"].forward(sched, mods["wte"].forward(sched, up(host, sched, ids)))
        dx = mods["ln1"].backward(sched, up(host, sched, randn((B, T, C), 90 + step)))
        mods["wte"].backward(sched, dx)
        grads = dict(root.named_gradients())
        for k, p in ref_params.items():
            p.grad = down(host, sched, grads[k]).clone() if k in used else None
        before = {k: down(host, sched, grads[k]).clone() for k in used}
        opt.step(sched)
        want = torch.nn.utils.clip_grad_norm_([ref_params[k] for k in used], 0.05, foreach=False)
        ref.step()
        got = down(host, sched, opt.last_grad_norm()).item()
        assert got > 0.05 and abs(got - want.item()) <= 1e-5 * want.item()
        for k in used:  # the fused step leaves the gradients as they were
            assert_bit_exact(down(host, sched, grads[k]), before[k], k)
        opt.zero_grad(sched)
    for k, p in root.named_parameters():
        assert torch.allclose(down(host, sched, p), ref_params[k].detach(), 1e-4, 1e-5), k


# ------------------------------------------------------ error conventions (no GPU)
def run_snippet(code):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-c", textwrap.dedent(code)], capture_output=True, text=True, env=env,
                          timeout=120)


def test_label_smoothing_aborts_like_the_reference():
    # src/compute/cross_entropy.cpp:30-31: CS_ASSERT_TRUE -> log critical + std::abort
    p = run_snippet("""
        from core_scheduler_amd import _cs_host as h
        h.CrossEntropy.init(h.Scheduler(), 1, -100, 0.1, -1)
    """)
    assert p.returncode != 0 and "label_smoothing" in (p.stderr + p.stdout)


def test_embedding_argument_checks_raise():
    # src/compute/embedding.cpp:80-92: TORCH_CHECK on padding_idx and max_norm
    p = run_snippet("""
        from core_scheduler_amd import _cs_host as h
        s = h.Scheduler()
        for kwargs in (dict(padding_idx=10), dict(padding_idx=-11), dict(max_norm=1.0)):
            try:
                h.Embedding.init(s, 10, 4, **kwargs)
            except RuntimeError as e:
                print("raised:", str(e).splitlines()[0])
    """)
    assert p.stdout.count("raised:") == 3, p.stdout + p.stderr


def test_layer_norm_without_affine_parameters_aborts_like_the_reference():
    # src/compute/layer_norm.cpp:78-79: CS_ASSERT_TRUE(elementwise_affine) -> log critical + std::abort
    p = run_snippet("""
        from core_scheduler_amd import _cs_host as h
        h.LayerNorm.init(h.Scheduler(), [8], elementwise_affine=False)
    """)
    assert p.returncode != 0 and "elementwise_affine" in (p.stderr + p.stdout)


@pytest.mark.gpu
def test_padding_idx_state_matches_the_reference(host, sched):
    # src/compute/embedding.cpp:80-90
    assert host.Embedding.init(sched, 10, 4, padding_idx=3).padding_idx == -1
    assert host.Embedding.init(sched, 10, 4, padding_idx=0).padding_idx == -1
    assert host.Embedding.init(sched, 10, 4, padding_idx=-2).padding_idx == 8
    assert host.Embedding.init(sched, 10, 4).padding_idx == -1


@pytest.mark.gpu
def test_exception_in_a_main_stream_task_aborts_and_names_the_task():
    # src/threading/dynamic_scheduler.cpp:176-195: a std::exception escaping a kMain task body becomes
    # log critical + std::abort with the task's name.  Float indices make Embedding::forward's body throw
    # (TORCH_CHECK) before it launches anything; the device is idle when the process aborts.
    p = run_snippet("""
        import torch
        from core_scheduler_amd import _cs_host as h
        s = h.DynamicScheduler(0)
        state = h.Embedding.init(s, 10, 4)
        state.weight.wait()
        idx = h.from_torch(s, torch.zeros(2, 3, device="cuda:0"))
        idx.wait()
        torch.cuda.synchronize()
        h.Embedding.forward(s, state, idx)
        print("not reached")
    """)
    out = p.stdout + p.stderr
    assert p.returncode != 0 and "not reached" not in out, out
    assert "cs::compute::Embedding::forward" in out and "int32 or int64" in out, out


def test_module_names_are_checked():
    # include/module/module.h:73-85: empty names and names with a dot are rejected
    p = run_snippet("""
        from core_scheduler_amd import _cs_host as h
        root = h.Container()
        for name in ("", "a.b"):
            try:
                root.register_module(name, h.Container())
            except RuntimeError as e:
                print("raised:", e)
        root.register_module("ok", h.Container())
        print("states:", root.named_states(), "parameters:", root.named_parameters())
    """)
    assert p.stdout.count("raised:") == 2 and "states: [] parameters: []" in p.stdout, p.stdout + p.stderr
