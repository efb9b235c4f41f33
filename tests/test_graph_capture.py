"""The C-ABI entry points allocate nothing, synchronise nothing and touch only the stream they
are given, so a sequence of them can be captured into a HIP graph and replayed.  The test
captures a forward/backward slice of a transformer step (gather-add, LayerNorm, GeLU, fused
classifier, their backward kernels, embedding backward, one AdamW launch), replays it several
times on new inputs with eager work and synchronisations in between, and checks every replay
against the eager result."""
import ctypes

import pytest
import torch

from _util import assert_bit_exact, randint, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_captured_step_replays_match_eager():
    from core_scheduler_amd import _capi

    lib = _capi.load()
    P = ctypes.c_void_p
    B, T, C, V, S = 4, 64, 256, 1000, 1024
    N = B * T
    bf = torch.bfloat16

    def buf(shape, dtype=bf):
        return torch.empty(shape, dtype=dtype, device=DEV)

    wte, wpe = randn((V, C), 1, std=0.02, dtype=bf).to(DEV), randn((T, C), 2, std=0.02, dtype=bf).to(DEV)
    gamma, beta = torch.ones(C, device=DEV), torch.zeros(C, device=DEV)
    ids, tgt = buf((B, T), torch.int64), buf((N,), torch.int64)
    logits = buf((N, S))
    x, y, act = buf((N, C)), buf((N, C)), buf((N, C))
    mean, rstd = buf((N,), torch.float32), buf((N,), torch.float32)
    row_loss, loss, tw = buf((N,), torch.float32), buf((), torch.float32), buf((), torch.float32)
    dact, dy, dx = buf((N, C)), buf((N, C)), buf((N, C))
    dgamma, dbeta = buf((C,), torch.float32), buf((C,), torch.float32)
    dwte, dwpe = buf((V, C)), buf((T, C))
    w, g, m, v = (torch.zeros(V * C, device=DEV) for _ in range(4))
    ce_ws = buf((lib.cs_fused_classifier_workspace_bytes(N),), torch.uint8)
    ln_ws = buf((lib.cs_layernorm_backward_workspace_bytes(N, C),), torch.uint8)
    emb_ws = buf((lib.cs_embedding_backward_workspace_bytes(N, C, V),), torch.uint8)

    def p(t):
        return P(t.data_ptr())

    def step(stream):
        st = P(stream.cuda_stream)
        rc = [
            lib.cs_embedding_forward_add(p(wte), p(wpe), p(ids), p(x), B, T, C, V, 3, 1, st),
            lib.cs_layernorm_forward(p(x), p(gamma), p(beta), p(y), p(mean), p(rstd), N, C, 1e-5, 3, 3, 0, st),
            lib.cs_gelu_forward(p(y), p(act), N * C, 3, 1, st),
            lib.cs_fused_classifier(p(logits), p(logits), p(tgt), p(row_loss), p(loss), p(tw), p(ce_ws), ce_ws.numel(),
                                    N, V, S, -100, 1, 1.0, 3, 3, st),
            lib.cs_gelu_backward(p(act), p(y), p(dact), N * C, 3, 1, st),
            lib.cs_layernorm_backward(p(dact), p(x), p(mean), p(rstd), p(gamma), p(dx), p(dgamma), p(dbeta), p(ln_ws),
                                      ln_ws.numel(), N, C, 3, 3, 3, 0, 0, st),
            lib.cs_embedding_backward_fused(p(dx), p(ids), p(dwte), p(dwpe), p(emb_ws), emb_ws.numel(), B, T, C, V, 3, 1,
                                            0, st),
            lib.cs_adamw_step(p(w), p(g), p(m), p(v), None, V * C, 0, 1e-3, 0.9, 0.999, 1e-8, 1e-2, 1, st),
        ]
        assert all(code == 0 for code in rc), rc

    def fill(seed):
        ids.copy_(randint(0, V, (B, T), seed))
        tgt.copy_(randint(0, V, (N,), seed + 1))
        logits.copy_(randn((N, S), seed + 2, std=2.0, dtype=bf))
        g.copy_(randn((V * C,), seed + 3, std=1e-3))
        w.copy_(randn((V * C,), seed + 4, std=0.02))
        m.zero_()
        v.zero_()

    outputs = (x, y, act, logits, row_loss, loss, dact, dx, dgamma, dbeta, dwte, dwpe, w, m, v)

    def snapshot():
        torch.cuda.synchronize()
        return [t.clone() for t in outputs]

    # eager reference for every input set (this also makes the one-time per-device set-up calls
    # of the library happen before any capture)
    eager = []
    for seed in (10, 20, 30, 40):
        fill(seed)
        step(torch.cuda.current_stream())
        eager.append(snapshot())

    graph = torch.cuda.CUDAGraph()
    fill(10)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream())
    for i, seed in enumerate((10, 20, 30, 40)):
        fill(seed)
        scratch = torch.randn(1 << 20, device=DEV).sum()  # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for a, b, name in zip(got, eager[i], "x y act dlogits row_loss loss dact dx dgamma dbeta dwte dwpe w m v".split()):
            assert_bit_exact(a, b, f"replay {i}: {name}")
        del scratch


def test_two_streams_give_the_serial_results():
    """The library keeps no per-call state of its own: the same ops issued on two streams at once,
    each with its own buffers and workspaces, give bit for bit what each gives alone."""
    from core_scheduler_amd import ops

    def work(seed):
        B, T, C, V = 8, 512, 768, 50257
        ids = randint(0, V, (B, T), seed).to(DEV)
        dout = randn((B, T, C), seed + 1, dtype=torch.bfloat16).to(DEV)
        x = randn((B * T, C), seed + 2, dtype=torch.bfloat16).to(DEV)
        gamma, beta = randn((C,), seed + 3).to(DEV), randn((C,), seed + 4).to(DEV)
        logits = randn((512, 50304), seed + 5, std=2.0, dtype=torch.bfloat16).to(DEV)
        tgt = randint(0, V, (512,), seed + 6).to(DEV)
        return dict(ids=ids, dout=dout, x=x, gamma=gamma, beta=beta, logits=logits, tgt=tgt, V=V)

    def run(wk):
        y, mean, rstd = ops.layernorm_forward(wk["x"], wk["gamma"], wk["beta"])
        dx, dgamma, dbeta = ops.layernorm_backward(wk["dout"].reshape(wk["x"].shape), wk["x"], mean, rstd, wk["gamma"])
        dwte, dwpe = ops.embedding_backward_fused(wk["dout"], wk["ids"], wk["V"])
        loss, row, d, _ = ops.fused_classifier(wk["logits"], wk["tgt"], wk["V"])
        act = ops.gelu_forward(y, "tanh")
        return [y, mean, rstd, dx, dgamma, dbeta, dwte, dwpe, loss, row, d, act]

    works = [work(500), work(600)]
    alone = [run(w) for w in works]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEV), torch.cuda.Stream(device=DEV)]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    together = [None, None]
    for rep in range(3):  # interleave the submissions
        for k, s in enumerate(streams):
            with torch.cuda.stream(s):
                together[k] = run(works[k])
    torch.cuda.synchronize()
    for k in range(2):
        for i, (a, b) in enumerate(zip(alone[k], together[k])):
            assert_bit_exact(b, a, f"stream {k} output {i}")
