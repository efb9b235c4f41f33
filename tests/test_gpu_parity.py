"""Parity of the gfx950 kernels with the CPU oracle, through the C ABI.

Every test feeds the same seeded inputs to the HIP path (core_scheduler_amd.ops
-> ctypes -> libcs_hip_kernels.so) and to the oracle (oracle/cs_oracle.c).
The bar (see tests/_util.py): bit-exact for the gather and gather-add;
fp32 within rtol 1e-5 plus the atol stated at each call; 16-bit outputs within
1 ulp of the oracle's once-rounded value.
Shapes follow the reference's own tests (test/test_*.cpp) and the benchmark
configurations; the largest ones are checked through the oracle on a sample of
rows plus properties that hold at any size.
"""
import math
import numpy as np

import pytest
import torch

from _util import (assert_bit_exact, assert_close, assert_sum_close, gpt2_param_shapes, randint, randn,
                   scatter_sum_tolerance, sum_tolerance,
                   zipf_ids)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from core_scheduler_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def co():
    from oracle import c_oracle

    return c_oracle


def dev(t):
    return None if t is None else t.to(DEV)


HYPER = dict(lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


# ------------------------------------------------------------------ AdamW
@pytest.mark.parametrize("n", [1, 127, 4096, 4097, 100003])
@pytest.mark.parametrize("amsgrad", [False, True])
def test_adamw_flat_f32(ops, co, n, amsgrad):
    w = randn(n, 1, std=0.02)
    m, v = torch.zeros(n), torch.zeros(n)
    x = torch.zeros(n) if amsgrad else None
    gw, gm, gv, gx = dev(w), dev(m), dev(v), dev(x)
    for t in range(1, 4):
        g = randn(n, 10 + t, std=1e-3)
        ops.adamw_step(gw, dev(g), gm, gv, t=t, v_max=gx, **HYPER)
        w, m, v, x = co.adamw_step(w, g, m, v, t=t, v_max=x, **HYPER)
    assert_close(gw, w, atol=1e-8, name="w")
    assert_close(gm, m, atol=1e-10, name="m")
    assert_close(gv, v, atol=1e-13, name="v")
    if amsgrad:
        assert_close(gx, x, atol=1e-13, name="v_max")


def test_adamw_reference_test_case(ops):
    # test/test_adamw.cpp:63-103, closed form written out there, its own tolerances
    for size in (128, 512, 1024):
        x = torch.rand(size, generator=torch.Generator().manual_seed(1))
        dx = torch.rand(size, generator=torch.Generator().manual_seed(2))
        gw, gm, gv = dev(x), dev(torch.zeros(size)), dev(torch.zeros(size))
        ops.adamw_step(gw, dev(dx), gm, gv, lr=1.0, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-2, t=1)
        xt = x - 1.0 * 1e-2 * x
        mt = (1 - 0.9) * dx
        vt = (1 - 0.999) * dx.square()
        xt = xt - 1.0 * (mt / (1 - 0.9)) / ((vt / (1 - 0.999)).sqrt() + 1e-8)
        assert torch.allclose(gw.cpu(), xt, 1e-4, 1e-5)
        assert torch.allclose(gm.cpu(), mt, 1e-4, 1e-5)
        assert torch.allclose(gv.cpu(), vt, 1e-4, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float64, torch.bfloat16, torch.float16])
def test_adamw_other_dtypes(ops, co, dtype):
    n = 9001
    w, g = randn(n, 2, std=0.5, dtype=dtype), randn(n, 3, std=0.1, dtype=dtype)
    m, v = torch.zeros(n, dtype=dtype), torch.zeros(n, dtype=dtype)
    gw, gm, gv = dev(w), dev(m), dev(v)
    ops.adamw_step(gw, dev(g), gm, gv, t=1, **HYPER)
    w2, m2, v2, _ = co.adamw_step(w, g, m, v, t=1, **HYPER)
    atol = 1e-14 if dtype == torch.float64 else 1e-7
    assert_close(gw, w2, atol=atol, name="w")
    assert_close(gm, m2, atol=atol, name="m")
    assert_close(gv, v2, atol=atol * 1e-3, name="v")


def test_adamw_unaligned_views(ops, co):
    # element 1 of an aligned buffer: 4-byte but not 16-byte aligned -> scalar path
    n = 5000
    bufs = [randn(n + 1, s, std=0.02) for s in (4, 5)] + [torch.zeros(n + 1), torch.zeros(n + 1)]
    gb = [dev(b) for b in bufs]
    ops.adamw_step(gb[0][1:], gb[1][1:], gb[2][1:], gb[3][1:], t=1, **HYPER)
    w2, m2, v2, _ = co.adamw_step(bufs[0][1:], bufs[1][1:], bufs[2][1:], bufs[3][1:], t=1, **HYPER)
    assert_close(gb[0][1:], w2, atol=1e-8, name="w")
    assert gb[0][0].item() == bufs[0][0].item() and gb[2][0].item() == 0  # the neighbour is untouched


def test_adamw_multi_tensor_small_set(ops, co):
    shapes = [(7,), (4096,), (33, 129), (4097,), (1,), (3, 5, 7)]
    ws = [randn(s, 20 + i, std=0.02) for i, s in enumerate(shapes)]
    gs = [randn(s, 40 + i, std=1e-3) for i, s in enumerate(shapes)]
    gws, ggs = [dev(w) for w in ws], [dev(g) for g in gs]
    flat = [w.clone() for w in gws]
    opt = ops.MultiTensorAdamW(gws, ggs, t=0, **HYPER)
    fm = [torch.zeros_like(w) for w in flat]
    fv = [torch.zeros_like(w) for w in flat]
    for t in range(1, 4):
        opt.step()
        for w, g, m, v in zip(flat, ggs, fm, fv):
            ops.adamw_step(w, g, m, v, t=t, **HYPER)
    ms = [torch.zeros(s) for s in shapes]
    vs = [torch.zeros(s) for s in shapes]
    for i in range(len(shapes)):
        w, m, v = ws[i], ms[i], vs[i]
        for t in range(1, 4):
            w, m, v, _ = co.adamw_step(w, gs[i], m, v, t=t, **HYPER)
        assert_close(gws[i], w.reshape(shapes[i]), atol=1e-8, name=f"w[{i}]")
        assert_close(opt.m[i], m.reshape(shapes[i]), atol=1e-10, name=f"m[{i}]")
        assert_bit_exact(gws[i], flat[i], f"multi == flat [{i}]")  # same arithmetic, two launch shapes


def test_adamw_multi_tensor_refresh_back_to_back_uses_each_steps_own_gradients(ops):
    """Gradients are re-allocated every step, so the descriptor table is rebuilt and uploaded
    every step while the host runs ahead of the device: each queued step must see the table
    that was built for it, not a later one."""
    n = 1 << 20
    w = dev(randn(n, 70, std=0.02))
    ref = w.clone()
    grads = [dev(randn(n, 71 + i, std=1e-3)) for i in range(6)]
    opt = ops.MultiTensorAdamW([w], [grads[0]], t=0, **HYPER)
    m, v = torch.zeros_like(ref), torch.zeros_like(ref)
    blocker_a = torch.empty(1 << 28, dtype=torch.uint8, device=DEV)
    blocker_b = torch.empty_like(blocker_a)
    for _ in range(8):
        blocker_b.copy_(blocker_a)  # the device is busy while the host queues all six steps
    for g in grads:
        opt.refresh([g])
        opt.step()
    torch.cuda.synchronize()
    for t, g in enumerate(grads, 1):
        ops.adamw_step(ref, g, m, v, t=t, **HYPER)
    assert_bit_exact(w, ref, "six queued steps, one table upload each")


def test_adamw_gpt2_small_ten_steps(ops, co):
    """Benchmark configuration 0: all 148 GPT-2-small tensors, 10 steps, fresh grads each step."""
    shapes = gpt2_param_shapes()
    sizes = [math.prod(s) for s in shapes]
    total = sum(sizes)
    assert len(shapes) == 148 and total == 124_439_808
    w = randn(total, 1337, std=0.02)
    gw_flat = dev(w)
    gg_flat = torch.empty(total, device=DEV)
    offs = [0]
    for s in sizes:
        offs.append(offs[-1] + s)
    gws = [gw_flat[offs[i]:offs[i + 1]] for i in range(len(sizes))]
    ggs = [gg_flat[offs[i]:offs[i + 1]] for i in range(len(sizes))]
    opt = ops.MultiTensorAdamW(gws, ggs, t=0, **HYPER)
    m, v = torch.zeros(total), torch.zeros(total)
    for t in range(1, 11):
        g = randn(total, 2000 + t, std=1e-3)
        gg_flat.copy_(g)
        opt.step()
        w, m, v, _ = co.adamw_step(w, g, m, v, t=t, **HYPER)
    assert_close(gw_flat, w, atol=1e-8, name="w after 10 steps")
    assert_close(torch.cat([x.flatten() for x in opt.m]), m, atol=1e-10, name="m")
    assert_close(torch.cat([x.flatten() for x in opt.v]), v, atol=1e-13, name="v")


@pytest.mark.parametrize("norm_type", [2.0, float("inf")])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_clip_grad_norm_and_clipped_step(ops, co, norm_type, dtype):
    """Utils::clip_grad_norm_ (src/compute/utils.cpp:700-746): norm, coefficient, in-place scaling,
    and the step that applies the coefficient while it reads the gradients."""
    shapes = [(7,), (4096,), (33, 129), (4097,), (1,), (3, 5, 7), (50000,)]
    ws = [randn(s, 20 + i, std=0.02, dtype=dtype) for i, s in enumerate(shapes)]
    gs = [randn(s, 40 + i, std=1e-1, dtype=dtype) for i, s in enumerate(shapes)]
    max_norm = 1.0 if norm_type == 2.0 else 0.1
    scaled, total, coef = co.clip_grad_norm(gs, max_norm, norm_type)
    assert coef < 1.0  # this case clips
    # (a) in-place clip, as the reference leaves the gradients
    gws, ggs = [dev(w) for w in ws], [dev(g) for g in gs]
    opt = ops.MultiTensorAdamW(gws, ggs, t=0, **HYPER)
    norm = opt.clip_grad_norm_(max_norm, norm_type)
    assert abs(norm.item() - total) <= 1e-5 * total
    for i in range(len(shapes)):
        assert_close(ggs[i], scaled[i], atol=1e-9, name=f"scaled g[{i}]")
    # (b) the fused form leaves the gradients alone and makes the same update as (a) + plain step
    gws2, ggs2 = [dev(w) for w in ws], [dev(g) for g in gs]
    opt2 = ops.MultiTensorAdamW(gws2, ggs2, t=0, **HYPER)
    norm2 = opt2.step(max_grad_norm=max_norm, norm_type=norm_type)
    assert norm2.item() == norm.item()  # the same two launches: the same bits
    opt.step()
    for i in range(len(shapes)):
        assert_bit_exact(ggs2[i], gs[i], f"gradient {i} untouched")
        assert_bit_exact(gws2[i], gws[i], f"fused == clip then step [{i}]")
        w2, _, _, _ = co.adamw_step(ws[i], scaled[i], torch.zeros_like(ws[i]), torch.zeros_like(ws[i]), t=1, **HYPER)
        assert_close(gws2[i], w2.reshape(shapes[i]), atol=1e-6, name=f"w[{i}]")
    # (c) below the threshold nothing changes
    opt3 = ops.MultiTensorAdamW([dev(w) for w in ws], [dev(g) for g in gs], t=0, **HYPER)
    opt3.clip_grad_norm_(1e9, norm_type)
    for i in range(len(shapes)):
        assert_bit_exact(opt3._grads[i], gs[i], f"no clipping [{i}]")


def test_grad_norm_gpt2_small_closed_form(ops):
    """All 124M gradients equal to c: the 2-norm is c * sqrt(n), the largest magnitude is c."""
    shapes = gpt2_param_shapes()
    sizes = [math.prod(s) for s in shapes]
    total = sum(sizes)
    flat_w = torch.zeros(total, device=DEV)
    flat_g = torch.full((total,), 3e-3, device=DEV)
    offs = [0]
    for s in sizes:
        offs.append(offs[-1] + s)
    opt = ops.MultiTensorAdamW([flat_w[offs[i]:offs[i + 1]] for i in range(len(sizes))],
                               [flat_g[offs[i]:offs[i + 1]] for i in range(len(sizes))], t=0, **HYPER)
    c = torch.tensor(3e-3, dtype=torch.float32).item()
    n2 = opt.grad_norm(1.0, 2.0).item()
    assert abs(n2 - c * math.sqrt(total)) <= 1e-6 * c * math.sqrt(total)
    assert abs(opt._clip.item() - 1.0 / (n2 + 1e-6)) <= 1e-6
    assert opt.grad_norm(1.0, float("inf")).item() == c


# ------------------------------------------------------------------- GeLU
GELU_ATOL = {torch.float32: 1e-6, torch.float64: 1e-14, torch.bfloat16: 1e-6, torch.float16: 1e-6}


@pytest.mark.parametrize("mode", ["none", "tanh"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("n", [1, 1000, 8192, 2 * 1024 * 768 + 3])
def test_gelu(ops, co, mode, dtype, n):
    # reference shapes: B=2, T in {128,512,1024} (test/test_gelu.cpp:59-102)
    x = randn(n, 3, std=1.5, dtype=dtype)
    dy = randn(n, 4, dtype=dtype)
    atol = GELU_ATOL[dtype]
    assert_close(ops.gelu_forward(dev(x), mode), co.gelu_forward(x, mode), atol=atol, name="fwd")
    # backward: the fp32 floor scales with |dy| (up to ~5) and |x|
    assert_close(ops.gelu_backward(dev(dy), dev(x), mode), co.gelu_backward(dy, x, mode), atol=atol * 5, name="bwd")


def test_gelu_edge_values(ops, co):
    x = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 20.0, -20.0, 88.0, -88.0, float("inf"), float("-inf")] * 8)
    for mode in ("none", "tanh"):
        for dtype in (torch.float32, torch.bfloat16):
            xx = x.to(dtype)
            got = ops.gelu_forward(dev(xx), mode).cpu().float()
            want = co.gelu_forward(xx, mode).float()
            finite = torch.isfinite(x)
            assert_close(got[finite], want[finite], atol=1e-6, name=f"{mode} {dtype}")
            assert got[8] == float("inf")  # gelu(+inf) = +inf; gelu(-inf) is 0 * inf in ATen's form (NaN)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode", ["none", "tanh"])
def test_gelu_every_16_bit_pattern(ops, co, mode, dtype):
    """All 65536 bit patterns of the storage type, forward and backward: finite inputs against the
    oracle, NaN in -> NaN out.  (Beyond |x| = 1e18 the reference's tanh derivative overflows into
    0 * inf = NaN where the value is 0 or 1; those are not compared.)"""
    x = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    ok = torch.isfinite(x.float()) & (x.float().abs() < 1e18)
    y, y2 = ops.gelu_forward(dev(x), mode).cpu(), co.gelu_forward(x, mode)
    assert_close(y[ok], y2[ok], atol=1e-6, name="forward")
    d, d2 = ops.gelu_backward(dev(torch.ones_like(x)), dev(x), mode).cpu(), co.gelu_backward(torch.ones_like(x), x, mode)
    assert_close(d[ok], d2[ok], atol=5e-6, name="backward")
    nan_in = torch.isnan(x.float())
    assert torch.isnan(y[nan_in].float()).all() and torch.isnan(d[nan_in].float()).all()
    assert not torch.isnan(d[ok].float()).any()


def test_gelu_config3_full_size(ops, co):
    x = randn((8192, 3072), 1340, std=1.5, dtype=torch.bfloat16)
    dy = randn((8192, 3072), 1341, dtype=torch.bfloat16)
    assert_close(ops.gelu_forward(dev(x), "tanh"), co.gelu_forward(x, "tanh"), atol=1e-6, name="fwd")
    assert_close(ops.gelu_backward(dev(dy), dev(x), "tanh"), co.gelu_backward(dy, x, "tanh"), atol=5e-6, name="bwd")


# -------------------------------------------------------------- LayerNorm
def _ln_case(ops, co, rows, C, x_dtype, p_dtype, bias=True, atol_y=2e-6):
    x = randn((rows, C), 50, dtype=x_dtype)
    gamma = randn(C, 51, std=0.02, mean=1.0, dtype=p_dtype)
    beta = randn(C, 52, std=0.02, dtype=p_dtype) if bias else None
    dy = randn((rows, C), 53, dtype=x_dtype)
    y, mean, rstd = ops.layernorm_forward(dev(x), dev(gamma), dev(beta), 1e-5)
    y2, mean2, rstd2 = co.layernorm_forward(x, gamma, beta, 1e-5)
    wide = x_dtype != torch.float64
    assert mean.dtype == (torch.float32 if wide else torch.float64)
    assert_close(y, y2, atol=atol_y, name="y")
    assert_close(mean, mean2, atol=1e-7, name="mean")
    assert_close(rstd, rstd2, atol=1e-6, name="rstd")
    # backward from the oracle's statistics, so only the backward kernel is judged
    dx, dg, db = ops.layernorm_backward(dev(dy), dev(x), dev(mean2), dev(rstd2), dev(gamma), need_dbeta=bias)
    dx2, dg2, db2 = co.layernorm_backward(dy, x, mean2, rstd2, gamma)
    assert_close(dx, dx2, atol=5e-6, name="dx")
    # dgamma and dbeta are column sums over the rows of dy * xhat and dy: the bar is derived from
    # those terms (see sum_tolerance), not a constant per row
    if wide:
        xhat = (x.double() - mean2.double().reshape(-1, 1)) * rstd2.double().reshape(-1, 1)
        tol_g, tol_b = sum_tolerance(dy.double() * xhat), sum_tolerance(dy)
    else:
        tol_g = tol_b = torch.full((C,), 1e-14, dtype=torch.float64)
    assert_sum_close(dg, dg2, tol_g, name="dgamma")
    if bias:
        assert_sum_close(db, db2, tol_b, name="dbeta")
    else:
        assert db is None


@pytest.mark.parametrize("rows,C,x_dtype,p_dtype", [
    (8192, 768, torch.bfloat16, torch.float32),     # benchmark configuration 3
    (2048, 1600, torch.bfloat16, torch.float32),    # XL width (2 rows per wave plan)
    (1024, 384, torch.float32, torch.float32),      # test/test_layer_norm.cpp:63-96 width
    (513, 768, torch.float16, torch.float16),
    (300, 768, torch.bfloat16, torch.bfloat16),
    (77, 4096, torch.bfloat16, torch.float32),      # 8 vectors per lane plan: two waves per row backward
    (2051, 1600, torch.float32, torch.float32),     # the same plan from fp32 rows, rows not a multiple of anything
    (3, 4096, torch.float16, torch.float16),        # fewer rows than wave pairs
    (1100, 2056, torch.bfloat16, torch.float32),    # just over 4 vectors per lane, several rows per pair
    (5, 768, torch.float32, torch.float32),         # fewer rows than one workgroup
    (4096, 384, torch.bfloat16, torch.float32),     # one vector per lane, 48 of 64 lanes busy
    (1000, 512, torch.float16, torch.float16),      # one vector per lane, every lane busy
    (777, 256, torch.float32, torch.float32),       # the same plan from fp32 rows
    (300, 8, torch.bfloat16, torch.bfloat16),       # a single vector per row
    (64, 50, torch.float32, torch.float32),         # C not a multiple of the vector width
    (2049, 50, torch.float32, torch.float32),       # the same with long column sums
    (33, 10000, torch.bfloat16, torch.float32),     # beyond the register plans
    (128, 384, torch.float64, torch.float64),       # test/test_layer_norm.cpp:99-134
    (301, 256, torch.bfloat16, torch.float32),      # two rows per wave, one vector per lane, odd row count
    (1001, 128, torch.float32, torch.float32),      # the same from fp32 rows
    (999, 760, torch.bfloat16, torch.float32),      # two rows per wave, 95 of 96 vector slots used
    (7, 24, torch.float16, torch.float16),          # three vectors per row
])
def test_layernorm(ops, co, rows, C, x_dtype, p_dtype):
    _ln_case(ops, co, rows, C, x_dtype, p_dtype)


@pytest.mark.parametrize("rows,C,x_dtype,p_dtype", [
    (8192, 768, torch.bfloat16, torch.float32),     # benchmark configuration 3
    (2048, 1600, torch.bfloat16, torch.float32),    # XL width
    (1024, 384, torch.float32, torch.float32),
    (513, 768, torch.float16, torch.float16),
    (77, 4096, torch.bfloat16, torch.float32),      # 8 vectors per lane plan
    (5, 768, torch.float32, torch.float32),
    (2000, 384, torch.bfloat16, torch.float32),     # one vector per lane
    (100, 64, torch.float16, torch.float16),
    (64, 50, torch.float32, torch.float32),         # general path
    (33, 10000, torch.bfloat16, torch.float32),     # general path
    (128, 384, torch.float64, torch.float64),
    (301, 256, torch.bfloat16, torch.float32),      # two rows per wave, one vector per lane, odd row count
    (999, 760, torch.bfloat16, torch.float32),      # two rows per wave, 95 of 96 vector slots used
])
def test_layernorm_with_residual_stream(ops, co, rows, C, x_dtype, p_dtype):
    """x + residual -> LayerNorm, and LayerNorm backward + dresidual, each in one pass
    (example/gpt2/gpt2_single_device.cpp:459-460 and :468-469).  The fused results must be the
    bits of the separate kernels, and agree with the oracle applied to the rounded sum."""
    x = randn((rows, C), 60, dtype=x_dtype)
    res = randn((rows, C), 61, dtype=x_dtype)
    gamma = randn(C, 62, std=0.02, mean=1.0, dtype=p_dtype)
    beta = randn(C, 63, std=0.02, dtype=p_dtype)
    dy = randn((rows, C), 64, dtype=x_dtype)
    dres = randn((rows, C), 65, dtype=x_dtype)
    gx, gres, gg, gb = dev(x), dev(res), dev(gamma), dev(beta)
    total, y, mean, rstd = ops.add_layernorm_forward(gx, gres, gg, gb, 1e-5)
    wide = torch.float64 if x_dtype == torch.float64 else torch.float32
    total_ref = (x.to(wide) + res.to(wide)).to(x_dtype)   # one add, one rounding
    assert_bit_exact(total, total_ref, "x + residual")
    y_sep, mean_sep, rstd_sep = ops.layernorm_forward(dev(total_ref), gg, gb, 1e-5)
    # rows of 5 to 8 vectors per lane run the register-resident kernel only without a residual,
    # so there the two results come from different summation orders
    vec_per_lane = -(-C * x.element_size() // 16 // 64)
    same_kernel = not (4 < vec_per_lane <= 8 and C * x.element_size() % 16 == 0 and x_dtype != torch.float64)
    same = assert_bit_exact if same_kernel else (lambda a, b, name: assert_close(a, b, atol=2e-6, name=name))
    same(y, y_sep, "y: fused == separate kernels")
    same(mean, mean_sep, "mean")
    same(rstd, rstd_sep, "rstd")
    y2, mean2, rstd2 = co.layernorm_forward(total_ref, gamma, beta, 1e-5)
    assert_close(y, y2, atol=2e-6, name="y vs oracle")
    assert_close(rstd, rstd2, atol=1e-6, name="rstd vs oracle")
    # in place: the sum lands in x's buffer
    gx2 = dev(x).clone()
    t2, y_ip, _, _ = ops.add_layernorm_forward(gx2, gres, gg, gb, 1e-5, inplace=True)
    assert t2.data_ptr() == gx2.data_ptr()
    assert_bit_exact(gx2, total_ref, "in-place sum")
    assert_bit_exact(y_ip, y, "in-place y")
    # backward
    gdy, gdres, gm, gr = dev(dy), dev(dres), dev(mean2), dev(rstd2)
    dx, dg, db = ops.layernorm_backward(gdy, dev(total_ref), gm, gr, gg, dresidual=gdres)
    dx_sep, dg_sep, db_sep = ops.layernorm_backward(gdy, dev(total_ref), gm, gr, gg)
    want = (dx_sep.to(wide) + gdres.to(wide)).to(x_dtype)
    if same_kernel:
        assert_bit_exact(dx, want, "dx: fused == separate kernels")
        assert_bit_exact(dg, dg_sep, "dgamma")
        assert_bit_exact(db, db_sep, "dbeta")
    # against the oracle: dx itself is held to one unit in the last place of dx, and that unit can
    # be several units of a smaller sum, so the bound is taken at the size of the terms
    dx2, _, _ = co.layernorm_backward(dy, total_ref, mean2, rstd2, gamma)
    want2 = dx2.to(wide) + dres.to(wide)
    unit = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5, torch.float64: 1e-12}[x_dtype]
    err = (dx.cpu().to(wide) - want2).abs()
    bound = unit * (dx2.to(wide).abs() + want2.abs()) + 5e-6
    assert (err <= bound).all(), f"dx vs oracle: max excess {(err - bound).max().item():.3e}"
    only_dx, none_g, none_b = ops.layernorm_backward(gdy, dev(total_ref), gm, gr, gg, need_dgamma=False,
                                                     need_dbeta=False, dresidual=gdres)
    assert none_g is None and none_b is None
    assert_bit_exact(only_dx, dx, "dx with mask {1,0,0}")


def test_layernorm_without_bias(ops, co):
    _ln_case(ops, co, 256, 768, torch.bfloat16, torch.float32, bias=False)
    _ln_case(ops, co, 64, 50, torch.float32, torch.float32, bias=False)


def test_layernorm_reference_test_values(ops):
    # test/test_layer_norm.cpp:63-96: x = rand, weight 1, bias 0, against torch's LayerNorm (ATen CPU here)
    x = torch.rand((16, 256, 384), generator=torch.Generator().manual_seed(1))
    w, b = torch.ones(384), torch.zeros(384)
    y, mean, rstd = ops.layernorm_forward(dev(x), dev(w), dev(b), 1e-5)
    xr = x.clone().requires_grad_()
    ln = torch.nn.LayerNorm(384)
    yr = ln(xr)
    dy = torch.rand(yr.shape, generator=torch.Generator().manual_seed(2))
    yr.backward(dy)
    dx, dg, db = ops.layernorm_backward(dev(dy), dev(x), mean, rstd, dev(w))
    assert_close(y, yr.detach(), atol=2e-6, name="y")
    assert_close(dx, xr.grad, atol=5e-6, name="dx")
    assert_close(dg, ln.weight.grad, atol=1e-3, rtol=1e-5, name="dgamma")  # sums of 4096 terms ~ 2e3
    assert_close(db, ln.bias.grad, atol=1e-3, rtol=1e-5, name="dbeta")


def test_layernorm_autocast_dtypes(ops, co):
    # test/test_autocast.cpp:112-156: bf16 x, fp32 parameters, fp32 y and fp32 dy/dx
    rows, C = 512, 768
    x = randn((rows, C), 60, dtype=torch.bfloat16)
    gamma, beta = randn(C, 61, std=0.02, mean=1.0), randn(C, 62, std=0.02)
    dy = randn((rows, C), 63)
    y, mean, rstd = ops.layernorm_forward(dev(x), dev(gamma), dev(beta), 1e-5, out_dtype=torch.float32)
    y2, mean2, rstd2 = co.layernorm_forward(x, gamma, beta, 1e-5, out_dtype=torch.float32)
    assert y.dtype == torch.float32
    assert_close(y, y2, atol=2e-6, name="y fp32")
    dx, dg, db = ops.layernorm_backward(dev(dy), dev(x), mean, rstd, dev(gamma), dx_dtype=torch.float32)
    dx2, dg2, db2 = co.layernorm_backward(dy, x, mean2, rstd2, gamma, out_dtype=torch.float32)
    assert_close(dx, dx2, atol=5e-6, name="dx fp32")
    assert_close(dg, dg2, atol=1e-5, name="dgamma")
    assert_close(db, db2, atol=1e-5, name="dbeta")


def test_layernorm_masks_and_accumulate(ops, co):
    rows, C = 700, 768
    x = randn((rows, C), 70, dtype=torch.bfloat16)
    gamma = randn(C, 71, std=0.02, mean=1.0)
    dy = randn((rows, C), 72, dtype=torch.bfloat16)
    _, mean, rstd = co.layernorm_forward(x, gamma, None, 1e-5)
    gx, gdy, gm, gr, gg = dev(x), dev(dy), dev(mean), dev(rstd), dev(gamma)
    full = ops.layernorm_backward(gdy, gx, gm, gr, gg)
    only_dx = ops.layernorm_backward(gdy, gx, gm, gr, gg, need_dgamma=False, need_dbeta=False)
    only_p = ops.layernorm_backward(gdy, gx, gm, gr, gg, need_dx=False)
    assert only_dx[1] is None and only_dx[2] is None and only_p[0] is None
    assert_bit_exact(only_dx[0], full[0], "dx alone")          # the reference's mask {1,0,0}
    assert_bit_exact(only_p[1], full[1], "dgamma alone")       # mask {0,1,1}
    assert_bit_exact(only_p[2], full[2], "dbeta alone")
    # += into existing gradients (src/compute/layer_norm.cpp:325-334)
    dg0, db0 = randn(C, 73), randn(C, 74)
    gdg, gdb = dev(dg0), dev(db0)
    ops.layernorm_backward(gdy, gx, gm, gr, gg, need_dx=False, dgamma=gdg, dbeta=gdb)
    _, dg2, db2 = co.layernorm_backward(dy, x, mean, rstd, gamma, dgamma=dg0, dbeta=db0)
    assert_close(gdg, dg2, atol=1e-5, name="dgamma +=")
    assert_close(gdb, db2, atol=1e-5, name="dbeta +=")
    # determinism: same bits on a second run
    again = ops.layernorm_backward(gdy, gx, gm, gr, gg)
    for a, b in zip(again, full):
        assert_bit_exact(a, b, "rerun")


@pytest.mark.parametrize("rows,C,x_dtype,p_dtype,wide_dy", [
    (8192, 768, torch.bfloat16, torch.float32, False),    # benchmark configuration 3
    (700, 768, torch.bfloat16, torch.float32, True),      # the autocast combination: fp32 dy and dx
    (2048, 1600, torch.bfloat16, torch.float32, False),   # XL width
    (513, 768, torch.float16, torch.float16, False),
    (77, 4096, torch.bfloat16, torch.float32, False),     # two waves per row
    (2051, 1600, torch.float32, torch.float32, False),
    (3, 768, torch.float32, torch.float32, False),
    (1500, 384, torch.bfloat16, torch.float32, True),     # one vector per lane
    (1027, 1600, torch.bfloat16, torch.float32, False),   # four vectors per lane: the sums alone run another kernel
    (2049, 768, torch.float16, torch.float16, False),     # two rows per wave
])
def test_layernorm_backward_as_two_calls(ops, rows, C, x_dtype, p_dtype, wide_dy):
    """Row pass on one stream, sum of the partial rows on another (the reference's main and
    assist tasks, src/compute/layer_norm.cpp:228-233): the bits of the single call."""
    x = randn((rows, C), 80, dtype=x_dtype)
    gamma = randn(C, 81, std=0.02, mean=1.0, dtype=p_dtype)
    dy = randn((rows, C), 82, dtype=torch.float32 if wide_dy else x_dtype)
    mean = x.float().mean(-1)
    rstd = 1.0 / torch.sqrt(x.float().var(-1, unbiased=False) + 1e-5)
    res = randn((rows, C), 83, dtype=dy.dtype)
    gx, gdy, gm, gr, gg, gres = dev(x), dev(dy), dev(mean), dev(rstd), dev(gamma), dev(res)
    whole = ops.layernorm_backward(gdy, gx, gm, gr, gg, dx_dtype=dy.dtype)
    side = torch.cuda.Stream()
    dx, partials = ops.layernorm_backward_rows(gdy, gx, gm, gr, gg, dx_dtype=dy.dtype)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        dg, db = ops.layernorm_backward_finalize(partials, x_dtype, p_dtype)
    side.synchronize()
    assert_bit_exact(dx, whole[0], "dx")
    assert_bit_exact(dg, whole[1], "dgamma")
    assert_bit_exact(db, whole[2], "dbeta")
    # dgamma only, += into an existing gradient, and dresidual in the row pass
    dg0 = randn(C, 84, dtype=p_dtype)
    acc_whole = dev(dg0)
    ops.layernorm_backward(gdy, gx, gm, gr, gg, need_dx=False, need_dbeta=False, dgamma=acc_whole)
    acc = dev(dg0)
    got = ops.layernorm_backward_finalize(partials, x_dtype, p_dtype, need_dbeta=False, dgamma=acc)
    assert got[1] is None and got[0] is acc
    assert_bit_exact(acc, acc_whole, "dgamma +=")
    with_res = ops.layernorm_backward(gdy, gx, gm, gr, gg, dx_dtype=dy.dtype, dresidual=gres)
    dx_r, partials_r = ops.layernorm_backward_rows(gdy, gx, gm, gr, gg, dx_dtype=dy.dtype, dresidual=gres)
    assert_bit_exact(dx_r, with_res[0], "dx + dresidual")
    assert_bit_exact(ops.layernorm_backward_finalize(partials_r, x_dtype, p_dtype)[0], with_res[1], "dgamma, residual form")
    # no dx: the parameter half on its own
    none_dx, partials_p = ops.layernorm_backward_rows(gdy, gx, gm, gr, gg, need_dx=False)
    assert none_dx is None
    assert_bit_exact(ops.layernorm_backward_finalize(partials_p, x_dtype, p_dtype)[1], whole[2], "dbeta without dx")


@pytest.mark.parametrize("rows,C,x_dtype,p_dtype", [
    (8192, 768, torch.bfloat16, torch.float32),    # benchmark shape: two rows per wave, three vectors per lane
    (1001, 384, torch.float32, torch.float32),     # the same plan at fp32, odd row count
    (333, 256, torch.bfloat16, torch.bfloat16),    # two rows per wave, one vector per lane
    (515, 1600, torch.bfloat16, torch.float32),    # a wave per row, four vectors per lane
    (64, 1024, torch.float16, torch.float32),      # two vectors per lane
    (77, 4096, torch.bfloat16, torch.float32),     # two waves per row: pending sums get a launch of their own
])
def test_layernorm_backward_chain(ops, rows, C, x_dtype, p_dtype):
    """Calls whose column sums ride in the next call's launch (cs_layernorm_backward_rows_pending):
    the bits of cs_layernorm_backward for every call of the chain, with a residual gradient, with
    accumulation into existing gradients, and across a change of width."""
    gamma = dev(randn(C, 181, std=0.02, mean=1.0, dtype=p_dtype))
    calls = []
    for i in range(4):
        x = randn((rows, C), 190 + 10 * i, dtype=x_dtype)
        mean = x.float().mean(-1)
        rstd = 1.0 / torch.sqrt(x.float().var(-1, unbiased=False) + 1e-5)
        calls.append(dict(x=dev(x), dy=dev(randn((rows, C), 191 + 10 * i, dtype=x_dtype)), mean=dev(mean), rstd=dev(rstd),
                          res=dev(randn((rows, C), 192 + 10 * i, dtype=x_dtype)) if i % 2 else None,
                          acc=(randn(C, 193 + 10 * i, dtype=p_dtype), randn(C, 194 + 10 * i, dtype=p_dtype)) if i == 2 else None))
    want = []
    for c in calls:
        acc = (dev(c["acc"][0]), dev(c["acc"][1])) if c["acc"] else (None, None)
        want.append(ops.layernorm_backward(c["dy"], c["x"], c["mean"], c["rstd"], gamma, dresidual=c["res"],
                                           dgamma=acc[0], dbeta=acc[1]))
    chain = ops.LayerNormBackwardChain()
    got = []
    for i, c in enumerate(calls):
        acc = (dev(c["acc"][0]), dev(c["acc"][1])) if c["acc"] else (None, None)
        got.append(chain.backward(c["dy"], c["x"], c["mean"], c["rstd"], gamma, dresidual=c["res"],
                                  dgamma=acc[0], dbeta=acc[1]))
        if i == 1:
            # another width in between: the pending sums of call 1 are flushed by the chain itself
            C2 = 512
            x2 = dev(randn((40, C2), 300, dtype=x_dtype))
            m2, r2 = dev(randn(40, 301)), dev(randn(40, 302).abs() + 0.5)
            g2 = dev(randn(C2, 303, dtype=p_dtype))
            other = chain.backward(x2, x2, m2, r2, g2)
            other_want = ops.layernorm_backward(x2, x2, m2, r2, g2)
    chain.flush()
    chain.flush()  # nothing pending: no launch, no error
    for i, (g, w) in enumerate(zip(got, want)):
        assert_bit_exact(g[0], w[0], f"dx of call {i}")
        assert_bit_exact(g[1], w[1], f"dgamma of call {i}")
        assert_bit_exact(g[2], w[2], f"dbeta of call {i}")
    for a, b, name in zip(other, other_want, ("dx", "dgamma", "dbeta")):
        assert_bit_exact(a, b, f"{name} of the call of another width")


def test_layernorm_backward_pending_rejects_shared_buffers(ops):
    """The pending partial rows are read while this call's are written: one buffer for both is refused."""
    import ctypes

    from core_scheduler_amd import _capi
    lib = _capi.load()
    rows, C = 64, 768
    x = dev(randn((rows, C), 310, dtype=torch.bfloat16))
    m, r, g = dev(randn(rows, 311)), dev(randn(rows, 312).abs() + 0.5), dev(randn(C, 313))
    n = lib.cs_layernorm_backward_partial_rows(rows, C, _capi.BF16)
    partials = torch.empty((n, 2, C), dtype=torch.float32, device="cuda:0")
    dg = torch.empty(C, device="cuda:0")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    dx = torch.empty_like(x)
    code = lib.cs_layernorm_backward_rows_pending(P(x), P(x), P(m), P(r), P(g), None, P(dx), P(partials), partials.numel() * 4,
                                                  P(partials), n, P(dg), P(dg), 0, rows, C, _capi.BF16, _capi.BF16,
                                                  _capi.BF16, _capi.F32, st)
    assert code == _capi.ERR_INVALID_ARGUMENT


def test_layernorm_backward_shapes_without_two_call_form(ops):
    lib = __import__("core_scheduler_amd._capi", fromlist=["load"]).load()
    assert lib.cs_layernorm_backward_partial_rows(64, 50, 0) == 0       # C not a multiple of the vector
    assert lib.cs_layernorm_backward_partial_rows(64, 10000, 3) == 0    # wider than the register plans
    assert lib.cs_layernorm_backward_partial_rows(0, 768, 3) == 0
    x = dev(randn((64, 50), 85))
    with pytest.raises(ValueError):
        ops.layernorm_backward_rows(x, x, dev(randn(64, 86)), dev(randn(64, 87)), dev(randn(50, 88)))


@pytest.mark.parametrize("N,V,stride,dtype,grad_dtype", [
    (512, 50257, 50304, torch.bfloat16, torch.bfloat16),   # the GPT-2 vocabulary, padded stride: the streaming kernel
    (300, 50257, 50304, torch.bfloat16, torch.float32),    # the same under the autocast rule
    (200, 32000, 32000, torch.float16, torch.float16),     # streaming kernel, four vectors per lane
    (96, 30000, 30000, torch.float32, torch.float32),      # streaming kernel, fp32 rows
    (300, 50257, 50257, torch.bfloat16, torch.float32),    # unpadded rows, the autocast combination
    (1024, 384, 384, torch.float32, torch.float32),        # the reference's test width
    (77, 1000, 1003, torch.float16, torch.float16),
    (64, 33, 33, torch.float64, torch.float64),
])
@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_cross_entropy_with_class_weights(ops, co, N, V, stride, dtype, grad_dtype, reduction):
    """at::nll_loss's per-class `weight` (src/compute/cross_entropy.cpp:52-63, 97-105)."""
    x = randn((N, stride), 800, std=2.0, dtype=dtype)
    t = randint(0, V, (N,), 801)
    t[::11] = -100
    w = (torch.rand(V, generator=torch.Generator().manual_seed(802)) * 2 + 0.05).float()
    w[3] = 0.0  # a class that carries no weight at all
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), V, reduction=reduction, class_weight=dev(w),
                                            dlogits_dtype=grad_dtype)
    want_loss, want_row, want_d, want_tw = co.cross_entropy(x, t, V, reduction=reduction, class_weight=w,
                                                            dlogits_dtype=grad_dtype)
    assert_close(tw.cpu().double(), want_tw.double(), atol=1e-3, name="total weight")
    assert_close(row.cpu().double(), want_row.double(), atol=2e-5, name="row losses")
    if reduction != "none":
        assert_close(loss.cpu().double(), want_loss.double(), atol=2e-5 * (N if reduction == "sum" else 1),
                     name="loss")
    atol = {torch.float32: 1e-7, torch.float64: 1e-7}.get(grad_dtype, 1e-7)
    assert_close(d, want_d, atol=atol, name="dlogits")
    assert (d.cpu()[:, V:] == 0).all()
    assert (d.cpu()[t == -100] == 0).all()
    # all weights 1: the bits of the unweighted call's loss
    ones = ops.fused_classifier(dev(x), dev(t), V, reduction=reduction, class_weight=dev(torch.ones(V)),
                                dlogits_dtype=grad_dtype)
    plain = ops.fused_classifier(dev(x), dev(t), V, reduction=reduction, dlogits_dtype=grad_dtype)
    assert_close(ones[1], plain[1].cpu(), atol=2e-6, name="weights of 1: row losses of the plain call")
    assert_close(ones[2], plain[2].cpu(), atol=1e-7, name="weights of 1: gradient of the plain call")


# -------------------------------------------------------------- Embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("idx_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("V,C,B,T", [(4095, 512, 2, 1024), (97, 24, 3, 11), (50, 7, 2, 5)])
def test_embedding_forward_bit_exact(ops, co, dtype, idx_dtype, V, C, B, T):
    w = randn((V, C), 80, dtype=dtype)
    wpe = randn((T, C), 81, dtype=dtype)
    ids = randint(0, V, (B, T), 82, dtype=idx_dtype)
    assert_bit_exact(ops.embedding_forward(dev(w), dev(ids)), co.embedding_forward(w, ids), "gather")
    assert_bit_exact(ops.embedding_forward_add(dev(w), dev(wpe), dev(ids)), co.embedding_forward_add(w, wpe, ids),
                     "gather-add")


def test_embedding_forward_out_of_range_ids_give_zero_rows(ops):
    w = randn((10, 16), 83)
    ids = torch.tensor([[0, 9, 10, -1, 3]], dtype=torch.int64)
    out = ops.embedding_forward(dev(w), dev(ids)).cpu()
    assert torch.equal(out[0, 0], w[0]) and torch.equal(out[0, 1], w[9]) and torch.equal(out[0, 4], w[3])
    assert (out[0, 2] == 0).all() and (out[0, 3] == 0).all()


EMB_ATOL = {torch.float32: 2e-5, torch.float16: 1e-6, torch.bfloat16: 1e-6, torch.float64: 1e-12}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_embedding_backward_reference_test_case(ops, co, dtype):
    # test/test_embedding.cpp:58-97: B 2, T 1024, vocab 4095, d 512, int32 ids in [0, 3): 2048 rows onto 3
    B, T, V, C = 2, 1024, 4095, 512
    ids = randint(0, 3, (B, T), 90, dtype=torch.int32)
    dout = randn((B, T, C), 91, dtype=dtype)
    got = ops.embedding_backward(dev(dout), dev(ids), V)
    # sums of ~680 N(0,1) terms are ~26 in size: fp32 accumulation leaves ~1e-5 absolute
    assert_close(got, co.embedding_backward(dout, ids, V), atol=EMB_ATOL[dtype], name="dweight")
    assert (got[3:] == 0).all()
    assert_bit_exact(ops.embedding_backward(dev(dout), dev(ids), V), got, "rerun is bitwise identical")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("n,V,C", [(1, 5, 8), (8, 5, 8), (9, 40, 16), (2048, 300, 64), (2049, 1000, 72),
                                   (5000, 7, 128), (4097, 100000, 8), (300, 50, 12), (64, 20, 7),
                                   # 64-bit sort keys (V * padded n >= 2^32): ranked in one launch / tile-sorted
                                   (3000, 2000000, 8), (5000, 2000000, 8),
                                   # 32-bit keys either side of the longest list that is ranked in one launch
                                   (8192, 3000, 16), (8193, 3000, 16), (20000, 50, 8)])
def test_embedding_backward_shapes(ops, co, dtype, n, V, C):
    ids = randint(0, V, (n,), 92)
    dout = randn((n, C), 93, dtype=dtype)
    got = ops.embedding_backward(dev(dout), dev(ids), V)
    assert_close(got, co.embedding_backward(dout, ids, V), atol=EMB_ATOL[dtype] * 4, name="dweight")


def test_embedding_backward_padding_accumulate_and_bad_ids(ops, co):
    n, V, C = 3000, 64, 32
    ids = randint(0, V, (n,), 94)
    dout = randn((n, C), 95)
    got = ops.embedding_backward(dev(dout), dev(ids), V, padding_idx=5)
    assert (got[5] == 0).all()
    assert_close(got, co.embedding_backward(dout, ids, V, padding_idx=5), atol=2e-5, name="padding_idx")
    base = randn((V, C), 96)
    acc = dev(base)
    ops.embedding_backward(dev(dout), dev(ids), V, dweight=acc)
    assert_close(acc, co.embedding_backward(dout, ids, V, dweight=base), atol=2e-5, name="+=")
    bad = ids.clone()
    bad[::7] = V + 3
    bad[1::7] = -2
    assert_close(ops.embedding_backward(dev(dout), dev(bad), V), co.embedding_backward(dout, bad, V), atol=2e-5,
                 name="out-of-range ids are skipped")


@pytest.mark.parametrize("n,C,V,hi,dtype,idx_dtype", [
    (2048, 512, 4095, 3, torch.float32, torch.int32),        # the reference's hot-row case: three ids, 2048 entries
    (8192, 768, 50257, 50257, torch.bfloat16, torch.int64),   # benchmark shape, ids spread over the table
    (16384, 1600, 50257, 2000, torch.bfloat16, torch.int64),  # the sort + merge path, segments across windows
    (5000, 96, 300, 300, torch.float16, torch.int64),
    (777, 50, 40, 40, torch.float32, torch.int64),            # rows that are not whole vectors: general path
    (300, 64, 10, 10, torch.float64, torch.int32),
])
def test_embedding_backward_scale_grad_by_freq(ops, co, n, C, V, hi, dtype, idx_dtype):
    """at::embedding_backward(..., scale_grad_by_freq = true) (src/compute/embedding.cpp:147-157): a
    row's sum divided by the number of entries that name it; segments inside a wave, across the
    waves of a window and across windows all take their own count."""
    ids = randint(0, hi, (n,), 700, dtype=idx_dtype)
    ids[: n // 3] = 1 if hi > 1 else 0  # one id in a third of the entries: a segment over many windows
    dout = randn((n, C), 701, dtype=dtype)
    got = ops.embedding_backward(dev(dout), dev(ids), V, scale_grad_by_freq=True)
    want = co.embedding_backward(dout, ids, V, scale_grad_by_freq=True)
    tol = {torch.float32: 2e-6, torch.float64: 1e-12}.get(dtype, 1e-6)
    assert_close(got, want, atol=tol, name="dweight, scaled")
    assert not torch.equal(got.cpu(), co.embedding_backward(dout, ids, V))  # the option does something
    # padding row, and += into an existing gradient: only the new part is scaled
    pad = ops.embedding_backward(dev(dout), dev(ids), V, padding_idx=1, scale_grad_by_freq=True)
    assert_close(pad, co.embedding_backward(dout, ids, V, padding_idx=1, scale_grad_by_freq=True), atol=tol,
                 name="dweight, scaled, padding row")
    base = randn((V, C), 702, dtype=dtype)
    acc = ops.embedding_backward(dev(dout), dev(ids), V, dweight=dev(base).clone(), scale_grad_by_freq=True)
    assert_close(acc, co.embedding_backward(dout, ids, V, dweight=base.clone(), scale_grad_by_freq=True),
                 atol=4 * tol, name="+= of the scaled sums")
    again = ops.embedding_backward(dev(dout), dev(ids), V, scale_grad_by_freq=True)
    assert_bit_exact(again, got, "rerun")


def test_embedding_backward_random_cases(ops, co):
    """Seeded random shapes around the kernel's internal boundaries (32-entry windows, 4-entry
    waves, 1024-key tiles, the 32/64-bit key switch) with id patterns that stress each level of
    the segmented sum: one hot id, a sorted stream, a single id, a padding row; `=` and `+=`."""
    import random

    rnd = random.Random(7)
    for case in range(80):
        n = rnd.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 1000, 1023, 1024, 1025, 2047, 2049, 3000, 5000, 9000])
        V = rnd.choice([1, 2, 3, 7, 33, 100, 1000, 5000, 70000])
        C = rnd.choice([8, 16, 64, 200, 768, 1032])
        dt = rnd.choice([torch.bfloat16, torch.float32, torch.float16])
        kind = rnd.choice(["uniform", "hot", "sorted", "allsame", "padding"])
        g = torch.Generator().manual_seed(case)
        ids = torch.randint(0, V, (n,), generator=g)
        if kind == "hot":
            ids = torch.where(torch.rand(n, generator=g) < 0.7, torch.full((n,), V // 2), ids)
        elif kind == "sorted":
            ids = torch.sort(ids)[0]
        elif kind == "allsame":
            ids = torch.full((n,), V - 1, dtype=torch.int64)
        kw = dict(padding_idx=V // 3) if kind == "padding" else {}
        if rnd.random() < 0.3:
            ids = ids.to(torch.int32)
        dout = torch.randn((n, C), generator=g).to(dt)
        tag = f"case {case}: n={n} V={V} C={C} {dt} {kind}"
        rnd_base = None
        if rnd.random() < 0.3:
            base = rnd_base = torch.randn((V, C), generator=g).to(dt)
            got = dev(base).clone()
            ops.embedding_backward(dev(dout), dev(ids), V, dweight=got, **kw)
            want = co.embedding_backward(dout, ids, V, dweight=base, **kw)
        else:
            got = ops.embedding_backward(dev(dout), dev(ids), V, **kw)
            want = co.embedding_backward(dout, ids, V, **kw)
        # every output row is held to the bar its own terms justify (an fp32 sum of k terms of
        # size ~1 is good to ~1e-7 sqrt(k log k)), not to one constant for all shapes
        tol = scatter_sum_tolerance(dout, ids, V) + 1e-7
        if "padding_idx" in kw:
            tol[kw["padding_idx"]] = 0  # gets no gradient at all
        if rnd_base is not None:
            tol = tol + 2.0 ** -24 * rnd_base.double().abs()
        assert_sum_close(got, want, tol, name=tag)


def test_embedding_backward_hot_rows_on_the_general_path(ops, co):
    """Rows that are not whole 16-byte vectors take the one-thread-per-column kernel; three ids
    share 11830 tokens, so each sum has ~3900 terms and partial sums of ~60."""
    V, C, B, T = 32, 250, 13, 910
    ids = randint(0, 3, (B, T), 541510594, dtype=torch.int32)
    dout = randn((B, T, C), 541510595)
    dwte, dwpe = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_sum_close(dwte, co.embedding_backward(dout, ids, V), scatter_sum_tolerance(dout, ids, V) + 1e-7, name="dwte")
    assert_sum_close(dwpe, co.embedding_backward_positions(dout), sum_tolerance(dout) + 1e-7, name="dwpe")


@pytest.mark.parametrize("kind", ["uniform", "zipf"])
def test_embedding_config1(ops, co, kind):
    """Benchmark configuration 1: wte 50257x768, wpe 1024x768 bf16, B 8, T 1024."""
    V, C, B, T = 50257, 768, 8, 1024
    wte, wpe = randn((V, C), 1338, std=0.02, dtype=torch.bfloat16), randn((T, C), 1339, std=0.02, dtype=torch.bfloat16)
    ids = (randint(0, V, (B * T,), 100) if kind == "uniform" else zipf_ids(B * T, V, 101)).reshape(B, T)
    dout = randn((B, T, C), 102, dtype=torch.bfloat16)
    assert_bit_exact(ops.embedding_forward_add(dev(wte), dev(wpe), dev(ids)), co.embedding_forward_add(wte, wpe, ids),
                     "gather-add")
    dwte, dwpe = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_close(dwte, co.embedding_backward(dout, ids, V), atol=1e-6, name="dwte")
    assert_close(dwpe, co.embedding_backward_positions(dout), atol=1e-6, name="dwpe")
    again = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_bit_exact(again[0], dwte, "dwte rerun")
    # accumulate into existing gradients
    ops.embedding_backward_fused(dev(dout), dev(ids), V, dwte=again[0], dwpe=again[1])
    assert_close(again[1], co.embedding_backward_positions(dout, dwpe=dwpe.cpu()), atol=1e-6, name="dwpe +=")
    assert_close(again[0], co.embedding_backward(dout, ids, V, dweight=dwte.cpu()), atol=1e-6, name="dwte +=")
    assert_close(ops.embedding_backward_positions(dev(dout)), co.embedding_backward_positions(dout), atol=1e-6,
                 name="positions alone")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float64])
@pytest.mark.parametrize("B,T,C", [(1, 8, 64), (8, 128, 768), (16, 64, 1600), (40, 33, 128), (300, 5, 72), (7, 9, 35),
                                   (0, 4, 64)])
def test_embedding_positions_alone(ops, co, dtype, B, T, C):
    """cs_embedding_backward_positions on its own: whole 16-byte vectors take the vector kernel (the batch cut
    into slices of lanes when it is long), anything else the scalar one; `=` and `+=`; an empty batch gives zeros."""
    dout = randn((B, T, C), 300 + B + C, dtype=dtype)
    want = co.embedding_backward_positions(dout) if B > 0 else torch.zeros((T, C), dtype=dtype)
    got = ops.embedding_backward_positions(dev(dout))
    # sums over the batch: the bar comes from the terms (fp64 sums are held to 1e-12)
    tol = sum_tolerance(dout) if dtype != torch.float64 else torch.full((T, C), 1e-12, dtype=torch.float64)
    assert_sum_close(got, want, tol, name="dwpe")
    if B > 0:
        first = got.cpu().clone()
        ops.embedding_backward_positions(dev(dout), dwpe=got)
        assert_sum_close(got, co.embedding_backward_positions(dout, dwpe=first), tol, name="dwpe +=")
        assert_bit_exact(ops.embedding_backward_positions(dev(dout)), ops.embedding_backward_positions(dev(dout)), "rerun")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,C,V", [(17, 64, 64, 300), (40, 64, 128, 1000), (100, 32, 72, 50), (300, 16, 256, 5000),
                                     (64, 128, 768, 50257), (37, 700, 64, 900)])
def test_embedding_backward_fused_long_batches(ops, co, dtype, B, T, C, V):
    """Batches long enough that the position-table sum splits them over 2 .. 16 lanes per
    vector (also where the batch does not divide evenly), on the ranking path (B * T <= 8192)
    and the tile-sort path."""
    ids = randint(0, V, (B, T), 130)
    dout = randn((B, T, C), 131, dtype=dtype)
    atol = 1e-6 if dtype == torch.bfloat16 else 4e-5
    dwte, dwpe = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_close(dwpe, co.embedding_backward_positions(dout), atol=atol, name="dwpe")
    assert_close(dwte, co.embedding_backward(dout, ids, V), atol=atol, name="dwte")
    again = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_bit_exact(again[1], dwpe, "dwpe rerun")
    ops.embedding_backward_fused(dev(dout), dev(ids), V, dwte=again[0], dwpe=again[1])
    assert_close(again[1], co.embedding_backward_positions(dout, dwpe=dwpe.cpu()), atol=atol, name="dwpe +=")


# ---------------------------------------------------------- Cross entropy
@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_cross_entropy_reference_test_case(ops, co, reduction, dtype):
    # test/test_cross_entropy.cpp:69-99: x = rand [B*256, 384], targets randint [0,384); fewer rows here
    N, V = 4096, 384
    x = torch.rand((N, V), generator=torch.Generator().manual_seed(1)).to(dtype)
    t = randint(0, V, (N,), 110)
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), reduction=reduction)
    loss2, row2, d2, tw2 = co.cross_entropy(x, t, reduction=reduction)
    assert_close(loss.double(), loss2.double(), atol=1e-5 if reduction != "sum" else 1e-1, name="loss")
    assert_close(row.double(), row2.double(), atol=2e-6, name="row loss")
    assert_close(d, d2, atol=1e-9 if reduction == "mean" else 1e-7, name="dlogits")
    assert tw.item() == tw2.item() == N


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("N,V,stride", [(64, 50257, 50304), (8, 50304, 50304), (33, 1000, 1024), (16, 4000, 4096),
                                        (5, 16385, 16392), (7, 100, 100), (3, 130000, 130048), (4, 77, 77),
                                        (40, 50257, 50257), (600, 1001, 1003), (3, 70001, 70001), (33, 1000, 1003),
                                        (5, 3, 3), (9, 1, 1), (6, 13, 17), (300, 32000, 32000), (260, 20000, 20008)])
def test_cross_entropy_shapes(ops, co, dtype, N, V, stride):
    x = randn((N, stride), 111, std=2.0, dtype=dtype)
    t = randint(0, V, (N,), 112)
    if N > 4:
        t[1] = -100  # an ignored row
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), V)
    loss2, row2, d2, tw2 = co.cross_entropy(x, t, V)
    assert_close(loss, loss2.float(), atol=1e-5, name="loss")
    assert_close(row, row2.float(), atol=1e-5, name="row loss")
    # softmax entries are ~1/V/N: a relative bar with a floor far below them.  With a handful of
    # columns p approaches 1 and (p - 1)/N is a cancellation: it is known to an ulp of the fp32 1/N
    assert_close(d, d2, atol=1e-10 if V >= 64 else 1.2e-7 / N, name="dlogits")
    assert (d[:, V:] == 0).all()
    assert tw.item() == tw2.item()


def test_cross_entropy_inplace_amp_and_dloss(ops, co):
    N, V, stride = 48, 50257, 50304
    x = randn((N, stride), 113, std=2.0, dtype=torch.bfloat16)
    t = randint(0, V, (N,), 114)
    _, _, d2, _ = co.cross_entropy(x, t, V)
    gx = dev(x)
    loss, row, d, _ = ops.fused_classifier(gx, dev(t), V, inplace=True)
    assert d.data_ptr() == gx.data_ptr()
    assert_close(gx, d2, atol=1e-10, name="in-place dlogits")
    # fp32 gradient from bf16 logits (the autocast rule, test/test_cross_entropy.cpp:102-139)
    _, _, d32, _ = ops.fused_classifier(dev(x), dev(t), V, dlogits_dtype=torch.float32)
    _, _, d32o, _ = co.cross_entropy(x, t, V, dlogits_dtype=torch.float32)
    assert_close(d32, d32o, atol=1e-10, name="fp32 dlogits")
    # upstream gradient, negative too; loss only
    for dloss in (0.25, -3.0, 0.0):
        _, _, dd, _ = ops.fused_classifier(dev(x), dev(t), V, dloss=dloss, dlogits_dtype=torch.float32)
        assert_close(dd, (d32o.double() * dloss).float(), atol=1e-10, name=f"dloss {dloss}")
    loss3, _, none, _ = ops.fused_classifier(dev(x), dev(t), V, want_dlogits=False)
    assert none is None and loss3.item() == loss.item()


@pytest.mark.parametrize("N,V,stride", [(300, 50257, 50304), (270, 59990, 60000), (5, 65536, 65536),
                                        (530, 50257, 50257), (70, 999, 1001)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_cross_entropy_autocast_wide_rows(ops, co, N, V, stride, dtype):
    """16-bit logits with fp32 gradients on the streaming kernel's register plan and the
    two-sweep kernel, with more rows than workgroups (so rows are prefetched) and ignored rows
    among them."""
    x = randn((N, stride), 116, std=2.0, dtype=dtype)
    t = randint(0, V, (N,), 117)
    t[1] = -100
    t[N - 1] = -100
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), V, dlogits_dtype=torch.float32)
    loss2, row2, d2, tw2 = co.cross_entropy(x, t, V, dlogits_dtype=torch.float32)
    assert d.dtype == torch.float32 and tw.item() == tw2.item() == N - 2
    assert_close(loss, loss2.float(), atol=1e-5, name="loss")
    assert_close(row, row2.float(), atol=1e-5, name="row loss")
    assert_close(d, d2, atol=1e-10, name="dlogits")
    assert (d[:, V:] == 0).all() and (d[1] == 0).all()


@pytest.mark.parametrize("N,V,stride,dtype,gdt", [(600, 17, 64, torch.bfloat16, torch.float32),
                                                   (64, 1000, 1024, torch.float32, None),
                                                   (300, 50257, 50304, torch.bfloat16, None),
                                                   (300, 50257, 50304, torch.bfloat16, torch.float32),
                                                   (16, 100000, 100000, torch.bfloat16, None),
                                                   (16, 100000, 100000, torch.bfloat16, torch.float32),
                                                   (6, 70001, 70004, torch.float32, None)])
def test_cross_entropy_confident_predictions(ops, co, N, V, stride, dtype, gdt):
    """Targets the model is nearly sure of: p close to 1 makes (p - 1) a cancellation, so a
    relative error of 1e-6 in p (what folding the normalisation into one exponent costs) would
    show as 1e-5 .. 1e-4 in the gradient at the target column."""
    x = randn((N, stride), 118, std=2.0, dtype=dtype)
    t = randint(0, V, (N,), 119)
    boost = torch.linspace(8.0, 20.0, N)  # p_target from ~0.9 to 1 - 1e-6
    x[torch.arange(N), t] = (x[torch.arange(N), t].float() + boost).to(dtype)
    kw = dict(dlogits_dtype=gdt) if gdt else {}
    loss, row, d, _ = ops.fused_classifier(dev(x), dev(t), V, **kw)
    loss2, row2, d2, _ = co.cross_entropy(x, t, V, **kw)
    assert_close(row, row2.float(), atol=1e-6, name="row loss")
    if d.dtype == torch.float32:
        at_target = d[torch.arange(N), dev(t)].cpu()
        want = d2[torch.arange(N), t]
        # p itself is an fp32 number next to 1: a handful of units in its last place (6e-8 each: the hardware exp2, the sum, the quotient), times 1/N,
        # is what (p - 1)/N can be known to; the relative bar covers everything above that
        excess = (at_target - want).abs() - (1e-5 * want.abs() + 5e-7 / N)
        worst = int(excess.argmax())
        assert excess[worst] <= 0, (f"gradient at the target column: row {worst} got {at_target[worst].item():.6e} "
                                    f"want {want[worst].item():.6e}")
    assert_close(d, d2, atol=5e-7 / N if d.dtype == torch.float32 else 1e-10, name="dlogits")


@pytest.mark.parametrize("N,V,stride,dtype,gdt", [(600, 66000, 66048, torch.bfloat16, None),
                                                   (530, 65537, 65544, torch.bfloat16, torch.float32),
                                                   (40, 128256, 128256, torch.float16, None),
                                                   (9, 151936, 151936, torch.bfloat16, torch.float32),
                                                   (5, 300000, 300000, torch.float32, None),
                                                   (3, 65540, 65540, torch.float32, None)])
def test_cross_entropy_rows_beyond_registers(ops, co, N, V, stride, dtype, gdt):
    """Vocabularies past 65536 columns (16 bit) run the two-sweep kernel: more rows than
    workgroups, ignored rows, padding columns, a target in the last column and in the first."""
    x = randn((N, stride), 120, std=2.0, dtype=dtype)
    t = randint(0, V, (N,), 121)
    t[0], t[2], t[N - 2], t[N - 1] = V - 1, 0, -100, V - 1
    kw = dict(dlogits_dtype=gdt) if gdt else {}
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), V, **kw)
    loss2, row2, d2, tw2 = co.cross_entropy(x, t, V, **kw)
    assert tw.item() == tw2.item() == N - 1
    assert_close(loss, loss2.float(), atol=1e-5, name="loss")
    assert_close(row, row2.float(), atol=1e-5, name="row loss")
    assert_close(d, d2, atol=1e-10, name="dlogits")
    assert (d[:, V:] == 0).all() and (d[N - 2] == 0).all()
    # in place, and loss only
    gx = dev(x)
    if not gdt:
        ops.fused_classifier(gx, dev(t), V, inplace=True)
        assert_bit_exact(gx, d, "in place")
    loss3, _, none, _ = ops.fused_classifier(dev(x), dev(t), V, want_dlogits=False)
    assert none is None and loss3.item() == loss.item()


@pytest.mark.parametrize("N,V,stride,dtype,gdt", [(6, 50257, 50304, torch.bfloat16, None),
                                                   (6, 50257, 50304, torch.bfloat16, torch.float32),
                                                   (6, 50257, 50304, torch.float32, None),
                                                   (6, 1000, 1024, torch.float32, None),
                                                   (6, 70000, 70000, torch.bfloat16, None),
                                                   (6, 50257, 50257, torch.float16, None),
                                                   (6, 301, 301, torch.float64, None)])
def test_cross_entropy_masked_vocabulary(ops, co, N, V, stride, dtype, gdt):
    """Logits masked with -inf, as when the vocabulary is restricted: whole lanes, waves and
    vectors without a finite value, next to finite logits far below zero (their exponentials
    relative to 0 would underflow) or of ordinary size."""
    x = torch.full((N, stride), float("-inf"), dtype=dtype)
    g = torch.Generator().manual_seed(122)
    keep = [slice(0, 100), slice(V - 37, V), slice(V // 2, V // 2 + 3), slice(5, 6), slice(0, V, 97), slice(0, V)]
    level = [-60.0, -60.0, 50.0, 0.0, -60.0, 0.0]
    t = torch.zeros(N, dtype=torch.int64)
    for r in range(N):
        cols = torch.arange(V)[keep[r]]
        x[r, cols] = (torch.randn(len(cols), generator=g) * 2 + level[r]).to(dtype)
        t[r] = cols[len(cols) // 2]
    x[N - 1, 17:min(4000, V // 3)] = float("-inf")  # a hole in an otherwise ordinary row, clear of its target
    kw = dict(dlogits_dtype=gdt) if gdt else {}
    loss, row, d, _ = ops.fused_classifier(dev(x), dev(t), V, **kw)
    loss2, row2, d2, _ = co.cross_entropy(x, t, V, **kw)
    assert torch.isfinite(row).all() and torch.isfinite(d.float()).all()
    assert_close(row, row2.to(row.dtype), atol=1e-5, name="row loss")
    assert_close(loss, loss2.to(loss.dtype), atol=1e-5, name="loss")
    assert_close(d, d2, atol=1.2e-7 / N, name="dlogits")
    assert (d[x.isinf().to(d.device)] == 0).all()


def test_cross_entropy_all_ignored_and_bad_targets(ops):
    x = randn((6, 128), 115, dtype=torch.bfloat16)
    t = torch.full((6,), -100, dtype=torch.int64)
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t), 100)
    assert math.isnan(loss.item()) and tw.item() == 0 and (row == 0).all() and (d == 0).all()  # mean over nothing
    t2 = torch.tensor([0, 99, 100, 5000, -7, 3], dtype=torch.int64)  # out-of-range targets count as ignored
    loss, row, d, tw = ops.fused_classifier(dev(x), dev(t2), 100)
    assert tw.item() == 3 and (row[2:5] == 0).all() and (d[2:5] == 0).all() and math.isfinite(loss.item())


def test_cross_entropy_config2_full_size(ops, co):
    """Benchmark configuration 2: [8192, 50257] bf16, stride 50304, in place."""
    N, V, stride = 8192, 50257, 50304
    x = randn((N, stride), 1339, std=2.0, dtype=torch.bfloat16)
    t = randint(0, V, (N,), 1340)
    gx = dev(x)
    loss, row, d, tw = ops.fused_classifier(gx, dev(t), V, inplace=True)
    assert tw.item() == N
    # size-independent properties
    assert (gx[:, V:] == 0).all()
    sums = gx[:, :V].float().sum(1)
    assert sums.abs().max().item() < 2e-6  # (softmax - onehot)/N sums to 0 up to bf16 rounding of 50257 terms
    assert abs(loss.item() - row.double().mean().item()) < 1e-5
    assert (gx[torch.arange(N), dev(t)] < 0).all()  # p - 1 < 0 at the target
    # the oracle on a sample of rows; dlogits of a row depends on the others only through 1/N
    pick = torch.arange(0, N, 171)
    _, row2, d2, _ = co.cross_entropy(x[pick], t[pick], V, reduction="sum", dloss=1.0 / N)
    assert_close(row[pick], row2.float(), atol=1e-5, name="row loss sample")
    assert_close(gx[pick], d2, atol=1e-10, name="dlogits sample")


# ------------------------------------------------ configuration 4: GPT-2-XL scale
def test_xl_cross_entropy(ops, co):
    """[16384, 50257] bf16, stride 50304: size-independent properties + the oracle on a sample of rows."""
    N, V, stride = 16384, 50257, 50304
    g = torch.Generator(device=DEV).manual_seed(1341)
    gx = (torch.randn((N, stride), generator=g, device=DEV) * 2.0).to(torch.bfloat16)
    t = randint(0, V, (N,), 1342)
    pick = torch.arange(0, N, 331)
    x_pick = gx[pick].cpu()
    loss, row, d, tw = ops.fused_classifier(gx, dev(t), V, inplace=True)
    assert tw.item() == N
    assert (gx[:, V:] == 0).all()
    assert gx[:, :V].float().sum(1).abs().max().item() < 2e-6
    assert abs(loss.item() - row.double().mean().item()) < 1e-5
    assert (gx[torch.arange(N), dev(t)] < 0).all()
    _, row2, d2, _ = co.cross_entropy(x_pick, t[pick], V, reduction="sum", dloss=1.0 / N)
    assert_close(row[pick], row2.float(), atol=1e-5, name="row loss sample")
    assert_close(gx[pick], d2, atol=1e-10, name="dlogits sample")


def test_xl_embedding(ops, co):
    """wte 50257x1600, wpe 1024x1600 bf16, B 16, T 1024, Zipf ids: the whole case against the oracle."""
    V, C, B, T = 50257, 1600, 16, 1024
    wte, wpe = randn((V, C), 1343, std=0.02, dtype=torch.bfloat16), randn((T, C), 1344, std=0.02, dtype=torch.bfloat16)
    ids = zipf_ids(B * T, V, 1345).reshape(B, T)
    dout = randn((B, T, C), 1346, dtype=torch.bfloat16)
    assert_bit_exact(ops.embedding_forward_add(dev(wte), dev(wpe), dev(ids)), co.embedding_forward_add(wte, wpe, ids),
                     "gather-add")
    dwte, dwpe = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_close(dwte, co.embedding_backward(dout, ids, V), atol=1e-6, name="dwte")
    assert_close(dwpe, co.embedding_backward_positions(dout), atol=1e-6, name="dwpe")
    # column sums of the dense gradient equal column sums of dout (nothing dropped, nothing doubled)
    want = dout.double().sum((0, 1))
    got = dwte.double().sum(0).cpu()
    assert (got - want).abs().max().item() < 0.05 * B * T ** 0.5  # bf16 rounding of each output row
    untouched = torch.ones(V, dtype=torch.bool)
    untouched[ids.flatten()] = False
    assert (dwte[dev(untouched)] == 0).all()
    again = ops.embedding_backward_fused(dev(dout), dev(ids), V)
    assert_bit_exact(again[0], dwte, "dwte rerun")


def test_xl_layernorm(ops, co):
    """[16384, 1600] bf16 with fp32 parameters: forward and backward against the oracle."""
    _ln_case(ops, co, 16384, 1600, torch.bfloat16, torch.float32)


def test_xl_adamw(ops, co):
    """All 580 GPT-2-XL tensors (1,557,611,200 fp32 parameters) in one launch, two steps; the oracle
    runs on a sample of tensors (the largest, the smallest, some from the middle and the last)."""
    shapes = gpt2_param_shapes(48, 1600)
    sizes = [math.prod(s) for s in shapes]
    total = sum(sizes)
    assert len(shapes) == 580 and total == 1_557_611_200
    g = torch.Generator(device=DEV).manual_seed(1347)
    w = torch.empty(total, device=DEV).normal_(0, 0.02, generator=g)
    grad = torch.empty(total, device=DEV).normal_(0, 1e-3, generator=g)
    offs = [0]
    for s in sizes:
        offs.append(offs[-1] + s)
    sample = [0, 1, 2, 4, 5, 300, 301, 575, 578, 579]
    w0 = {i: w[offs[i]:offs[i + 1]].cpu() for i in sample}
    grads = []
    opt = ops.MultiTensorAdamW([w[offs[i]:offs[i + 1]] for i in range(len(sizes))],
                               [grad[offs[i]:offs[i + 1]] for i in range(len(sizes))], t=0, **HYPER)
    for step in range(2):
        if step == 1:
            grad.normal_(0, 1e-3, generator=g)
        grads.append({i: grad[offs[i]:offs[i + 1]].cpu() for i in sample})
        opt.step()
    for i in sample:
        ww, m, v = w0[i], torch.zeros(sizes[i]), torch.zeros(sizes[i])
        for t in (1, 2):
            ww, m, v, _ = co.adamw_step(ww, grads[t - 1][i], m, v, t=t, **HYPER)
        assert_close(w[offs[i]:offs[i + 1]], ww, atol=1e-8, name=f"w[{i}]")
        assert_close(opt.m[i].flatten(), m, atol=1e-10, name=f"m[{i}]")
        assert_close(opt.v[i].flatten(), v, atol=1e-13, name=f"v[{i}]")
    # no element outside the sample was skipped: after two steps from m = 0 with these hyper-parameters
    # every first moment is non-zero wherever the gradients are, and they are everywhere
    m_all = torch.cat([x.flatten() for x in opt.m[3:4]])
    assert (m_all != 0).all()
    del opt, w, grad
    torch.cuda.empty_cache()


# ------------------------------------------------ more than 2^31 elements per tensor
# Element offsets past 2^31 (and byte offsets past 2^32) in every kernel family; the oracle runs
# on slices taken from the start, the middle and the very end.
BIG = 2**31 + 2**20 + 24


def _gpu_randn(shape, seed, dtype, std=1.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    out = torch.empty(shape, dtype=dtype, device=DEV)
    rows = shape[0]
    step = max(1, rows // 8)
    for r0 in range(0, rows, step):  # in pieces: the fp32 staging buffer stays small
        piece = out[r0:r0 + step]
        piece.copy_(torch.randn(piece.shape, generator=g, device=DEV) * std)
    return out


def test_big_gelu(ops, co):
    x = _gpu_randn((BIG,), 1401, torch.bfloat16, 1.5)
    dy = _gpu_randn((BIG,), 1402, torch.bfloat16)
    y = ops.gelu_forward(x, "tanh")
    dx = ops.gelu_backward(dy, x, "tanh")
    for a in (0, 2**31 - 4096, BIG - 5000):
        sl = slice(a, a + 5000)
        assert_close(y[sl], co.gelu_forward(x[sl].cpu(), "tanh"), atol=1e-6, name=f"y[{a}:]")
        assert_close(dx[sl], co.gelu_backward(dy[sl].cpu(), x[sl].cpu(), "tanh"), atol=1e-6, name=f"dx[{a}:]")
    del x, dy, y, dx
    torch.cuda.empty_cache()


def test_big_layernorm(ops, co):
    C = 1600
    rows = BIG // C + 7
    x = _gpu_randn((rows, C), 1403, torch.bfloat16)
    dy = _gpu_randn((rows, C), 1404, torch.bfloat16)
    gamma, beta = randn((C,), 1405, mean=1.0, std=0.02), randn((C,), 1406, std=0.02)
    y, mean, rstd = ops.layernorm_forward(x, dev(gamma), dev(beta))
    dx, dgamma, dbeta = ops.layernorm_backward(dy, x, mean, rstd, dev(gamma))
    for a in (0, rows // 2, rows - 300):
        sl = slice(a, a + 300)
        y2, mean2, rstd2 = co.layernorm_forward(x[sl].cpu(), gamma, beta)
        assert_close(y[sl], y2, atol=1e-6, name=f"y[{a}:]")
        assert_close(mean[sl], mean2.flatten(), atol=1e-6, name=f"mean[{a}:]")
        dx2, _, _ = co.layernorm_backward(dy[sl].cpu(), x[sl].cpu(), mean2, rstd2, gamma)
        assert_close(dx[sl], dx2, atol=1e-6, name=f"dx[{a}:]")
    # dbeta is the column sum of dy over all rows: ~N(0, rows), so the fp32 sum of `rows` terms is good
    # to a few e-4 of its spread; torch's own column sum (fp32 tree over the same data) as the check
    want = dy.float().sum(0)
    assert (dbeta - want).abs().max().item() < 2e-3 * math.sqrt(rows)
    del x, dy, y, dx
    torch.cuda.empty_cache()


def test_big_cross_entropy(ops, co):
    V, stride = 50257, 50304
    N = BIG // stride + 3
    gx = _gpu_randn((N, stride), 1407, torch.bfloat16, 2.0)
    t = randint(0, V, (N,), 1408)
    t[5] = -100
    pick = torch.tensor([0, 1, 5, N // 2, 2**31 // stride, 2**31 // stride + 1, N - 2, N - 1])
    x_pick = gx[pick.to(DEV)].cpu()
    loss, row, d, tw = ops.fused_classifier(gx, dev(t), V, inplace=True)
    assert tw.item() == N - 1
    assert abs(loss.item() - row.double().sum().item() / (N - 1)) < 1e-5
    _, row2, d2, _ = co.cross_entropy(x_pick, t[pick], V, reduction="sum", dloss=1.0 / (N - 1))
    assert_close(row[pick.to(DEV)], row2.float(), atol=1e-5, name="row loss sample")
    assert_close(gx[pick.to(DEV)], d2, atol=1e-10, name="dlogits sample")
    del gx
    torch.cuda.empty_cache()


def test_big_embedding(ops, co):
    V, C = 50257, 1600
    n = BIG // C + 5  # tokens
    ids = randint(0, V, (n,), 1409)
    w = _gpu_randn((V, C), 1410, torch.bfloat16, 0.02)
    out = ops.embedding_forward(w, dev(ids))
    w_cpu = w.cpu()
    for a in (0, n // 2, n - 400):
        sl = slice(a, a + 400)
        assert_bit_exact(out[sl], co.embedding_forward(w_cpu, ids[sl]), f"rows {a}:")
    # backward over the same number of tokens: every row of the table collects ~27 of them
    dwte = ops.embedding_backward(out, dev(ids), V)
    rows = torch.tensor([0, 17, V // 2, V - 1])
    for r in rows.tolist():
        hits = (ids == r).sum().item()
        want = w_cpu[r].float() * hits  # out[i] == w[ids[i]], so row r of the gradient is hits * w[r]
        assert_close(dwte[r].float().cpu(), want, atol=4e-4 * hits, name=f"dwte[{r}] ({hits} tokens)")  # one bf16 ulp at 0.1 * hits
    del out, dwte, w
    torch.cuda.empty_cache()


def test_big_adamw(ops, co):
    n = BIG
    g = torch.Generator(device=DEV).manual_seed(1411)
    w = torch.empty(n, device=DEV).normal_(0, 0.02, generator=g)
    grad = torch.empty(n, device=DEV).normal_(0, 1e-3, generator=g)
    m, v = torch.zeros(n, device=DEV), torch.zeros(n, device=DEV)
    cuts = (0, 2**31 - 3000, n - 5000)
    w0 = {a: w[a:a + 5000].cpu() for a in cuts}
    ops.adamw_step(w, grad, m, v, t=1, **HYPER)
    for a in cuts:
        sl = slice(a, a + 5000)
        ww, mm, vv, _ = co.adamw_step(w0[a], grad[sl].cpu(), torch.zeros(5000), torch.zeros(5000), t=1, **HYPER)
        assert_close(w[sl], ww, atol=1e-8, name=f"w[{a}:]")
        assert_close(m[sl], mm, atol=1e-10, name=f"m[{a}:]")
        assert_close(v[sl], vv, atol=1e-13, name=f"v[{a}:]")
    # one tensor of the multi-tensor launch past 2^31 elements as well
    opt = ops.MultiTensorAdamW([w[:1000], w[1000:]], [grad[:1000], grad[1000:]], t=0, **HYPER)
    w1 = {a: w[a:a + 5000].cpu() for a in cuts}
    opt.step()
    for a in cuts[1:]:
        sl = slice(a, a + 5000)
        ww, _, _, _ = co.adamw_step(w1[a], grad[sl].cpu(), torch.zeros(5000), torch.zeros(5000), t=1, **HYPER)
        assert_close(w[sl], ww, atol=1e-8, name=f"multi w[{a}:]")
    del opt, w, grad, m, v
    torch.cuda.empty_cache()


# ------------------------------------------------------------- empty inputs
def test_empty_inputs(ops, co):
    """Zero rows / tokens / elements: every call returns without launching anything harmful and
    leaves well-defined outputs (an embedding gradient for no tokens is all zeros)."""
    z = torch.empty((0, 768), dtype=torch.bfloat16, device=DEV)
    gamma, beta = torch.ones(768, device=DEV), torch.zeros(768, device=DEV)
    y, mean, rstd = ops.layernorm_forward(z, gamma, beta)
    assert y.shape == (0, 768) and mean.numel() == 0
    dx, dg, db = ops.layernorm_backward(z, z, mean, rstd, gamma)
    assert dx.shape == (0, 768)
    assert ops.gelu_forward(z).shape == (0, 768) and ops.gelu_backward(z, z).shape == (0, 768)
    # embedding: no tokens -> an empty activation, a zero gradient (and an untouched one when accumulating)
    wte = randn((50, 16), 1, dtype=torch.bfloat16)
    ids = torch.empty((0, 8), dtype=torch.int64, device=DEV)
    assert ops.embedding_forward(dev(wte), ids).shape == (0, 8, 16)
    dw = ops.embedding_backward(torch.empty((0, 8, 16), dtype=torch.bfloat16, device=DEV), ids, 50)
    assert dw.shape == (50, 16) and (dw == 0).all()
    keep = dev(wte).clone()
    ops.embedding_backward(torch.empty((0, 8, 16), dtype=torch.bfloat16, device=DEV), ids, 50, dweight=keep)
    assert_bit_exact(keep, wte, "accumulating nothing")
    # AdamW: an empty tensor alone, and one among others in the multi-tensor table
    e = torch.empty(0, device=DEV)
    ops.adamw_step(e, e, e, e, t=1, **HYPER)
    ws = [randn((5,), 2), torch.empty(0), randn((4097,), 3)]
    gs = [randn((5,), 4), torch.empty(0), randn((4097,), 5)]
    gws = [dev(w) for w in ws]
    opt = ops.MultiTensorAdamW(gws, [dev(g) for g in gs], t=0, **HYPER)
    opt.step()
    for i in (0, 2):
        w2, _, _, _ = co.adamw_step(ws[i], gs[i], torch.zeros_like(ws[i]), torch.zeros_like(ws[i]), t=1, **HYPER)
        assert_close(gws[i], w2, atol=1e-8, name=f"w[{i}]")
    # cross entropy over no rows: sum is 0, mean is 0/0
    x = torch.empty((0, 128), dtype=torch.bfloat16, device=DEV)
    t = torch.empty((0,), dtype=torch.int64, device=DEV)
    loss, row, d, tw = ops.fused_classifier(x, t, 100, reduction="sum")
    assert loss.item() == 0 and tw.item() == 0 and d.shape == (0, 128)
    loss, _, _, _ = ops.fused_classifier(x, t, 100)
    assert math.isnan(loss.item())


# ------------------------------------------------------------ calibration kernels
@pytest.mark.gpu
@pytest.mark.parametrize("nbytes", [16, 4096 * 3 + 16, (64 << 20) + 48])
def test_stream_copy_read_fill(nbytes):
    """The benchmark's calibration kernels move exactly the bytes they are asked to."""
    import ctypes

    from core_scheduler_amd import _capi

    lib = _capi.load()
    dev = torch.device("cuda:0")
    P = ctypes.c_void_p
    st = P(torch.cuda.current_stream(dev).cuda_stream)
    g = torch.Generator(device="cpu").manual_seed(nbytes)
    src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g).to(dev)
    dst = torch.zeros(nbytes + 64, dtype=torch.uint8, device=dev)
    _capi.check("cs_stream_copy", lib.cs_stream_copy(P(dst.data_ptr()), P(src.data_ptr()), nbytes, st))
    assert torch.equal(dst[:nbytes], src) and int(dst[nbytes:].sum()) == 0
    words = lib.cs_stream_read_out_words(nbytes)
    out = torch.zeros(words, dtype=torch.int32, device=dev)
    _capi.check("cs_stream_read", lib.cs_stream_read(P(src.data_ptr()), P(out.data_ptr()), nbytes, st))
    want = 0
    for w in src.cpu().numpy().view("<u4").tolist():
        want ^= w
    got = 0
    for w in out.cpu().numpy().view("<u4").tolist():
        got ^= w
    assert got == want, "the read pass saw other bytes than the buffer holds"
    _capi.check("cs_stream_fill", lib.cs_stream_fill(P(dst.data_ptr()), nbytes, 0x01020304, st))
    torch.cuda.synchronize()
    assert int(dst[nbytes:].sum()) == 0
    assert bool((dst[:nbytes].view(torch.int32) == 0x01020304).all())
    # four arrays in, three rewritten: a_k = (a0 ^ a1 ^ a2 ^ a3) + k per 32-bit word
    arrs = [torch.randint(0, 256, (nbytes + 16,), dtype=torch.uint8, generator=g) for _ in range(4)]
    gpu = [a.to(dev) for a in arrs]
    _capi.check("cs_stream_update4", lib.cs_stream_update4(*[P(a.data_ptr()) for a in gpu], nbytes, st))
    words = [a[:nbytes].numpy().view("<u4").astype("uint32") for a in arrs]
    x = words[0] ^ words[1] ^ words[2] ^ words[3]
    assert torch.equal(gpu[0].cpu(), arrs[0])
    for k in (1, 2, 3):
        got = gpu[k].cpu()
        assert (got[:nbytes].numpy().view("<u4") == x + np.uint32(k)).all(), f"array {k}"
        assert torch.equal(got[nbytes:], arrs[k][nbytes:]), "wrote past the end"
