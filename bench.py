#!/usr/bin/env python3
"""Benchmark of the GPT-2 training kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one fused-classifier call (row softmax + cross-entropy + in-place
dlogits) on logits [8192, 50257] bf16 with row stride 50304 - the
configuration the headline metric is quoted on.  W untimed steps, then exactly
K timed steps between device synchronisations; one JSON line on stdout.

The same line carries
  roofline      the dominant kernel (the row pass) against the 8 TB/s HBM peak,
                its duration measured with HIP events inside the timed region
  per_op        every op of the hot path at its benchmark configuration, one
                short record each (op, cfg, ms and fraction of the HBM peak per
                call on cold buffers).  The full table goes to stderr as one
                JSON line after "[bench-full]" (and to --full-json PATH): ms,
                GB/s of algorithmic bytes and fraction of the HBM peak, warm
                (same buffers) and cold (inputs and outputs rotated over
                > 600 MB so the 256 MB Infinity Cache cannot serve them), each
                the duration of one call inside a batch of back-to-back calls
                between one pair of events, and three calibration kernels
                (plain copy, read only, write only).  The stdout line stays
                under 8000 bytes
  cpu_baseline  the reference's own op sequence on the ATen CPU backend
                (oracle/aten_port.py), timed here on this box's host cores

Inputs are synthetic (seeded normal logits, uniform targets) and resident in
HBM before the timed region starts.  This build is single-GPU: --gpus above 1
is refused.
"""
import argparse
import ctypes
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth

# benchmark configuration 2
CE_N, CE_V, CE_STRIDE = 8192, 50257, 50304
# algorithmic bytes per fused-classifier call: read the class columns of the logits once and
# write them once (bf16), read the int64 targets, write fp32 row losses and the mean
CE_BYTES = 2 * CE_N * CE_V * 2 + CE_N * 8 + CE_N * 4 + 4
CE_ROWS_TRAFFIC_BYTES = 1_649_121_000  # measured with rocprofv3 --pmc (profiles/ce_rows_stream_kernel_hbm_traffic_pmc.txt)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gpt2_param_sizes(n_layer, C, V=50257, T=1024):
    sizes = [V * C, T * C]
    for _ in range(n_layer):
        sizes += [C, C, C * 3 * C, 3 * C, C * C, C, C, C, C * 4 * C, 4 * C, 4 * C * C, C]
    return sizes + [C, C]


_BLOCKER = {}


def hold_gpu(torch, ms=6.0):
    """Queues ~`ms` of plain copies so that the launches that follow are all enqueued while the
    GPU is still busy: the timed calls then run back to back, as they do inside a training step,
    instead of each waiting for the host to issue it."""
    from core_scheduler_amd import _capi

    if "buf" not in _BLOCKER:
        _BLOCKER["buf"] = (torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0"),
                           torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0"))
    a, b = _BLOCKER["buf"]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(max(1, int(ms / 0.35))):  # 1 GiB each way takes ~0.35 ms
        _capi.load().cs_stream_copy(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()), 1 << 30, st)


def _capi_lib():
    from core_scheduler_amd import _capi

    return _capi.load()


def event_ms(fn, reps, torch, rounds=3):
    """Duration of one call when `reps` calls run back to back: one pair of events around the
    whole batch (no event, hence no gap, between the calls), median over `rounds` batches.  Also
    returns the median of per-call event pairs, which carries the events' own cost (~3 us)."""
    batch = []
    for _ in range(rounds):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        hold_gpu(torch)
        e0.record()
        for i in range(reps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        batch.append(e0.elapsed_time(e1) / reps)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    torch.cuda.synchronize()
    hold_gpu(torch)
    for i in range(reps):
        starts[i].record()
        fn(i)
        ends[i].record()
    torch.cuda.synchronize()
    per_call = statistics.median(s.elapsed_time(e) for s, e in zip(starts, ends))
    return statistics.median(batch), per_call


class HipTimer:
    """HIP events made with hipEventDisableSystemFence, the flag the runtime offers for events that
    only measure time: recording one does not flush and invalidate the caches around the kernel it
    brackets (a default event costs the stream ~2.7 us per record here, a fence-free one ~0.9 us)."""

    _hip = None
    FLAGS = 0x20000000  # hipEventDisableSystemFence; timing stays enabled

    @classmethod
    def hip(cls):
        if cls._hip is None:
            h = ctypes.CDLL("libamdhip64.so")
            h.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
            h.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
            h.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
            h.hipEventDestroy.argtypes = [ctypes.c_void_p]
            cls._hip = h
        return cls._hip

    def __init__(self):
        self.ev = ctypes.c_void_p()
        rc = self.hip().hipEventCreateWithFlags(ctypes.byref(self.ev), self.FLAGS)
        if rc != 0:
            raise RuntimeError(f"hipEventCreateWithFlags failed: {rc}")

    def record(self, stream):
        rc = self.hip().hipEventRecord(self.ev, stream)
        if rc != 0:
            raise RuntimeError(f"hipEventRecord failed: {rc}")

    def ms_until(self, other):
        out = ctypes.c_float()
        rc = self.hip().hipEventElapsedTime(ctypes.byref(out), self.ev, other.ev)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return out.value

    def __del__(self):
        if self.ev:
            self.hip().hipEventDestroy(self.ev)


def run_headline(args, torch, ops, capi):
    dev = torch.device("cuda:0")
    lib = capi.load()
    K, W = args.steps, args.warmup
    n_buf = min(K + W, args.max_buffers)
    g = torch.Generator(device=dev)
    g.manual_seed(1337 + 2)
    master = (torch.randn((CE_N, CE_STRIDE), generator=g, device=dev, dtype=torch.float32) * 2.0).to(torch.bfloat16)
    targets = torch.randint(0, CE_V, (CE_N,), generator=g, device=dev, dtype=torch.int64)
    bufs = [master.clone() for _ in range(n_buf)]
    row_loss = torch.empty(CE_N, dtype=torch.float32, device=dev)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    tw = torch.empty((), dtype=torch.float32, device=dev)
    ws_bytes = lib.cs_fused_classifier_workspace_bytes(CE_N)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    P = ctypes.c_void_p

    def phase(buf, which):
        code = lib.cs_fused_classifier_phases(P(buf.data_ptr()), P(buf.data_ptr()), P(targets.data_ptr()),
                                              P(row_loss.data_ptr()), P(loss.data_ptr()), P(tw.data_ptr()),
                                              P(ws.data_ptr()), ws_bytes, CE_N, CE_V, CE_STRIDE, -100, capi.REDUCTION_MEAN,
                                              1.0, capi.BF16, capi.BF16, which, stream)
        capi.check("cs_fused_classifier_phases", code)

    def step(i, ev=None):
        buf = bufs[i % n_buf]
        phase(buf, 1)
        if ev:
            ev[0].record(stream)
        phase(buf, 2)
        if ev:
            ev[1].record(stream)
        phase(buf, 4)

    for i in range(W):
        step(i)
    evs = [(HipTimer(), HipTimer()) for _ in range(K)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        step(W + i, evs[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kernel_ms = [a.ms_until(b) for a, b in evs]
    first_loss = loss.item()
    reused = K + W > n_buf
    return {
        "seconds": t1 - t0,
        "ms_per_step": (t1 - t0) / K * 1e3,
        "rows_kernel_ms_avg": sum(kernel_ms) / K,
        "rows_kernel_ms_median": statistics.median(kernel_ms),
        "loss": first_loss,
        "buffers": n_buf,
        "buffers_reused": reused,
    }


def per_op_table(args, torch, ops):
    """Every op at its benchmark configuration; returns a list of dicts."""
    dev = torch.device("cuda:0")
    reps = args.op_reps
    g = torch.Generator(device=dev)
    g.manual_seed(1337)
    out = []

    def randn(shape, std=1.0, mean=0.0, dtype=torch.bfloat16):
        return (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std + mean).to(dtype)

    only = [o for o in args.ops.split(",") if o]
    lib = _capi_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def stream_copy(dst, src):
        lib.cs_stream_copy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), src.numel(), stream)

    def stream_read(src, out):
        lib.cs_stream_read(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(out.data_ptr()), src.numel(), stream)

    def stream_fill(dst):
        lib.cs_stream_fill(ctypes.c_void_p(dst.data_ptr()), dst.numel(), 0, stream)

    def wanted(name):
        return not only or name == "stream_copy" or any(name.startswith(o) for o in only)

    copy_points = []  # (bytes moved, ms) of the plain copy, the practical ceiling at each size

    def copy_ms_at(nbytes):
        """Time a plain copy moving `nbytes` would take, interpolated between measured sizes."""
        pts = sorted(copy_points)
        if not pts:
            return None
        if nbytes <= pts[0][0]:
            return pts[0][1]  # below the smallest size the launch floor dominates
        for (b0, t0), (b1, t1) in zip(pts, pts[1:]):
            if nbytes <= b1:
                return t0 + (t1 - t0) * (nbytes - b0) / (b1 - b0)
        return pts[-1][1] * nbytes / pts[-1][0]

    def add(name, config, nbytes, make_set, call):
        """make_set() builds one set of buffers; call(set) issues the op once."""
        if not wanted(name):
            return
        n_cold = max(2, math.ceil(600e6 / nbytes) + 1)
        n_cold = min(n_cold, 64)
        sets = [make_set() for _ in range(n_cold)]
        op = call

        def call(s_):
            # what the op returns stays alive until this set's next turn, so the allocator hands
            # every call a block that was last written n_cold calls ago: outputs are cold too
            s_["_out"] = op(s_)

        for s in sets[:2]:
            call(s)
        warm_med, warm_call = event_ms(lambda i: call(sets[0]), reps, torch)
        cold_med, cold_call = event_ms(lambda i: call(sets[i % n_cold]), reps, torch)
        rec = {
            "op": name, "config": config, "algorithmic_bytes": nbytes,
            "ms_warm": round(warm_med, 5), "ms_cold": round(cold_med, 5),
            "ms_cold_per_call_events": round(cold_call, 5),
            "gbps_warm": round(nbytes / warm_med / 1e6, 1), "gbps_cold": round(nbytes / cold_med / 1e6, 1),
            "frac_cold": round(nbytes / cold_med / 1e6 / HBM_PEAK_GBPS, 4),
            "buffer_sets": n_cold, "calls_per_batch": reps,
        }
        if name == "stream_copy":
            copy_points.append((nbytes, cold_med))
        elif not name.startswith("stream_"):
            ceiling = copy_ms_at(nbytes)
            if ceiling:
                rec["copy_ms_same_bytes"] = round(ceiling, 5)
                rec["frac_of_copy"] = round(ceiling / cold_med, 3)
        out.append(rec)
        log(f"[per-op] {name:28s} {config:34s} warm {warm_med*1e3:9.1f} us  cold {cold_med*1e3:9.1f} us  "
            f"{rec['gbps_cold']:8.1f} GB/s  {rec['frac_cold']*100:5.1f}% of HBM peak"
            + (f"  {rec['frac_of_copy']*100:5.1f}% of a plain copy" if "frac_of_copy" in rec else ""))
        del sets
        torch.cuda.empty_cache()

    # ---- calibration: what trivial kernels reach at the sizes of the ops below.  A plain copy
    # moving the same number of bytes (half read, half written) is the practical ceiling of an op
    # at that size; the read-only and write-only passes show which half limits it.
    for mb in (25, 100, 400, 1600, 3500):
        nbytes = int(mb * 1e6) // 32 * 32

        def mk(nb=nbytes):
            return {"a": torch.empty(nb // 2, dtype=torch.uint8, device=dev),
                    "b": torch.empty(nb // 2, dtype=torch.uint8, device=dev)}

        add("stream_copy", f"{mb} MB moved", nbytes, mk,
            lambda s_: stream_copy(s_["b"], s_["a"]))
    for mb in (25, 100, 400, 3500):
        nbytes = int(mb * 1e6) // 32 * 32

        def mk1(nb=nbytes):
            return {"a": torch.empty(nb, dtype=torch.uint8, device=dev),
                    "o": torch.empty(max(1, lib.cs_stream_read_out_words(nb)), dtype=torch.int32, device=dev)}

        add("stream_read", f"{mb} MB read", nbytes, mk1, lambda s_: stream_read(s_["a"], s_["o"]))
        add("stream_fill", f"{mb} MB written", nbytes, mk1, lambda s_: stream_fill(s_["a"]))

    # ---- configuration 3: LayerNorm [8192,768] bf16, fp32 parameters
    for tag, rows, C in (("small", 8192, 768), ("xl", 16384, 1600)):
        gamma, beta = randn(C, 0.02, 1.0, torch.float32), randn(C, 0.02, 0.0, torch.float32)
        fwd_bytes = 2 * rows * C * 2 + 2 * C * 4 + 2 * rows * 4
        bwd_bytes = 3 * rows * C * 2 + 2 * rows * 4 + C * 4 + 2 * C * 4

        def mk():
            x = randn((rows, C))
            y, mean, rstd = ops.layernorm_forward(x, gamma, beta, 1e-5)
            return {"x": x, "dy": randn((rows, C)), "mean": mean, "rstd": rstd}

        add("layernorm_fwd", f"{tag} [{rows},{C}] bf16", fwd_bytes, mk,
            lambda s: ops.layernorm_forward(s["x"], gamma, beta, 1e-5))
        add("layernorm_bwd", f"{tag} [{rows},{C}] bf16", bwd_bytes, mk,
            lambda s: ops.layernorm_backward(s["dy"], s["x"], s["mean"], s["rstd"], gamma))

        # the reference's schedule: input gradient on the main stream, parameter gradients on the
        # assist stream.  The timed stream runs the row pass; a second stream adds the partial rows
        # up, and the timed stream waits for that two calls later, as the host scheduler does
        side = torch.cuda.Stream(dev)
        pending = []

        def two_streams(s):
            main = torch.cuda.current_stream(dev)
            if len(pending) >= 2:
                main.wait_event(pending.pop(0))
            dx, partials = ops.layernorm_backward_rows(s["dy"], s["x"], s["mean"], s["rstd"], gamma)
            side.wait_stream(main)
            with torch.cuda.stream(side):
                dg, db = ops.layernorm_backward_finalize(partials, torch.bfloat16, torch.float32)
                done = torch.cuda.Event()
                done.record(side)
            partials.record_stream(side)
            pending.append(done)
            return dx, dg, db

        add("layernorm_bwd_two_streams", f"{tag} [{rows},{C}] bf16, row pass timed, sums on a second stream",
            bwd_bytes, mk, two_streams)

        # the residual stream folded into the call (x + residual -> LayerNorm; LayerNorm backward
        # + dresidual), next to the same work as a separate elementwise add around the plain call
        def mk_res():
            st = mk()
            st["res"] = randn((rows, C))
            return st

        add("add_layernorm_fwd", f"{tag} [{rows},{C}] bf16, one call", fwd_bytes + 2 * rows * C * 2, mk_res,
            lambda s: ops.add_layernorm_forward(s["x"], s["res"], gamma, beta, 1e-5))
        add("add_then_layernorm_fwd", f"{tag} [{rows},{C}] bf16, torch.add + call", fwd_bytes + 2 * rows * C * 2, mk_res,
            lambda s: ops.layernorm_forward(torch.add(s["x"], s["res"]), gamma, beta, 1e-5))
        add("layernorm_bwd_add", f"{tag} [{rows},{C}] bf16, one call", bwd_bytes + rows * C * 2, mk_res,
            lambda s: ops.layernorm_backward(s["dy"], s["x"], s["mean"], s["rstd"], gamma, dresidual=s["res"]))
        add("layernorm_bwd_then_add", f"{tag} [{rows},{C}] bf16, call + torch.add", bwd_bytes + rows * C * 2, mk_res,
            lambda s: torch.add(ops.layernorm_backward(s["dy"], s["x"], s["mean"], s["rstd"], gamma)[0], s["res"]))

        # one call after another, as the norms of a training step: each call's launch also adds up
        # the partial rows of the call before it (cs_layernorm_backward_rows_pending), so no call
        # has a launch of its own for the column sums
        chain = ops.LayerNormBackwardChain()
        add("layernorm_bwd_chained", f"{tag} [{rows},{C}] bf16, column sums in the next call's launch", bwd_bytes, mk,
            lambda s: chain.backward(s["dy"], s["x"], s["mean"], s["rstd"], gamma))
        chain.flush()
        add("layernorm_bwd_add_chained", f"{tag} [{rows},{C}] bf16, column sums in the next call's launch",
            bwd_bytes + rows * C * 2, mk_res,
            lambda s: chain.backward(s["dy"], s["x"], s["mean"], s["rstd"], gamma, dresidual=s["res"]))
        chain.flush()

    # ---- configuration 3: GeLU [8192,3072] bf16, tanh (benchmark) and erf (the reference's form)
    n = 8192 * 3072
    for mode in ("tanh", "none"):
        def mk():
            return {"x": randn(n, 1.5), "dy": randn(n)}

        label = "tanh" if mode == "tanh" else "erf"
        add(f"gelu_fwd_{label}", "[8192,3072] bf16", 2 * n * 2, mk, lambda s: ops.gelu_forward(s["x"], mode))
        add(f"gelu_bwd_{label}", "[8192,3072] bf16", 3 * n * 2, mk, lambda s: ops.gelu_backward(s["dy"], s["x"], mode))

    # ---- configuration 1: token + position embedding.  Every buffer set has its own tables and
    # ids: with one table for all sets the gathered rows would come from the last-level cache.
    V, T = 50257, 1024
    for tag, B, C in (("small", 8, 768), ("xl", 16, 1600)):
        ranks = torch.arange(1, V + 1, dtype=torch.float64, device=dev).pow(-1.1)
        for kind in ("uniform", "zipf"):
            if tag == "xl" and kind == "uniform":
                continue
            fwd_bytes = B * T * 8 + B * T * C * 2 + T * C * 2 + B * T * C * 2
            bwd_bytes = B * T * 8 + B * T * C * 2 + V * C * 2 + T * C * 2

            def mk_ids():
                if kind == "uniform":
                    return torch.randint(0, V, (B, T), generator=g, device=dev, dtype=torch.int64)
                return torch.multinomial(ranks / ranks.sum(), B * T, replacement=True, generator=g).reshape(B, T)

            distinct = []

            def mk_fwd():
                ids_ = mk_ids()
                distinct.append(int(torch.unique(ids_).numel()))
                return {"wte": randn((V, C), 0.02), "wpe": randn((T, C), 0.02), "ids": ids_}

            def mk_bwd():
                return {"dout": randn((B, T, C)), "ids": mk_ids()}

            # a table row that several tokens name is read from memory once: the bytes that have to
            # move count each distinct row once (measured for this row's own id sets), which is what
            # the fraction of the HBM peak is taken against; `bytes_every_token_row` keeps the figure
            # that counts one table row per token
            n_before = len(out)
            add("embedding_fwd", f"{tag} {kind} B{B} T{T} C{C}", fwd_bytes, mk_fwd,
                lambda s: ops.embedding_forward_add(s["wte"], s["wpe"], s["ids"]))
            if len(out) > n_before and distinct:
                rec = out[-1]
                rows_read = sum(distinct) / len(distinct)
                nb = int(B * T * 8 + rows_read * C * 2 + T * C * 2 + B * T * C * 2)
                rec["bytes_every_token_row"] = fwd_bytes
                rec["distinct_rows_mean"] = round(rows_read, 1)
                rec["algorithmic_bytes"] = nb
                for k, ms in (("warm", rec["ms_warm"]), ("cold", rec["ms_cold"])):
                    rec[f"gbps_{k}"] = round(nb / ms / 1e6, 1)
                rec["frac_cold"] = round(nb / rec["ms_cold"] / 1e6 / HBM_PEAK_GBPS, 4)
                ceiling = copy_ms_at(nb)
                if ceiling:
                    rec["copy_ms_same_bytes"] = round(ceiling, 5)
                    rec["frac_of_copy"] = round(ceiling / rec["ms_cold"], 3)
                log(f"[per-op]   distinct table rows {rows_read:.0f} of {B * T} tokens: {nb} bytes have to move, "
                    f"{rec['gbps_cold']:.1f} GB/s, {rec['frac_cold']*100:.1f}% of HBM peak")
            add("embedding_bwd", f"{tag} {kind} B{B} T{T} C{C}", bwd_bytes, mk_bwd,
                lambda s: ops.embedding_backward_fused(s["dout"], s["ids"], V))

    # ---- configuration 0 / 4: AdamW over the GPT-2-small / XL parameter sets, one launch
    for tag, n_layer, C in (("small", 12, 768), ("xl", 48, 1600)):
        torch.cuda.empty_cache()  # fresh, unfragmented blocks for the four large parameter-sized buffers
        sizes = gpt2_param_sizes(n_layer, C)
        total = sum(sizes)
        if (tag == "xl" and not args.xl_adamw) or not wanted("adamw"):
            continue
        w = torch.empty(total, device=dev, dtype=torch.float32).normal_(0, 0.02, generator=g)
        grad = torch.empty(total, device=dev, dtype=torch.float32).normal_(0, 1e-3, generator=g)
        offs = [0]
        for s in sizes:
            offs.append(offs[-1] + s)
        ws_ = [w[offs[i]:offs[i + 1]] for i in range(len(sizes))]
        gs_ = [grad[offs[i]:offs[i + 1]] for i in range(len(sizes))]
        opt = ops.MultiTensorAdamW(ws_, gs_, lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
        opt.step()
        med, _ = event_ms(lambda i: opt.step(), max(5, reps // 4), torch)
        nbytes = 28 * total
        rec = {"op": "adamw_multi_tensor", "config": f"{tag} {len(sizes)} tensors {total} fp32 params",
               "algorithmic_bytes": nbytes, "ms_warm": round(med, 5), "ms_cold": round(med, 5),
               "gbps_warm": round(nbytes / med / 1e6, 1), "gbps_cold": round(nbytes / med / 1e6, 1),
               "frac_cold": round(nbytes / med / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1}
        ceiling = copy_ms_at(nbytes)
        if ceiling:
            rec["copy_ms_same_bytes"] = round(ceiling, 5)
            rec["frac_of_copy"] = round(ceiling / med, 3)
        out.append(rec)
        log(f"[per-op] adamw_multi_tensor           {tag:34s} {med*1e3:9.1f} us  {rec['gbps_cold']:8.1f} GB/s  "
            f"{rec['frac_cold']*100:5.1f}% of HBM peak")
        if tag == "small":
            # global-norm clipping folded into the step: a 4 B/parameter norm pass, then the step
            opt.step(max_grad_norm=1.0)
            med_c, _ = event_ms(lambda i: opt.step(max_grad_norm=1.0), reps, torch)
            nb_c = 32 * total
            out.append({"op": "adamw_multi_tensor_clipped", "config": f"{tag} norm pass + step, {total} fp32 params",
                        "algorithmic_bytes": nb_c, "ms_warm": round(med_c, 5), "ms_cold": round(med_c, 5),
                        "gbps_warm": round(nb_c / med_c / 1e6, 1), "gbps_cold": round(nb_c / med_c / 1e6, 1),
                        "frac_cold": round(nb_c / med_c / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1})
            log(f"[per-op] adamw + grad-norm clip       {tag:34s} {med_c*1e3:9.1f} us  {nb_c / med_c / 1e6:8.1f} GB/s")
            # the reference's launch shape: one launch per tensor (src/module/adamw.cpp:32-38)
            ms_, vs_ = [torch.zeros_like(x) for x in ws_], [torch.zeros_like(x) for x in ws_]

            def per_tensor(i):
                for a, b, c, d in zip(ws_, gs_, ms_, vs_):
                    ops.adamw_step(a, b, c, d, lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, t=1)

            per_tensor(0)
            med2, _ = event_ms(per_tensor, max(3, reps // 4), torch)
            out.append({"op": "adamw_per_tensor_launches", "config": f"{tag} {len(sizes)} launches",
                        "algorithmic_bytes": nbytes, "ms_warm": round(med2, 5), "ms_cold": round(med2, 5),
                        "gbps_warm": round(nbytes / med2 / 1e6, 1), "gbps_cold": round(nbytes / med2 / 1e6, 1),
                        "frac_cold": round(nbytes / med2 / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1})
            log(f"[per-op] adamw, {len(sizes)} launches      {tag:34s} {med2*1e3:9.1f} us")
            del ms_, vs_
        del opt, w, grad, ws_, gs_
        torch.cuda.empty_cache()
        # the same traffic without the arithmetic: four arrays of that many floats read, three
        # rewritten.  What this reaches is the ceiling for the step's access pattern.
        arrs = [torch.zeros(total, device=dev, dtype=torch.float32) for _ in range(4)]
        nb4 = total * 4 // 16 * 16

        def update4(i):
            lib.cs_stream_update4(*[ctypes.c_void_p(a.data_ptr()) for a in arrs], nb4, stream)

        update4(0)
        med4, _ = event_ms(update4, max(5, reps // 4), torch)
        out.append({"op": "stream_update4", "config": f"{tag} 4 x {total} floats read, 3 rewritten",
                    "algorithmic_bytes": 7 * nb4, "ms_warm": round(med4, 5), "ms_cold": round(med4, 5),
                    "gbps_warm": round(7 * nb4 / med4 / 1e6, 1), "gbps_cold": round(7 * nb4 / med4 / 1e6, 1),
                    "frac_cold": round(7 * nb4 / med4 / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1})
        rec["update4_ms_same_traffic"] = round(med4, 5)
        rec["frac_of_update4"] = round(med4 / rec["ms_cold"], 3)
        log(f"[per-op] stream_update4               {tag:34s} {med4*1e3:9.1f} us  {7 * nb4 / med4 / 1e6:8.1f} GB/s")
        del arrs
        torch.cuda.empty_cache()

    # ---- configuration 4: XL fused classifier [16384, 50257]
    if args.xl_ce and wanted("fused_classifier"):
        N = 16384
        x = randn((N, CE_STRIDE), 2.0)
        t = torch.randint(0, CE_V, (N,), generator=g, device=dev, dtype=torch.int64)
        nbytes = 2 * N * CE_V * 2 + N * 12 + 4
        bufs = [x.clone() for _ in range(3)]
        ops.fused_classifier(bufs[0], t, CE_V, inplace=True)
        med, _ = event_ms(lambda i: ops.fused_classifier(bufs[i % 3], t, CE_V, inplace=True), max(5, reps // 4), torch)
        out.append({"op": "fused_classifier", "config": f"xl [{N},{CE_V}] bf16 stride {CE_STRIDE}",
                    "algorithmic_bytes": nbytes, "ms_warm": round(med, 5), "ms_cold": round(med, 5),
                    "gbps_warm": round(nbytes / med / 1e6, 1), "gbps_cold": round(nbytes / med / 1e6, 1),
                    "frac_cold": round(nbytes / med / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 3})
        log(f"[per-op] fused_classifier xl          {med*1e3:9.1f} us  {nbytes/med/1e6:8.1f} GB/s")
        del bufs, x
        torch.cuda.empty_cache()

    # ---- reference-faithful variants of the headline op, whole call (three launches) each:
    #      every column a class (V == stride == 50304), and the autocast rule (bf16 logits in,
    #      fp32 gradient out: test/test_cross_entropy.cpp:102-139)
    if wanted("fused_classifier"):
        N = CE_N
        t = torch.randint(0, CE_V, (N,), generator=g, device=dev, dtype=torch.int64)
        bufs = [randn((N, CE_STRIDE), 2.0) for _ in range(3)]
        grads = [torch.empty((N, CE_STRIDE), dtype=torch.float32, device=dev) for _ in range(2)]
        variants = (
            ("in place, V 50257", 2 * N * CE_V * 2, lambda i: ops.fused_classifier(bufs[i % 3], t, CE_V, inplace=True)),
            ("in place, V = stride = 50304", 2 * N * CE_STRIDE * 2,
             lambda i: ops.fused_classifier(bufs[i % 3], t, CE_STRIDE, inplace=True)),
            ("bf16 logits -> fp32 gradient (autocast)", N * CE_V * 6,
             lambda i: ops.fused_classifier(bufs[i % 3], t, CE_V, dlogits_dtype=torch.float32)),
        )
        for tag, nbytes, fn in variants:
            fn(0)
            med, _ = event_ms(fn, max(5, reps // 4), torch)
            out.append({"op": "fused_classifier_call", "config": f"[{N},{CE_STRIDE}] bf16, {tag}",
                        "algorithmic_bytes": nbytes, "ms_warm": round(med, 5), "ms_cold": round(med, 5),
                        "gbps_warm": round(nbytes / med / 1e6, 1), "gbps_cold": round(nbytes / med / 1e6, 1),
                        "frac_cold": round(nbytes / med / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 3})
            log(f"[per-op] fused_classifier call        {tag:42s} {med*1e3:9.1f} us  {nbytes/med/1e6:8.1f} GB/s")
        del grads

    # ---- every launch of the path in one GPT-2-small training step (B 8, T 1024, C 768, 12
    #      blocks, vocabulary 50257), back to back on one stream, each on buffers of its own as a
    #      training step holds them: gather-add, 25 LayerNorm forward (24 of them with the residual
    #      add), 12 GeLU forward, the fused classifier, then the backward launches of the same and
    #      one AdamW step over all 148 parameter tensors.  The matrix products and attention that
    #      sit between them in a model are not part of the path and are not run.
    if wanted("gpt2_small_step_path"):
        torch.cuda.empty_cache()
        B, T, C, L, V = 8, 1024, 768, 12, CE_V
        rows = B * T
        wte, wpe = randn((V, C), 0.02), randn((T, C), 0.02)
        ids = torch.randint(0, V, (B, T), generator=g, device=dev, dtype=torch.int64)
        gamma, beta = randn(C, 0.02, 1.0, torch.float32), randn(C, 0.02, 0.0, torch.float32)
        n_ln = 2 * L + 1
        xs = [randn((rows, C)) for _ in range(n_ln)]        # LayerNorm inputs (the residual stream)
        res = [randn((rows, C)) for _ in range(n_ln)]       # what is added to it before each norm
        dys = [randn((rows, C)) for _ in range(n_ln)]
        hs = [randn((rows, 4 * C), 1.5) for _ in range(L)]  # GeLU inputs
        dhs = [randn((rows, 4 * C)) for _ in range(L)]
        logits = randn((rows, CE_STRIDE), 2.0)
        targets = torch.randint(0, V, (rows,), generator=g, device=dev, dtype=torch.int64)
        dout = randn((B, T, C))
        _, mean, rstd = ops.layernorm_forward(xs[0], gamma, beta, 1e-5)
        sizes = gpt2_param_sizes(L, C)
        total = sum(sizes)
        w = torch.empty(total, device=dev, dtype=torch.float32).normal_(0, 0.02, generator=g)
        grad = torch.empty(total, device=dev, dtype=torch.float32).normal_(0, 1e-3, generator=g)
        offs = [0]
        for sz in sizes:
            offs.append(offs[-1] + sz)
        opt = ops.MultiTensorAdamW([w[offs[i]:offs[i + 1]] for i in range(len(sizes))],
                                   [grad[offs[i]:offs[i + 1]] for i in range(len(sizes))],
                                   lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
        keep = {}
        ln_chain = ops.LayerNormBackwardChain()

        def path_step(i):
            k = []
            k.append(ops.embedding_forward_add(wte, wpe, ids))
            k.append(ops.layernorm_forward(xs[0], gamma, beta, 1e-5))
            for j in range(1, n_ln):
                k.append(ops.add_layernorm_forward(xs[j], res[j], gamma, beta, 1e-5))
            for j in range(L):
                k.append(ops.gelu_forward(hs[j], "tanh"))
            k.append(ops.fused_classifier(logits, targets, V, inplace=True))
            for j in range(L):
                k.append(ops.gelu_backward(dhs[j], hs[j], "tanh"))
            for j in range(1, n_ln):
                k.append(ln_chain.backward(dys[j], xs[j], mean, rstd, gamma, dresidual=res[j]))
            k.append(ln_chain.backward(dys[0], xs[0], mean, rstd, gamma))
            ln_chain.flush()  # the first norm's column sums: the one launch of that kind in the step
            k.append(ops.embedding_backward_fused(dout, ids, V))
            opt.step()
            keep[i % 2] = k  # outputs stay alive for a step, as activations and gradients do

        ln_f = 2 * rows * C * 2 + 2 * C * 4 + 2 * rows * 4
        ln_b = 3 * rows * C * 2 + 2 * rows * 4 + 3 * C * 4
        nbytes = ((rows * C * 2 + rows * 8 + T * C * 2 + rows * C * 2)                # gather-add
                  + ln_f + (n_ln - 1) * (ln_f + 2 * rows * C * 2)                     # LayerNorm forward
                  + L * 2 * rows * 4 * C * 2 + L * 3 * rows * 4 * C * 2               # GeLU forward, backward
                  + 2 * rows * CE_V * 2 + rows * 12                                   # fused classifier
                  + ln_b + (n_ln - 1) * (ln_b + rows * C * 2)                         # LayerNorm backward
                  + rows * C * 2 + V * C * 2 + T * C * 2                              # embedding backward
                  + 28 * total)                                                       # AdamW
        launches = 1 + n_ln + L + 3 + L + n_ln + 1 + 3 + 1
        path_step(0)
        med, _ = event_ms(path_step, 5, torch)
        out.append({"op": "gpt2_small_step_path", "config": f"B{B} T{T} C{C} {L} blocks V{V}: {launches} launches of the path, "
                                                           "one training step, no matrix products",
                    "algorithmic_bytes": nbytes, "ms_warm": round(med, 5), "ms_cold": round(med, 5),
                    "gbps_warm": round(nbytes / med / 1e6, 1), "gbps_cold": round(nbytes / med / 1e6, 1),
                    "frac_cold": round(nbytes / med / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1, "launches": launches})
        log(f"[per-op] gpt2_small_step_path         {launches} launches {med*1e3:9.1f} us  {nbytes/med/1e6:8.1f} GB/s  "
            f"{nbytes/med/1e6/HBM_PEAK_GBPS*100:5.1f}% of HBM peak")
        del opt, w, grad, xs, res, dys, hs, dhs, logits, keep
        torch.cuda.empty_cache()

    # ---- the same step submitted as tasks through the C++ host layer (cs::compute:: /
    #      cs::optimizer:: calls, three-stream scheduler, Python binding): what a program written
    #      against the reference's API gets: the same launches as the row above (LayerNorm through
    #      the host layer's forward_with_residual / backward_with_residual), the optimizer as two
    #      tasks (fp32 parameters, bf16 tables).  Wall clock from the first submission to the host's
    #      wait for the last parameter.
    if wanted("gpt2_small_step_host_layer"):
        try:
            from core_scheduler_amd import _cs_host as host
        except ImportError as e:  # the binding is built by __graft_entry__.build()
            host = None
            log(f"[per-op] gpt2_small_step_host_layer skipped: {e}")
        if host is not None:
            out.append(host_layer_step(torch, host, g))
            torch.cuda.empty_cache()
    return out


def host_layer_step(torch, host, g):
    import time

    dev = "cuda:0"
    B, T, C, L, V = 8, 1024, 768, 12, CE_V
    rows = B * T
    sched = host.DynamicScheduler(0)

    def rn(shape, dtype=torch.bfloat16, std=1.0):
        return torch.empty(shape, device=dev, dtype=torch.float32).normal_(0, std, generator=g).to(dtype)

    def up(t):
        return host.from_torch(sched, t)

    wte = host.Embedding.init(sched, V, C, dtype="bfloat16")
    wpe = host.Embedding.init(sched, T, C, dtype="bfloat16")
    n_ln = 2 * L + 1
    lns = [host.LayerNorm.init(sched, [C], dtype="float32") for _ in range(n_ln)]
    gelus = [host.GeLU.init(sched, 1) for _ in range(L)]
    ids = up(torch.randint(0, V, (B, T), device=dev, generator=g))
    targets = up(torch.randint(0, V, (rows,), device=dev, generator=g))
    hs = [up(rn((B, T, 4 * C), std=1.5)) for _ in range(L)]
    dhs = [up(rn((B, T, 4 * C))) for _ in range(L)]
    dy_last = up(rn((B, T, C)))
    res = [up(rn((B, T, C))) for _ in range(n_ln)]   # what is added to the stream before each norm
    dres = [up(rn((B, T, C))) for _ in range(n_ln)]  # the gradient that flows past each norm
    logits = [up(rn((rows, CE_STRIDE), std=2.0)) for _ in range(2)]
    shapes = []
    for _ in range(L):  # attention and MLP parameters: only the optimizer touches them here
        shapes += [(3 * C, C), (3 * C,), (C, C), (C,), (4 * C, C), (4 * C,), (C, 4 * C), (C,)]
    other_w = [up(rn(sh, torch.float32, 0.02)) for sh in shapes]
    other_g = [up(rn(sh, torch.float32, 1e-3)) for sh in shapes]
    hp = dict(lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    states = []

    def step(k):
        h = host.Embedding.forward_with_positions(sched, wte, wpe, ids)
        h = host.LayerNorm.forward(sched, lns[0], h)
        for j in range(1, n_ln):
            h, _ = host.LayerNorm.forward_with_residual(sched, lns[j], h, res[j])
        for j in range(L):
            host.GeLU.forward(sched, gelus[j], hs[j])
        ce = host.CrossEntropy.init(sched, num_classes=V)
        host.CrossEntropy.forward(sched, ce, logits[k % 2], targets)
        host.CrossEntropy.backward(sched, ce)
        for j in reversed(range(L)):
            host.GeLU.backward(sched, gelus[j], dhs[j])
        d = dy_last
        for j in reversed(range(1, n_ln)):
            d = host.LayerNorm.backward_with_residual(sched, lns[j], d, dres[j])
        d = host.LayerNorm.backward(sched, lns[0], d)
        host.Embedding.backward_with_positions(sched, wte, wpe, d)
        ws, grads = [], []
        for st in lns:
            ws += [st.weight, st.bias]
            grads += [st.grad_weight, st.grad_bias]
        ws += other_w
        grads += other_g
        tabs, tgrads = [wte.weight, wpe.weight], [wte.grad_weight, wpe.grad_weight]
        if not states:
            states.append([host.AdamW.init(sched, w, **hp) for w in ws])
            states.append([host.AdamW.init(sched, w, **hp) for w in tabs])
        host.AdamW.step_all(sched, states[0], ws, grads)
        host.AdamW.step_all(sched, states[1], tabs, tgrads)
        for st in lns:
            st.zero_grad()
        wte.zero_grad()
        wpe.zero_grad()
        return ws[0]

    for k in range(3):
        step(k).wait()
    torch.cuda.synchronize()
    K, times, submits = 10, [], []
    for _ in range(3):
        t0 = time.perf_counter()
        for k in range(K):
            last = step(k)
        submits.append((time.perf_counter() - t0) / K)
        last.wait()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) / K)
    sec, sub = sorted(times)[1], sorted(submits)[1]
    ln_f = 2 * rows * C * 2 + 2 * C * 4 + 2 * rows * 4
    ln_b = 3 * rows * C * 2 + 2 * rows * 4 + 3 * C * 4
    n_fp32 = n_ln * 2 * C + sum(int(torch.tensor(sh).prod()) for sh in shapes)
    nbytes = ((rows * C * 2 + rows * 8 + T * C * 2 + rows * C * 2) + ln_f + (n_ln - 1) * (ln_f + 2 * rows * C * 2)
              + L * 2 * rows * 4 * C * 2 + L * 3 * rows * 4 * C * 2 + 2 * rows * CE_V * 2 + rows * 12
              + ln_b + (n_ln - 1) * (ln_b + rows * C * 2)
              + rows * C * 2 + V * C * 2 + T * C * 2 + 28 * n_fp32 + 14 * (V * C + T * C))
    tasks = 1 + n_ln + L + 2 + n_ln + L + 1 + 2
    ms = sec * 1e3
    log(f"[per-op] gpt2_small_step_host_layer   {tasks} tasks {ms*1e3:9.1f} us  {nbytes/ms/1e6:8.1f} GB/s  "
        f"{nbytes/ms/1e6/HBM_PEAK_GBPS*100:5.1f}% of HBM peak  (the host submits a step in {sub*1e6:.0f} us)")
    return {"op": "gpt2_small_step_host_layer",
            "config": f"B{B} T{T} C{C} {L} blocks V{V}: {tasks} tasks through the C++ host layer, wall clock",
            "algorithmic_bytes": nbytes, "ms_warm": round(ms, 5), "ms_cold": round(ms, 5),
            "gbps_warm": round(nbytes / ms / 1e6, 1), "gbps_cold": round(nbytes / ms / 1e6, 1),
            "frac_cold": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "buffer_sets": 1, "tasks": tasks,
            "host_submit_ms": round(sub * 1e3, 4)}


def fill_sweep(torch):
    """The write path on its own: cs_stream_fill_shape over launch shapes and sizes, cold buffers,
    back-to-back launches between one pair of events.  Prints a table (us per launch, TB/s) on
    stdout; `python bench.py --fill-sweep` is the whole command."""
    lib = _capi_lib()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    sizes = [int(x) // 65536 * 65536 for x in (25e6, 77.2e6, 100e6, 400e6, 3.5e9)]
    pool = torch.empty(int(7.2e9), dtype=torch.uint8, device=dev).zero_()

    def timed(shape, nbytes, reps):
        nsets = max(2, min(64, int(7e9 // nbytes)))
        if nsets * nbytes < 6e8:
            nsets = min(64, int(6e8 // nbytes) + 1)

        def call(i):
            code = lib.cs_stream_fill_shape(ctypes.c_void_p(pool.data_ptr() + (i % nsets) * nbytes), nbytes, 0, *shape, stream)
            if code != 0:
                raise RuntimeError(f"cs_stream_fill_shape{shape}: {code}")

        call(0)
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            hold_gpu(torch, 2.0)
            e0.record()
            for i in range(reps):
                call(i)
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / reps * 1e3)
        return best

    print("write-only kernel, us per launch and TB/s; lanes x vectors per lane, layout (block: lane-strided chunks, "
          "wave-KB: whole kilobytes per wave), store, grid (chunks: one chunk per workgroup, k/CU: k persistent workgroups per CU)")
    print(f"{'lanes':>5s} {'vec':>3s} {'layout':>7s} {'store':>5s} {'grid':>6s} | " + " | ".join(f"{b / 1e6:9.0f} MB" for b in sizes))
    best = {b: (float("inf"), None) for b in sizes}
    for plain in (0, 1):
        for wave_kb in (0, 1):
            for lanes in (256, 1024):
                for vec in (1, 2, 4, 8):
                    for per_cu in ((0, 8) if plain == 0 else (0,)):
                        shape = (lanes, vec, wave_kb, plain, per_cu)
                        cells = []
                        for b in sizes:
                            us = timed(shape, b, 30 if b < 1e9 else 8)
                            cells.append(f"{us:7.1f} {b / us / 1e6:4.2f}")
                            if us < best[b][0]:
                                best[b] = (us, shape)
                        print(f"{lanes:5d} {vec:3d} {'wave-KB' if wave_kb else 'block':>7s} {'plain' if plain else 'nt':>5s} "
                              f"{(str(per_cu) + '/CU') if per_cu else 'chunks':>6s} | " + " | ".join(cells), flush=True)
    for b in sizes:
        print(f"fastest at {b / 1e6:.0f} MB: {best[b][0]:.1f} us, (lanes, vectors, wave-KB, plain stores, workgroups per CU) = {best[b][1]}")


def cpu_baseline(args, torch):
    """The reference's cross-entropy op sequence on the ATen CPU backend, full configuration-2 size."""
    from oracle import aten_port as ap

    rows = args.cpu_rows
    g = torch.Generator().manual_seed(1337 + 2)
    # the values the GPU sees: bf16 logits, widened to fp32 as the reference's AMP path does
    x = (torch.randn((rows, CE_V), generator=g) * 2.0).to(torch.bfloat16).float()
    t = torch.randint(0, CE_V, (rows,), generator=g)
    times = []
    for i in range(1 + args.cpu_reps):
        t0 = time.perf_counter()
        loss, grad, _ = ap.cross_entropy(x, t)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times[1:])
    nbytes = CE_BYTES * rows / CE_N
    return {
        "value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{rows} of {CE_N} rows x {CE_V} classes, fp32-widened bf16 logits; at::log_softmax + nll_loss_forward + "
                  f"nll_loss_backward + _log_softmax_backward_data on the ATen CPU backend; median of {args.cpu_reps} "
                  f"after 1 warm-up; {med*1e3:.1f} ms per call; same algorithmic bytes per row as the GPU figure",
        "ms": round(med * 1e3, 3),
    }


def cpu_per_op(args, torch, table):
    """The reference's CPU path for every small-configuration row of the per-op table: the ATen
    CPU ops its task bodies call (fp32 inputs, as its CPU tests run them) and, for AdamW, the C
    restatement of its kernel.  Attaches `cpu_ms` (median of 3 after a warm-up) to the records."""
    from oracle import aten_port as ap
    from oracle import c_oracle as co

    g = torch.Generator().manual_seed(1337)

    def med(fn, reps=3):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return statistics.median(ts) * 1e3

    cpu = {}
    rows, C = 8192, 768
    x, dy = torch.randn((rows, C), generator=g), torch.randn((rows, C), generator=g)
    gamma, beta = torch.ones(C), torch.zeros(C)
    _, mean, rstd = ap.layernorm_forward(x, gamma, beta)
    cpu[("layernorm_fwd", "small")] = med(lambda: ap.layernorm_forward(x, gamma, beta))
    cpu[("layernorm_bwd", "small")] = med(lambda: ap.layernorm_backward(dy, x, mean, rstd, gamma, beta))
    xg, dg = torch.randn(8192 * 3072, generator=g) * 1.5, torch.randn(8192 * 3072, generator=g)
    for mode, tag in (("tanh", "tanh"), ("none", "erf")):
        cpu[(f"gelu_fwd_{tag}", "")] = med(lambda: ap.gelu_forward(xg, mode))
        cpu[(f"gelu_bwd_{tag}", "")] = med(lambda: ap.gelu_backward(dg, xg, mode))
    V, B, T = 50257, 8, 1024
    wte, wpe = torch.randn((V, C), generator=g) * 0.02, torch.randn((T, C), generator=g) * 0.02
    ids = torch.randint(0, V, (B, T), generator=g)
    dout = torch.randn((B, T, C), generator=g)
    cpu[("embedding_fwd", "small uniform")] = med(lambda: ap.token_position_forward(wte, wpe, ids))
    cpu[("embedding_bwd", "small uniform")] = med(lambda: ap.token_position_backward(dout, ids, V))
    total = sum(gpt2_param_sizes(12, 768))
    w, gr = torch.randn(total, generator=g) * 0.02, torch.randn(total, generator=g) * 1e-3
    m, v = torch.zeros(total), torch.zeros(total)
    hp = dict(lr=6e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    cpu[("adamw_multi_tensor", "small")] = med(lambda: co.adamw_step(w, gr, m, v, t=1, **hp), reps=2)
    for rec in table:
        for (op, tag), ms in cpu.items():
            if rec["op"] == op and rec["config"].startswith(tag):
                rec["cpu_ms"] = round(ms, 3)
                rec["cpu_path"] = ("C restatement of src/optimizer/adamw.cu, 1 thread" if op.startswith("adamw")
                                   else f"ATen CPU ops of the reference's task body, fp32, {torch.get_num_threads()} threads")
                log(f"[cpu]    {op:28s} {rec['config'][:34]:34s} {ms:10.2f} ms on the CPU, {rec['ms_cold']*1e3:9.1f} us on the GPU")
    return table


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--op-reps", type=int, default=40, help="timed calls per op in the per-op table")
    ap.add_argument("--max-buffers", type=int, default=32, help="distinct logits buffers rotated by the headline loop")
    ap.add_argument("--no-per-op", action="store_true")
    ap.add_argument("--ops", default="", help="comma list of op-name prefixes to keep in the per-op table")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-xl-adamw", dest="xl_adamw", action="store_false", help="skip the 25 GB XL AdamW line")
    ap.add_argument("--no-xl-ce", dest="xl_ce", action="store_false")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="K",
                    help="also run K plain 1 GiB copies (to scale hardware traffic counters)")
    ap.add_argument("--full-json", default="", metavar="PATH", help="also write the full per-op table to this file")
    ap.add_argument("--fill-sweep", action="store_true",
                    help="only sweep the write-only calibration kernel over launch shapes and print the table")
    ap.add_argument("--cpu-rows", type=int, default=CE_N)
    ap.add_argument("--cpu-reps", type=int, default=5)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (no collectives are part of it); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device visible; the kernels have no CPU path", file=sys.stderr)
        sys.exit(3)
    from core_scheduler_amd import _capi as capi
    from core_scheduler_amd import ops

    capi.load()  # raises if the kernel library is not built
    log(f"[bench] device: {torch.cuda.get_device_name(0)}; torch {torch.__version__}")
    if args.fill_sweep:
        fill_sweep(torch)
        return

    head = run_headline(args, torch, ops, capi)
    achieved = CE_BYTES / (head["rows_kernel_ms_avg"] * 1e-3) / 1e9
    value = CE_BYTES * args.steps / head["seconds"] / 1e9
    log(f"[bench] fused classifier: {head['ms_per_step']:.4f} ms/step wall, row kernel {head['rows_kernel_ms_avg']:.4f} ms "
        f"(events), {achieved:.0f} GB/s = {achieved / HBM_PEAK_GBPS * 100:.1f}% of HBM peak, loss {head['loss']:.4f}")

    if args.calibrate_copy:
        # a known-size kernel next to the row pass, for scaling hardware traffic counters
        a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
        b = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(args.calibrate_copy):
            capi.check("cs_stream_copy", capi.load().cs_stream_copy(ctypes.c_void_p(b.data_ptr()),
                                                                      ctypes.c_void_p(a.data_ptr()), 1 << 30, st))
        torch.cuda.synchronize()
        del a, b

    table = [] if args.no_per_op else per_op_table(args, torch, ops)
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(args, torch)
        log(f"[bench] CPU baseline (ATen CPU, {cpu['cores']} threads): {cpu['ms']:.1f} ms, {cpu['value']} GB/s")
        if table:
            cpu_per_op(args, torch, table)

    line = result_line(args, head, value, achieved, cpu, table)
    full = dict(line, per_op=table)
    log("[bench-full] " + json.dumps(full))
    if args.full_json:
        with open(args.full_json, "w") as f:
            json.dump(full, f, indent=1)
    print(json.dumps(line), flush=True)


MAX_LINE_BYTES = 8000  # the result line on stdout stays below this; the full table goes to stderr


# Rows that time an alternative way of issuing an op (the reference's two-stream LayerNorm
# backward, a separate add launch, one AdamW launch per tensor) next to the library's own way.
# They are in the full table, under their own names; the result line carries the ops themselves.
COMPARISON_ROWS = ("layernorm_bwd_two_streams", "add_then_layernorm_fwd", "layernorm_bwd_then_add",
                   "adamw_per_tensor_launches")


def compact_per_op(table):
    """One short record per row of the per-op table: op, configuration tag, cold ms per call,
    cold fraction of the HBM peak.  Everything else a row carries is in the full table, and so
    are the comparison rows."""
    out = []
    for rec in table:
        if rec["op"] in COMPARISON_ROWS:
            continue
        parts = rec["config"].split(":")[0].split(", ")
        cfg = ", ".join(parts[:2]) if rec["op"] == "fused_classifier_call" else parts[0]
        out.append({"op": rec["op"], "cfg": cfg[:44], "ms": rec["ms_cold"], "frac": rec["frac_cold"]})
    return out


def result_line(args, head, value, achieved, cpu, table):
    """The one JSON line for stdout.  `per_op` is compact and comes before `roofline` and
    `cpu_baseline`, so the end of the line always shows those two."""
    line = {
        "metric": "per-op HBM GB/s (% of MI355X peak); fused CE ms at 8192x50257 bf16",
        "metric_note": "value = the fused classifier's whole-step GB/s (the ms is ms_per_step); every other op is in per_op "
                       "(ms and fraction of the HBM peak per call, cold buffers); the full table, with rows that time alternative ways of issuing an op, is on stderr after [bench-full]",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "fused classifier (softmax + cross-entropy + in-place dlogits), logits [8192, 50257] bf16, "
                        "row stride 50304, int64 targets, mean reduction (benchmark configuration 2)",
            "algorithmic_bytes_per_step": CE_BYTES,
            "logits_buffers_rotated": head["buffers"],
            "loss": round(head["loss"], 5),
        },
        "per_op": compact_per_op(table),
        "roofline": {
            "bound": "hbm",
            "kernel": "ce_rows_stream_kernel<bf16_t, bf16_t, 7, 8, false>",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "kernel_ms_avg": round(head["rows_kernel_ms_avg"], 5),
            "kernel_ms_median": round(head["rows_kernel_ms_median"], 5),
            # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
            # profiles/ce_rows_stream_kernel_hbm_traffic_pmc.txt (scaled by a plain copy's readings)
            "traffic": CE_ROWS_TRAFFIC_BYTES,
            "traffic_over_algorithmic": round(CE_ROWS_TRAFFIC_BYTES / CE_BYTES, 4),
        },
        "cpu_baseline": cpu,
    }
    # the calibration rows go first if the line ever has to shrink
    while len(json.dumps(line)) > MAX_LINE_BYTES and line["per_op"]:
        drop = next((i for i, r in enumerate(line["per_op"]) if r["op"].startswith("stream_")), len(line["per_op"]) - 1)
        line["per_op"].pop(drop)
        line["per_op_truncated"] = True
    return line


if __name__ == "__main__":
    main()
