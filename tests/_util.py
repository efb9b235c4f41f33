"""Shared helpers of the test-suite: seeded inputs, tolerances, ulp distance."""
import torch

# ---- tolerances (the parity bar) -------------------------------------------
# fp32 results: |got - want| <= atol + RTOL * |want|, RTOL = 1e-5, with an atol
# stated per op (the reference's own tests use at::allclose, rtol 1e-5).
# 16-bit results: at most 1 ulp of the storage type away from the oracle's
# value rounded once, or inside the same atol (which covers results that
# cancel to ~0, where an ulp is arbitrarily small).
RTOL = 1e-5


def gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def randn(shape, seed, std=1.0, mean=0.0, dtype=torch.float32):
    return (torch.randn(shape, generator=gen(seed), dtype=torch.float32) * std + mean).to(dtype)


def randint(lo, hi, shape, seed, dtype=torch.int64):
    return torch.randint(lo, hi, shape, generator=gen(seed), dtype=torch.int64).to(dtype)


def zipf_ids(n, vocab, seed, s=1.1):
    """Rank r (1-based) drawn with probability ~ r^-s; id = rank - 1."""
    ranks = torch.arange(1, vocab + 1, dtype=torch.float64)
    p = ranks.pow(-s)
    p /= p.sum()
    return torch.multinomial(p, n, replacement=True, generator=gen(seed)).to(torch.int64)


def _ordered(t):
    """Maps 16-bit float bit patterns to integers that are monotone in value."""
    bits = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    neg = bits >= 0x8000
    return torch.where(neg, 0x8000 - bits, bits)


def ulp_distance(got, want):
    assert got.dtype == want.dtype and got.dtype in (torch.bfloat16, torch.float16)
    return (_ordered(got) - _ordered(want)).abs()


def assert_close(got, want, atol, name="", rtol=RTOL):
    """The parity bar, for fp32/fp64 and for 16-bit storage."""
    got, want = got.detach().cpu(), want.detach().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert got.dtype == want.dtype, f"{name}: dtype {got.dtype} vs {want.dtype}"
    gf, wf = got.double(), want.double()
    nan_mismatch = torch.isnan(gf) != torch.isnan(wf)
    assert not nan_mismatch.any(), f"{name}: NaN pattern differs"
    err = (gf - wf).abs()
    ok = err <= atol + rtol * wf.abs()
    if got.dtype in (torch.bfloat16, torch.float16):
        ok |= ulp_distance(got, want) <= 1
    ok |= torch.isnan(wf)
    if not ok.all():
        bad = (~ok).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(
            f"{name}: {bad.shape[0]} of {ok.numel()} elements off; first at {i}: got {got[i].item()!r} "
            f"want {want[i].item()!r}; max abs err {err.max().item():.3e}")


def sum_tolerance(terms, dim=0):
    """Per-output tolerance for fp32 sums over `dim` of `terms`, derived from the data.

    Each of the n - 1 additions rounds its partial sum by at most u = 2^-24 of it; with partial
    sums of a blocked summation at most ~sqrt(n) rms(terms) and rounding errors of either sign,
    the error of one sum is ~ u sqrt(log2 n) sqrt(sum terms^2).  Two fp32 evaluations are compared
    (kernel and oracle) over thousands of outputs, hence the factor 7 (2 x a 3.5 sigma maximum).
    """
    t = terms.double()
    n = max(2, t.shape[dim])
    return 7.0 * 2.0 ** -24 * torch.sqrt(torch.log2(torch.tensor(float(n))) * (t * t).sum(dim))


def scatter_sum_tolerance(terms, ids, num_rows):
    """sum_tolerance for a scatter-add: out[ids[i]] += terms[i].  Row r of the result gets the bar
    its own terms justify (rows nothing was added to get 0, plus the 1e-7 floor of the caller)."""
    t = terms.reshape(ids.numel(), -1).double()
    idx = ids.reshape(-1).long()
    keep = (idx >= 0) & (idx < num_rows)
    sq = torch.zeros((num_rows, t.shape[1]), dtype=torch.float64).index_add_(0, idx[keep], (t * t)[keep])
    n = max(2, ids.numel())
    return 7.0 * 2.0 ** -24 * torch.sqrt(torch.log2(torch.tensor(float(n))) * sq)


def assert_sum_close(got, want, tol, name="", rtol=RTOL):
    """|got - want| <= tol + rtol |want| with a per-element `tol` (see sum_tolerance); 16-bit
    results may instead be within 1 ulp."""
    got, want = got.detach().cpu(), want.detach().cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, name
    err = (got.double() - want.double()).abs()
    ok = err <= tol.reshape(want.shape) + rtol * want.double().abs()
    if got.dtype in (torch.bfloat16, torch.float16):
        ok |= ulp_distance(got, want) <= 1
    if not ok.all():
        i = tuple((~ok).nonzero()[0].tolist())
        raise AssertionError(f"{name}: {(~ok).sum().item()} of {ok.numel()} sums off; first at {i}: got "
                             f"{got[i].item()!r} want {want[i].item()!r}, allowed {tol.reshape(want.shape)[i].item():.3e}")


def assert_bit_exact(got, want, name=""):
    got, want = got.detach().cpu().contiguous(), want.detach().cpu().contiguous()
    assert got.shape == want.shape and got.dtype == want.dtype, name
    n = got.element_size()
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[n]
    same = got.view(view) == want.view(view)
    assert same.all(), f"{name}: {(~same).sum().item()} elements differ bitwise"


# GPT-2 parameter shapes (example/gpt2/gpt2_single_device.cpp:56-75: vocab 50257,
# block 1024; small: 12 layers, C 768; XL: 48 layers, C 1600), biases included.
def gpt2_param_shapes(n_layer=12, C=768, V=50257, T=1024):
    shapes = [(V, C), (T, C)]
    for _ in range(n_layer):
        shapes += [(C,), (C,), (C, 3 * C), (3 * C,), (C, C), (C,), (C,), (C,), (C, 4 * C), (4 * C,),
                   (4 * C, C), (C,)]
    shapes += [(C,), (C,)]
    return shapes
