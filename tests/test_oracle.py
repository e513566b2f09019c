"""Pins the CPU oracle (oracle/cats_oracle.c and the torch restatement in oracle/cats_oracle.py).

The reference holds no golden vectors for this path (its test file prints, it never asserts), so each oracle
function is pinned by what the mathematics fixes: exhaustive dtype conversion against numpy / torch, SiLU closed
forms, hand-built threshold boundary vectors, special cases that reduce to library GEMVs, exactness of a single
product, and float64 brute force on small shapes.  Each check is chosen so that a plausible slip (dropped term,
<= instead of <, transposed weight, wrong rounding point) fails it.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests.util import load_golden, make_mlp

DTYPES = [torch.float16, torch.bfloat16, torch.float32]


# ---- dtype conversion -----------------------------------------------------------------------------------------

def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_bits_table()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rounding_against_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(20000) * 1e-6).astype(np.float32),      # subnormal halves
        (rng.standard_normal(5000) * 3e4).astype(np.float32),        # near the fp16 maximum
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  3 * 2.0 ** -25, 6.1035e-05, 6.0976e-05, np.inf, -np.inf], dtype=np.float32),
    ])
    # exact ties between two adjacent halves: must go to even
    h = rng.integers(0, 0x7bff, 5000).astype(np.uint16)
    lo, hi = h.view(np.float16).astype(np.float64), (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    vals = np.concatenate([vals, ((lo + hi) / 2).astype(np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_conversion_against_torch(oracle):
    L = oracle.lib()
    g = torch.Generator().manual_seed(0)
    vals = torch.cat([torch.randn(20000, generator=g), torch.randn(5000, generator=g) * 1e-30, torch.randn(5000, generator=g) * 1e30,
                      torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.005859375, 3.3895e38, float("inf")])])
    want = vals.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    got = np.array([L.oracle_f32_to_bf16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    back = np.array([L.oracle_bf16_to_f32(int(b)) for b in want[:1000]], dtype=np.float32)
    assert np.array_equal(back, vals[:1000].to(torch.bfloat16).float().numpy())


# ---- SiLU -------------------------------------------------------------------------------------------------------

def test_silu_closed_forms(oracle):
    L = oracle.lib()
    assert L.oracle_silu(0.0) == 0.0
    # silu(x) - silu(-x) = x * (sigmoid(x) - (1 - sigmoid(x))) + ... = x  (identity of x*sigmoid(x))
    for x in (0.1, 0.5, 1.0, 2.5, 7.0, 20.0):
        assert abs(L.oracle_silu(x) - L.oracle_silu(-x) - x) < 1e-6 * max(1.0, x)
    # global minimum: x* solves 1 + exp(-x) + x exp(-x) = 0 -> x* = -1.2784645..., silu(x*) = -0.2784645...
    xs = np.linspace(-3, 0, 30001)
    ys = np.array([L.oracle_silu(float(x)) for x in xs])
    i = int(ys.argmin())
    assert abs(xs[i] - (-1.2784645)) < 2e-4 and abs(ys[i] - (-0.2784645)) < 1e-6
    # asymptotes and a library cross-check over a wide range
    assert abs(L.oracle_silu(30.0) - 30.0) < 1e-5 and abs(L.oracle_silu(-30.0)) < 1e-10
    t = torch.linspace(-20, 20, 4001)
    got = torch.tensor([L.oracle_silu(float(v)) for v in t])
    torch.testing.assert_close(got, F.silu(t.double()).float(), rtol=2e-7, atol=1e-9)


# ---- mask rule ----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_mask_rule_boundaries(oracle, dtype):
    """active <=> |a| > t with t cast to the tensor dtype; strict; sign-symmetric; t < 0 keeps exact zeros."""
    t = 0.1
    tr = float(torch.tensor(t).to(dtype))           # what torch compares against
    assert oracle.c_round(dtype, t) == tr
    up = float(torch.nextafter(torch.tensor(tr, dtype=dtype), torch.tensor(1.0, dtype=dtype)))
    dn = float(torch.nextafter(torch.tensor(tr, dtype=dtype), torch.tensor(0.0, dtype=dtype)))
    a = torch.tensor([tr, -tr, up, -up, dn, -dn, 0.0, -0.0, 1e-7, 5.0, -5.0], dtype=dtype)
    want = torch.tensor([0, 0, 1, 1, 0, 0, 0, 0, 0, 1, 1], dtype=torch.bool)
    assert torch.equal(oracle.torch_flags(a, t), want)                       # reference expression (__init__.py:41)
    assert torch.equal(~(a.abs() <= t), want)                               # reference expression (ugly_utils.py:897)
    assert torch.equal(a.float().abs() > oracle.c_round(dtype, t), want)    # C oracle's rule
    # SparseSiLU (nn.Threshold) keeps the same set
    xs = torch.tensor([-3.0, -0.05, 0.0, 0.05, 0.2, 3.0])      # silu: -0.142, -0.024, 0, 0.026, 0.110, 2.858
    kept = oracle.torch_sparse_silu(xs, 0.1)
    assert torch.equal(kept != 0, torch.tensor([1, 0, 0, 0, 1, 1], dtype=torch.bool))
    assert torch.equal(kept != 0, oracle.torch_flags(F.silu(xs), 0.1))
    # the rounding of t itself matters: a threshold just below a representable value rounds up to it
    if dtype != torch.float32:
        t2 = tr - 1e-7
        assert float(torch.tensor(t2).to(dtype)) == tr
        assert not bool(oracle.torch_flags(torch.tensor([tr], dtype=dtype), t2)[0])
        assert oracle.c_round(dtype, t2) == tr
    # negative threshold: everything is active, including exact zeros
    assert bool(oracle.torch_flags(torch.zeros(3, dtype=dtype), -1.0).all())


def test_gate_flags_through_c_oracle_on_crafted_rows(oracle):
    """x = e_0 picks column 0 of wgate, so a[j] = round(silu(wgate[j, 0])) exactly -- no summation involved."""
    for dtype in DTYPES:
        H, I = 16, 12
        x = torch.zeros(1, H, dtype=dtype); x[0, 0] = 1.0
        g = torch.linspace(-3, 3, I).to(dtype)
        wg = torch.zeros(I, H, dtype=dtype); wg[:, 0] = g
        a, flag = oracle.c_gate(x, wg, 0.2)
        want_a = F.silu(g.double()).to(dtype)       # correctly rounded silu of the stored gate value
        ulp = {torch.float32: 1.2e-7, torch.float16: 9.8e-4, torch.bfloat16: 7.9e-3}[dtype]
        torch.testing.assert_close(a[0].float(), want_a.float(), rtol=ulp, atol=0)   # at most one unit in the last place
        assert torch.equal(flag[0], a[0].abs() > 0.2)
        assert int(flag.sum()) == int((want_a.abs() > 0.2).sum())


# ---- the MLP ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_c_mlp_matches_reference_formula(oracle, dtype):
    """C restatement vs the literal four lines of ugly_utils.py:895-899 on CPU tensors."""
    tol = {torch.float32: dict(rtol=1e-5, atol=1e-6), torch.float16: dict(rtol=2e-3, atol=2e-4), torch.bfloat16: dict(rtol=1.6e-2, atol=2e-3)}[dtype]
    for (H, I, B, seed) in ((64, 96, 1, 0), (128, 200, 3, 1), (256, 384, 2, 2)):
        m = make_mlp(H, I, B, dtype, seed)
        a_abs = F.silu(F.linear(m["x"].float(), m["wg"].float())).abs().flatten()
        for q in (0.3, 0.7):
            t = float(torch.quantile(a_abs, q))
            r = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
            y_t, a_t, dead = oracle.torch_cats_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
            torch.testing.assert_close(r["a"].float(), a_t.float(), **tol)
            flips = r["flag"] != ~dead
            # a flag may only differ where the two gate values straddle t by a rounding step
            assert int(flips.sum()) <= 2
            if not flips.any():
                torch.testing.assert_close(r["y"].float(), y_t.float(), **tol)
            # and with identical gate values the outputs must agree regardless
            r2 = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a_t, flag_in=~dead)
            torch.testing.assert_close(r2["y"].float(), y_t.float(), **tol)


def test_c_mlp_float64_brute_force(oracle):
    """fp32 oracle vs an independent float64 loop-free evaluation with the mask taken from the oracle."""
    m = make_mlp(48, 80, 2, torch.float32, seed=7)
    t = 0.15
    r = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
    x, wg, wu, wd = (m[k].double() for k in ("x", "wg", "wu", "wd"))
    g = x @ wg.t()
    a = g / (1 + torch.exp(-g))
    assert torch.equal(r["flag"], a.abs().float() > t) or int((r["flag"] != (a.abs() > t)).sum()) == 0
    y = ((a * r["flag"]) * (x @ wu.t())) @ wd.t()
    torch.testing.assert_close(r["y"].double(), y, rtol=1e-5, atol=1e-6)
    # a transposed down weight or a dropped up factor would not survive this
    y_wrong = ((a * r["flag"])) @ wd.t()
    assert not torch.allclose(r["y"].double(), y_wrong, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_special_cases(oracle, dtype):
    m = make_mlp(128, 160, 2, dtype, seed=3)
    # all active: the dense SwiGLU MLP, three library GEMVs
    r = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], -1.0)
    assert bool(r["flag"].all())
    dense = oracle.torch_dense_mlp(m["x"].float(), m["wg"].float(), m["wu"].float(), m["wd"].float())
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=3e-3)
    torch.testing.assert_close(r["y"].float(), dense, **tol)
    # all dead: exact zeros
    r = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], float("inf"))
    assert not bool(r["flag"].any()) and torch.count_nonzero(r["y"]) == 0
    # one live neuron: y = round(z_j * wd[:, j]) -- one product per output, no sum
    a = oracle.c_gate(m["x"][:1], m["wg"], -1.0)[0].float().abs().flatten()
    top = a.sort(descending=True).values
    t = float((top[0] + top[1]) / 2)
    r = oracle.c_mlp(m["x"][:1], m["wg"], m["wu"], m["wd"], t)
    assert int(r["flag"].sum()) == 1
    j = int(r["flag"].flatten().nonzero()[0])
    want = (r["z"][0, j].float() * m["wd"][:, j].float()).to(dtype)
    assert torch.equal(r["y"][0], want)


def test_sparse_up_down_equal_dense_on_masked_operands(oracle):
    for dtype in DTYPES:
        m = make_mlp(96, 144, 3, dtype, seed=9, corr=0.5)
        a, flag = oracle.c_gate(m["x"], m["wg"], 0.05)
        z = oracle.c_sparse_up(m["x"], m["wu"], a, flag)
        want_z = (m["x"].double() @ m["wu"].double().t()) * a.double() * flag
        torch.testing.assert_close(z.double(), want_z, rtol=1e-6, atol=1e-9)
        zt = z.to(dtype)
        y = oracle.c_sparse_down(zt, m["wdt"], flag)
        torch.testing.assert_close(y.double(), zt.double() @ m["wdt"].double(), rtol=1e-6, atol=1e-7)
        # union semantics: a row's own dead entries are zero in z, so the union does not leak across rows
        for b in range(3):
            yb = oracle.c_sparse_down(zt[b:b + 1], m["wdt"], flag[b:b + 1])
            torch.testing.assert_close(yb[0], y[b], rtol=1e-6, atol=1e-7)


def test_compact_list(oracle):
    g = torch.Generator().manual_seed(0)
    for n in (1, 7, 64, 65, 1000):
        flag = torch.rand(n, generator=g) > 0.4
        idx, cnt = oracle.c_compact(flag)
        assert cnt == int(flag.sum()) and torch.equal(idx, flag.nonzero().flatten())
    idx, cnt = oracle.c_compact(torch.zeros(10, dtype=torch.bool))
    assert cnt == 0 and idx.numel() == 0


# ---- threshold calibration ---------------------------------------------------------------------------------------------

def test_histogram_bins_and_counts(oracle):
    edges = oracle.histogram_bins()
    assert edges.numel() == 1000 and math.isinf(float(edges[0])) and math.isinf(float(edges[-1]))
    assert abs(float(edges[2] - edges[1]) - 2.0 / 997) < 1e-6
    g = torch.Generator().manual_seed(0)
    v = torch.cat([torch.randn(5000, generator=g), torch.tensor([-1.0, 1.0, 0.0, 5.0, -5.0])])
    want = torch.histogram(v, bins=edges)[0]
    got = oracle.c_histogram(v, edges)
    assert torch.equal(got, want) and float(got.sum()) == v.numel()


def test_get_threshold_brute_force(oracle):
    """searchsorted(cumsum, s, right) == number of cumulative masses <= s; the returned edge is the LEFT edge of the
    first bin whose cumulative mass exceeds s -- checked on tiny histograms with exactly representable masses."""
    edges = torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0, 5.0])
    counts = torch.tensor([1.0, 1.0, 2.0, 0.0, 4.0])            # cdf: .125 .25 .5 .5 1.0
    for s, want_idx in ((0.0, 0), (0.1, 0), (0.125, 1), (0.2, 1), (0.25, 2), (0.4, 2), (0.5, 4), (0.75, 4), (0.99, 4)):
        t_c, idx_c = oracle.c_get_threshold(edges, counts, s)
        t_t = float(oracle.torch_get_threshold(edges, counts, s))
        brute = sum(1 for c in torch.cumsum(counts / counts.sum(), 0).tolist() if c <= s)
        assert idx_c == brute == want_idx, (s, idx_c, brute)
        assert t_c == t_t == float(edges[want_idx])
    # monotone in s, and on a real histogram the achieved sparsity lands within one bin's mass of the target
    g = torch.Generator().manual_seed(1)
    act = F.silu(torch.randn(200000, generator=g) * 1.3).abs()
    bins = oracle.histogram_bins()
    hist = torch.histogram(act, bins=bins)[0]
    last = -1.0
    for s in (0.1, 0.3, 0.5, 0.7, 0.9):
        t_c, idx = oracle.c_get_threshold(bins, hist, s)
        assert t_c == float(oracle.torch_get_threshold(bins, hist, s)) and t_c >= last
        last = t_c
        achieved = float((act <= t_c).float().mean())
        assert achieved <= s + 1e-6 and s - achieved <= float(hist.max() / hist.sum()) + 1e-6


def test_percentile_threshold(oracle):
    a = torch.arange(1, 101).float()
    assert oracle.percentile_threshold(a, 0.0) == -1.0
    t = oracle.percentile_threshold(a, 0.5)
    assert t == 50.0 and float((a <= t).float().mean()) == 0.5


# ---- RMS norm (the decoder layer's post-attention norm, folded into the fused entry point) -----------------------

def test_rms_norm_closed_forms(oracle):
    # a constant row: mean of squares = c^2, so norm(x) = c / sqrt(c^2 + eps) everywhere
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        h = torch.full((2, 1, 64), 3.0, dtype=dtype)
        w = torch.full((64,), 0.5, dtype=dtype)
        got = oracle.torch_rms_norm(h, w, 1e-5)
        want = 0.5 * 3.0 / (9.0 + 1e-5) ** 0.5
        assert got.dtype == dtype
        assert float((got.double() - want).abs().max()) <= want * float(torch.finfo(dtype).eps)
    # a one-hot row of length n with value v: mean = v^2 / n, norm = sign(v) * sqrt(n) (eps negligible), zeros stay zero
    h = torch.zeros(1, 1, 256)
    h[0, 0, 17] = -5.0
    got = oracle.torch_rms_norm(h, torch.ones(256), 0.0)
    assert float(got[0, 0, 17]) == pytest.approx(-16.0, rel=1e-6)
    assert int((got != 0).sum()) == 1
    # scale invariance: norm(k x) = norm(x) for eps = 0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 1, 128, generator=g)
    w = torch.randn(128, generator=g)
    torch.testing.assert_close(oracle.torch_rms_norm(4.0 * x, w, 0.0), oracle.torch_rms_norm(x, w, 0.0), rtol=1e-6, atol=1e-7)


def test_rms_norm_matches_installed_transformers(oracle):
    """The reference calls the HF module; the installed transformers is a later release than the one the reference
    pins, the RMS-norm forward is unchanged between them."""
    mod = pytest.importorskip("transformers.models.llama.modeling_llama")
    g = torch.Generator().manual_seed(1)
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        n = mod.LlamaRMSNorm(320, eps=1e-5)
        n.weight.data = torch.randn(320, generator=g).to(dtype)
        h = (torch.randn(4, 1, 320, generator=g) * 3).to(dtype)
        assert torch.equal(n(h), oracle.torch_rms_norm(h, n.weight.data, 1e-5))


def test_layer_tail_is_residual_plus_mlp_of_norm(oracle):
    g = torch.Generator().manual_seed(2)
    H, I = 64, 96
    h = torch.randn(2, 1, H, generator=g)
    nw, wg, wu, wd = torch.randn(H, generator=g), torch.randn(I, H, generator=g) * .1, torch.randn(I, H, generator=g) * .1, torch.randn(H, I, generator=g) * .1
    got = oracle.torch_layer_tail(h, nw, 1e-5, wg, wu, wd, 0.05)
    x = oracle.torch_rms_norm(h, nw, 1e-5)
    y, _, _ = oracle.torch_cats_mlp(x, wg, wu, wd, 0.05)
    assert torch.equal(got, h + y)
    # with t < 0 nothing is masked: the tail is the plain SwiGLU layer tail
    dense = h + oracle.torch_dense_mlp(x, wg, wu, wd)
    torch.testing.assert_close(oracle.torch_layer_tail(h, nw, 1e-5, wg, wu, wd, -1.0), dense)


# ---- frozen vectors --------------------------------------------------------------------------------------------

def test_oracle_reproduces_the_frozen_vectors_bit_for_bit(oracle):
    """tests/golden/cats_mlp_small.npz was written by this oracle (see make_fixtures.py there for why it is not a
    reference output); any change of its rounding points or accumulation shows up here."""
    cases = load_golden()
    assert set(cases) == {"f16_b1", "f16_b3", "bf16_b2", "f32_b2"}
    for name, c in cases.items():
        ref = oracle.c_mlp(c["x"], c["wg"], c["wu"], c["wd"], c["t"])
        assert torch.equal(ref["flag"], c["flag"]), name
        assert torch.equal(ref["a"].view(torch.int16 if c["dtype"] != torch.float32 else torch.int32),
                           c["a"].view(torch.int16 if c["dtype"] != torch.float32 else torch.int32)), name
        assert torch.equal(ref["y"].view(torch.int16 if c["dtype"] != torch.float32 else torch.int32),
                           c["y"].view(torch.int16 if c["dtype"] != torch.float32 else torch.int32)), name
        # and the literal PyTorch formula agrees with the frozen output to the parity tolerance
        y_t, _, dead = oracle.torch_cats_mlp(c["x"].float(), c["wg"].float(), c["wu"].float(), c["wd"].float(), c["t"])
        if torch.equal(~dead, c["flag"]):
            torch.testing.assert_close(y_t, c["y"].float(), rtol=1e-2, atol=2e-3 * max(1.0, float(c["y"].float().abs().max())))


def test_index_list_projections_brute_force_and_special_cases(oracle):
    """The index-list pair is pinned by plain float64 loops on a small case, by reducing to the dense library GEMV when
    the list is every row once, by linearity for duplicate entries, and by a wrong formula shown to fail."""
    g = torch.Generator().manual_seed(3)
    B, N, Z = 2, 24, 17
    x = torch.randn(B, N, generator=g)
    w = torch.randn(Z, N, generator=g)
    bias_up = torch.randn(Z, generator=g)
    idx = torch.tensor([5, 0, 16, 5, 9])     # unsorted, one duplicate
    scale = torch.randn(idx.numel(), generator=g)
    for act in ("id", "relu", "squared_relu", "swish"):
        got = oracle.torch_gather_gemv(x, w, idx, bias_up, act, scale)
        want = torch.zeros(B, idx.numel(), dtype=torch.float64)
        for b in range(B):
            for m, j in enumerate(idx.tolist()):
                v = sum(float(x[b, k]) * float(w[j, k]) for k in range(N)) + float(bias_up[j])
                if act == "relu":
                    v = max(v, 0.0)
                elif act == "squared_relu":
                    v = max(v, 0.0) ** 2
                elif act == "swish":
                    v = v / (1.0 + math.exp(-v))
                want[b, m] = v * float(scale[m])
        torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    # bias indexed by position instead of by weight row (a plausible slip) is a different function
    wrong = x @ w[idx].t() + bias_up[: idx.numel()]
    assert not torch.allclose(oracle.torch_gather_gemv(x, w, idx, bias_up), wrong, atol=1e-3)
    # the whole matrix once: the library's dense GEMV
    every = torch.arange(Z)
    torch.testing.assert_close(oracle.torch_gather_gemv(x, w, every), torch.nn.functional.linear(x, w))

    H = 11
    wd = torch.randn(Z, H, generator=g)
    z = torch.randn(B, idx.numel(), generator=g)
    bias_dn = torch.randn(H, generator=g)
    got = oracle.torch_gather_transposed_gemv(z, wd, idx, bias_dn)
    want = torch.zeros(B, H, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            want[b, h] = sum(float(z[b, m]) * float(wd[j, h]) for m, j in enumerate(idx.tolist())) + float(bias_dn[h])
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    # duplicates add: listing row 5 twice with z1, z2 equals listing it once with z1 + z2
    merged_idx = torch.tensor([5, 0, 16, 9])
    merged_z = torch.stack([z[:, 0] + z[:, 3], z[:, 1], z[:, 2], z[:, 4]], dim=1)
    torch.testing.assert_close(got, oracle.torch_gather_transposed_gemv(merged_z, wd, merged_idx, bias_dn), rtol=1e-5, atol=1e-5)
    # the whole matrix once: z @ wd, and the sorted active list reproduces the flag-based sparse down of the C oracle
    zz = torch.randn(B, Z, generator=g)
    torch.testing.assert_close(oracle.torch_gather_transposed_gemv(zz, wd, every), zz @ wd, rtol=1e-5, atol=1e-5)
    flag = torch.zeros(B, Z, dtype=torch.bool)
    flag[:, merged_idx] = True
    live = torch.nonzero(flag[0]).flatten()
    dense = oracle.c_sparse_down(torch.where(flag, zz, torch.zeros_like(zz)), wd, flag)
    torch.testing.assert_close(oracle.torch_gather_transposed_gemv(zz[:, live], wd, live), dense, rtol=1e-5, atol=1e-5)
