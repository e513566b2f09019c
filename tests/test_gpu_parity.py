"""GPU parity: the HIP kernels, called through the C ABI (cats_amd.capi -> libcats_gemv.so), against the CPU
oracle on the same seeded inputs.

Bar: masks bit-exact against the reference rule |a| > t evaluated on identical gate values (the kernel's own
stored activations); outputs within rtol 1e-2 / atol 2e-3 (fp16, bf16) and 1e-5 (fp32) of the dense-masked MLP.
"""
import math

import pytest
import torch

from tests.util import A_TOL, TOL, calibrate, dev, load_golden, make_mlp

pytestmark = pytest.mark.gpu

capi = None


@pytest.fixture(scope="module", autouse=True)
def _load():
    global capi
    assert torch.cuda.is_available(), "these tests need the GPU"
    from cats_amd import capi as _capi

    _capi.lib()
    capi = _capi


def _ws(B, H, I):
    return capi.Workspace(B, H, I)


def close(got, want, dtype):
    """The parity tolerance.  atol is stated for outputs of order one (the benchmark configurations); for the
    reference's U(-0.5, 0.5) recipe, whose outputs reach the hundreds, it scales with the largest output."""
    tol = dict(TOL[dtype])
    tol["atol"] *= max(1.0, float(want.float().abs().max()))
    torch.testing.assert_close(got.float(), want.float(), **tol)


def check_mlp_case(oracle, m, t, *, tag, ws=None, expect_flip_free=False):
    """Full set of parity checks for one (weights, x, threshold)."""
    dtype = m["x"].dtype
    B, H = m["x"].shape
    I = m["wg"].shape[0]
    print(f"[case] {tag} dtype={dtype} B={B} H={H} I={I} t={t}", flush=True)
    d = dev(m)
    ws = ws or _ws(B, H, I)

    a, flag = capi.gate_flag(d["x"], d["wg"], t)
    y, flag2, count = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
    if (I * m["x"].element_size()) % 16 == 0:
        y_rm = capi.mlp_rowmajor_down(d["x"], d["wg"], d["wu"], d["wd"], t, ws)
    else:  # rows of the (H, I) down weight are not 16-byte aligned: rejected, not mis-read
        with pytest.raises(capi.CatsError, match="aligned"):
            capi.mlp_rowmajor_down(d["x"], d["wg"], d["wu"], d["wd"], t, ws)
        y_rm = y
    # fp32-accumulate contract (fuse_gemv_gemv_gemv, flag_gemv_gemv_atomic): the call adds onto what the buffer holds
    y32 = torch.ones(B, H, dtype=torch.float32, device="cuda")
    _, flag32, count32 = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True, y_f32=y32)
    torch.cuda.synchronize()
    a, flag, y, flag2, y_rm = a.cpu(), flag.cpu(), y.cpu(), flag2.cpu(), y_rm.cpu()
    y32 = y32.cpu() - 1.0
    assert torch.equal(flag32.cpu(), flag2), f"{tag}: fp32-accumulate call disagrees on flags"
    assert int(count32.item()) == int(count.item()), f"{tag}: fp32-accumulate call disagrees on the active count"

    # 1. mask rule, bit-exact on identical gate values: torch's own comparison on the kernel's activations
    want_flag = torch.abs(a) > t
    assert torch.equal(flag, want_flag), f"{tag}: flag != (|a| > t) on the kernel's own a"
    assert torch.equal(flag2, flag), f"{tag}: the fused MLP pass and the gate pass disagree on flags"
    union = flag.any(dim=0)
    if count is not None:  # above 8 rows (two passes) this is the union of the flags, counted by one more small kernel
        assert int(count.item()) == int(union.sum()), f"{tag}: active count {int(count.item())} != {int(union.sum())}"
    # the C oracle's rule on the same activations (independent of torch's scalar casting)
    tr = oracle.c_round(dtype, t)
    assert torch.equal(flag, a.float().abs() > tr)

    # 2. activations vs the oracle's own gate stage
    ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
    a_tol = dict(A_TOL[dtype])
    a_tol["atol"] *= max(1.0, float(ref["a"].float().abs().max()))  # same scaling rule as close()
    torch.testing.assert_close(a.float(), ref["a"].float(), **a_tol)

    # 3. mask vs the oracle's mask on ITS gate values: may differ only within rounding distance of t
    flips = flag != ref["flag"]
    nflip = int(flips.sum())
    if nflip:
        band = a_tol["atol"] + a_tol["rtol"] * abs(tr)
        dist = (ref["a"].float().abs() - tr).abs()[flips]
        assert float(dist.max()) <= band, f"{tag}: {nflip} mask flips, one {float(dist.max())} away from t (band {band})"
    print(f"        active={int(union.sum())}/{I} flips_vs_oracle={nflip}", flush=True)
    if expect_flip_free:
        assert nflip == 0

    # 4. output vs the dense-masked oracle on identical gate values (kernel's a and flags fed to the oracle)
    ref_same = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a, flag_in=flag)
    close(y, ref_same["y"], dtype)
    close(y_rm, ref_same["y"], dtype)
    close(y32, ref_same["y"], dtype)  # atomics: summation order varies run to run, hence the tolerance and not bits
    # 5. and vs the fully independent oracle / the literal PyTorch formula when no flag flipped
    if nflip == 0:
        close(y, ref["y"], dtype)
        if dtype == torch.float32:
            y_t, _, dead = oracle.torch_cats_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
            if torch.equal(~dead, flag):
                close(y, y_t, dtype)
    return dict(y=y, a=a, flag=flag)


SMALL = [
    # H, I, B, dtype
    (64, 96, 1, torch.float16), (64, 96, 2, torch.bfloat16), (64, 96, 3, torch.float32),
    (72, 100, 1, torch.float16),      # H not a multiple of 64 vectors, I not a multiple of 8
    (520, 1000, 4, torch.float16), (512, 1024, 8, torch.bfloat16), (260, 333, 5, torch.float32),
    (4096, 512, 1, torch.float16), (2048, 640, 2, torch.float32), (8192, 256, 1, torch.bfloat16),
]


@pytest.mark.parametrize("H,I,B,dtype", SMALL)
@pytest.mark.parametrize("dist", ["normal", "uniform"])
def test_small_shapes(oracle, H, I, B, dtype, dist):
    m = make_mlp(H, I, B, dtype, seed=H * 7 + I + B, dist=dist)
    scale = 1.0 if dist == "normal" else 1.0
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    for q in (0.0, 0.5, 0.9):
        t = -1.0 if q == 0.0 else float(torch.quantile(a_abs, q)) * scale
        check_mlp_case(oracle, m, t, tag=f"small-{dist}-q{q}")


def _random_shapes(n, seed):
    import random

    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dtype = [torch.float16, torch.bfloat16, torch.float32][i % 3]
        vec = 4 if dtype == torch.float32 else 8
        H = vec * rnd.choice([1, 2, 3, 9, 31, 64, 65, 100, 128, 255, 256, 512, 513])   # rows are whole 16-byte vectors
        I = rnd.choice([1, 2, 7, 8, 9, 63, 64, 65, 127, 200, 343, 344, 345, 1000, 2049])
        out.append((H, I, rnd.randint(1, 8), dtype))
    return out


@pytest.mark.parametrize("H,I,B,dtype", _random_shapes(24, seed=2024))
def test_seeded_random_shapes(oracle, H, I, B, dtype):
    """Odd sizes on purpose: rows of one vector, fewer neurons than a mask byte, ranges that end inside a byte,
    lists of odd length (the down kernel pairs rows), every batch size."""
    m = make_mlp(H, I, B, dtype, seed=H * 31 + I * 7 + B)
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    for q in (0.0, 0.4, 0.8):
        t = -1.0 if q == 0.0 else float(torch.quantile(a_abs, q))
        check_mlp_case(oracle, m, t, tag=f"random-q{q}")


def test_frozen_vectors():
    """The committed vectors (tests/golden): flags bit-exact wherever the activation is not within rounding distance of
    the threshold, activations and outputs to the parity tolerance."""
    for name, c in load_golden().items():
        dtype = c["dtype"]
        B, H = c["x"].shape
        I = c["wg"].shape[0]
        d = {k: c[k].cuda() for k in ("x", "wg", "wu", "wdt")}
        a, flag = capi.gate_flag(d["x"], d["wg"], c["t"])
        y = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], c["t"], _ws(B, H, I))
        torch.cuda.synchronize()
        a, flag, y = a.cpu(), flag.cpu(), y.cpu()
        torch.testing.assert_close(a.float(), c["a"].float(), **A_TOL[dtype])
        flips = flag != c["flag"]
        if int(flips.sum()):
            band = A_TOL[dtype]["atol"] + A_TOL[dtype]["rtol"] * abs(c["t"])
            assert float((c["a"].float().abs() - c["t"]).abs()[flips].max()) <= band, name
        else:
            close(y, c["y"], dtype)


def test_all_dead_and_all_active(oracle):
    m = make_mlp(512, 768, 2, torch.float16, seed=5)
    d = dev(m)
    ws = _ws(2, 512, 768)
    y = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], float("inf"), ws)
    assert torch.count_nonzero(y) == 0
    # a second call on the same workspace after an all-dead call must still be right (accumulator stays clean)
    y = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], -1.0, ws)
    dense = oracle.torch_dense_mlp(m["x"].float(), m["wg"].float(), m["wu"].float(), m["wd"].float())
    torch.testing.assert_close(y.cpu().float(), dense, **TOL[torch.float16])


def test_single_active_neuron_is_exact(oracle):
    """One live neuron: y = round(z_j * wdown_t[j, :]) -- a single product per column, bit-checkable."""
    for dtype in (torch.float16, torch.bfloat16, torch.float32):
        m = make_mlp(256, 384, 1, dtype, seed=11)
        d = dev(m)
        a, _ = capi.gate_flag(d["x"], d["wg"], -1.0)
        mags = a.float().abs().flatten().sort(descending=True).values
        assert mags[0] > mags[1]
        t = float((mags[0] + mags[1]) / 2)
        ws = _ws(1, 256, 384)
        y, flag, count = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        assert int(count.item()) == 1 and int(flag.sum()) == 1
        j = int(flag.flatten().nonzero()[0])
        z = capi.gate_up(d["x"], d["wg"], d["wu"], t)[0][0, j]
        want = (z.float() * d["wdt"][j].float()).to(dtype)
        assert torch.equal(y[0], want), f"{dtype}: single-neuron output is not the exact product"


def test_workspace_reuse_and_repeatability(oracle):
    """Back-to-back calls on one workspace (different thresholds and batch sizes) do not contaminate each other."""
    H, I = 1024, 2048
    ws = _ws(8, H, I)
    outs = {}
    for rep in range(2):
        for B, q in ((8, 0.5), (1, 0.9), (4, 0.0), (2, 0.7)):
            m = make_mlp(H, I, B, torch.float16, seed=100 + B)
            a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
            t = -1.0 if q == 0.0 else float(torch.quantile(a_abs, q))
            d = dev(m)
            y = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws).cpu()
            ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
            torch.testing.assert_close(y.float(), ref["y"].float(), **TOL[torch.float16])
            if rep == 0:
                outs[B] = y
            else:
                torch.testing.assert_close(y.float(), outs[B].float(), **TOL[torch.float16])


def test_batch_rows_are_independent(oracle):
    """Row b of a batched call equals the single-row call on x[b] (union gathering must not leak between rows)."""
    H, I, B = 1024, 1536, 4
    m = make_mlp(H, I, B, torch.float16, seed=21, corr=0.5)
    t = calibrate(m["wg"], [0.5])[0]
    d = dev(m)
    ws = _ws(B, H, I)
    yb, fb, _ = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
    for b in range(B):
        y1, f1, _ = capi.mlp(d["x"][b:b + 1].contiguous(), d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        assert torch.equal(f1[0], fb[b])
        torch.testing.assert_close(y1[0].float(), yb[b].float(), **TOL[torch.float16])


@pytest.mark.parametrize("H,I,B,dtype", [(4096, 1000, 1, torch.float16), (520, 333, 3, torch.bfloat16), (260, 96, 8, torch.float32),
                                         (4096, 11008, 1, torch.float16), (512, 200, 12, torch.float16),
                                         # 3..8 rows of a 16-bit type with rows of 2048 / 4096 elements: the matrix-core up kernel
                                         (4096, 1003, 3, torch.float16), (2048, 777, 7, torch.bfloat16), (4096, 11008, 4, torch.float16),
                                         (2048, 64, 8, torch.float16), (4096, 8, 5, torch.bfloat16), (4096, 520, 12, torch.float16)])
def test_up_down_given_the_gate_activations(oracle, H, I, B, dtype):
    """cats_up_down (the reference's gemv_gemv_triton): the caller supplies a = act(gate(x)); flags = |a| > t are derived
    on the device and must be the ones torch derives; output against the oracle on those activations and flags."""
    m = make_mlp(H, I, B, dtype, seed=3 * H + I + B)
    a = oracle.c_gate(m["x"], m["wg"], -1.0)[0]                       # (B, I) in dtype
    t = float(torch.quantile(a.float().abs().flatten(), 0.5))
    flag = torch.abs(a) > t
    d = dev(m)
    ws = _ws(B, H, I)
    y = capi.up_down(d["x"], a.cuda(), d["wu"], d["wdt"], t, ws)
    torch.cuda.synchronize()
    ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a, flag_in=flag)
    close(y.cpu(), ref["y"], dtype)
    # and the two-call spelling gives the same bits
    z = capi.up_flag(d["x"], d["wu"], a.cuda(), flag.cuda())
    y2 = capi.down_flag(z, d["wdt"], flag.cuda(), ws)
    torch.cuda.synchronize()
    close(y.cpu(), y2.cpu(), dtype)
    # the sparse up call alone: against the oracle's z, as fp32 (the same values before the last rounding is undone:
    # z is rounded to the storage type either way), and in place over a (the reference's fuse_flag_gemv_local contract)
    close(z.cpu(), ref["z"], dtype)
    z32 = capi.up_flag(d["x"], d["wu"], a.cuda(), flag.cuda(), out_f32=True)
    a_inplace = a.cuda().clone()
    capi.check(capi.lib().cats_up_flag(capi._p(d["x"]), capi._p(d["wu"]), capi._p(a_inplace), capi._p(flag.cuda()), capi._p(a_inplace), 0,
                                       B, H, I, capi.DTYPE_CODE[dtype], capi._stream(a_inplace)), "cats_up_flag in place")
    torch.cuda.synchronize()
    assert torch.equal(z32.to(dtype), z)
    assert torch.equal(a_inplace, z)
    assert torch.equal(z.cpu()[~flag], torch.zeros_like(z.cpu()[~flag]))
    # thresholds that keep everything and nothing, and the wave-per-row kernels on the same call
    for t2 in (-1.0, 1e9):
        y3 = capi.up_down(d["x"], a.cuda(), d["wu"], d["wdt"], t2, ws)
        try:
            capi.set_tuning(-1, 0, 0, 0)
            y4 = capi.up_down(d["x"], a.cuda(), d["wu"], d["wdt"], t2, ws)
        finally:
            capi.set_tuning(0, 0, 0, 0)
        torch.cuda.synchronize()
        ref2 = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t2, a_in=a, flag_in=torch.abs(a) > t2)
        close(y3.cpu(), ref2["y"], dtype)
        close(y4.cpu(), ref2["y"], dtype)


def test_gate_compact_list(oracle):
    # 11008 neurons = 1376 mask bytes = six workgroups of the list kernel; 2051 ends inside a byte; 20000 is three passes per workgroup
    for (H, I, dtype) in ((64, 96, torch.float16), (512, 1000, torch.bfloat16), (4096, 2048, torch.float16), (256, 300, torch.float32),
                          (4096, 11008, torch.float16), (128, 2051, torch.bfloat16), (64, 20000, torch.float16), (64, 150000, torch.float16)):
        m = make_mlp(H, I, 1, dtype, seed=31)
        d = dev(m)
        ws = _ws(1, H, I)
        for q in (0.0, 0.5, 0.95, 1.1):
            a_ref, _ = capi.gate_flag(d["x"], d["wg"], -1.0)
            mags = a_ref.float().abs().flatten()
            t = -1.0 if q == 0.0 else (float("inf") if q > 1 else float(torch.quantile(mags, q)))
            for _ in range(2):  # twice: nothing may be left behind in the workspace
                vals, idx, n = capi.gate_compact(d["x"], d["wg"], t, ws)
                a, flag = capi.gate_flag(d["x"], d["wg"], t)
                want_idx, want_n = oracle.c_compact(flag[0])
                assert n == want_n == int(flag.sum())
                assert torch.equal(idx[:n].cpu(), want_idx), "index list is not ascending nonzero(mask)"
                assert torch.equal(vals[:n].cpu(), a[0].cpu()[want_idx])


INDEX_LIST = [
    # H (row length), Z (rows of the weight), M (list length), B, dtype
    (4096, 11008, 5500, 1, torch.float16), (4096, 2048, 700, 2, torch.bfloat16), (520, 1000, 333, 3, torch.float16),
    (260, 333, 333, 4, torch.float32), (4096, 512, 1, 1, torch.float16), (2048, 640, 77, 8, torch.bfloat16), (64, 96, 200, 2, torch.float32),
]


@pytest.mark.parametrize("H,Z,M,B,dtype", INDEX_LIST)
def test_index_list_up_and_down(oracle, H, Z, M, B, dtype):
    """cats_up_index / cats_down_index through the C ABI against the reference's formulas (oracle.torch_gather_gemv /
    torch_gather_transposed_gemv): sorted lists, unsorted lists with duplicates (M may exceed Z), bias, every activation,
    the compact scale vector, entries outside the matrix, the empty list."""
    g = torch.Generator().manual_seed(H + Z + M)
    x = torch.randn(B, H, generator=g).to(dtype)
    w = (torch.randn(Z, H, generator=g) * 0.05).to(dtype)
    wd = (torch.randn(Z, H, generator=g) * 0.05).to(dtype)
    bias_up = torch.randn(Z, generator=g).to(dtype)
    bias_dn = torch.randn(H, generator=g).to(dtype)
    sorted_idx = torch.sort(torch.randperm(Z, generator=g)[: min(M, Z)]).values
    any_idx = torch.randint(0, Z, (M,), generator=g)
    ws = _ws(B, H, Z)
    dx, dw, dwd = x.cuda(), w.cuda(), wd.cuda()
    for idx in (sorted_idx, any_idx):
        di = idx.cuda()
        scale = torch.randn(idx.numel(), generator=g).to(dtype)
        for act in ("id", "relu", "squared_relu", "swish"):
            for b_, sc in ((None, None), (bias_up, None), (None, scale), (bias_up, scale)):
                got = capi.up_index(dx, dw, di, None if b_ is None else b_.cuda(), None if sc is None else sc.cuda(), act)
                want = oracle.torch_gather_gemv(x, w, idx, b_, act, sc)
                close(got.cpu(), want, dtype)
        z = (torch.randn(B, idx.numel(), generator=g) * 0.5).to(dtype)
        for b_ in (None, bias_dn):
            got = capi.down_index(z.cuda(), dwd, di, ws, None if b_ is None else b_.cuda())
            want = oracle.torch_gather_transposed_gemv(z, wd, idx, b_)
            close(got.cpu(), want, dtype)
            again = capi.down_index(z.cuda(), dwd, di, ws, None if b_ is None else b_.cuda())
            assert torch.equal(got, again), "index-list down is not repeatable bit for bit"
    # entries outside [0, Z) give 0 (up) / contribute nothing (down) instead of reading outside the matrix
    bad = any_idx.clone()
    bad[::3] = Z + 5
    bad[1::7] = -1
    ok = (bad >= 0) & (bad < Z)
    got = capi.up_index(dx, dw, bad.cuda())
    want = oracle.torch_gather_gemv(x, w, bad.clamp(0, Z - 1))
    want[:, ~ok] = 0
    close(got.cpu(), want, dtype)
    z = (torch.randn(B, M, generator=g) * 0.5).to(dtype)
    got = capi.down_index(z.cuda(), dwd, bad.cuda(), ws)
    close(got.cpu(), oracle.torch_gather_transposed_gemv(z[:, ok], wd, bad[ok]), dtype)
    # the empty list: y = bias, or zeros
    empty = torch.zeros(0, dtype=torch.int64, device="cuda")
    ze = torch.zeros(B, 0, dtype=dtype, device="cuda")
    assert torch.equal(capi.down_index(ze, dwd, empty, ws).cpu(), torch.zeros(B, H, dtype=dtype))
    assert torch.equal(capi.down_index(ze, dwd, empty, ws, bias_dn.cuda()).cpu(), bias_dn.expand(B, H))
    assert capi.up_index(dx, dw, empty).shape == (B, 0)


def test_index_list_package_functions(oracle):
    """The reference's Python names on top of the index-list kernels: gather_gemv (batch 1..4, bias, activations),
    gather_transposed_gemv, the *_indirect_index_2d pair and both composites, against the oracle's formulas."""
    import flash_gemv as fg
    from flash_gemv import kernels as K

    g = torch.Generator().manual_seed(12)
    H, Z = 1024, 1536
    dtype = torch.float16
    w = (torch.randn(Z, H, generator=g) * 0.05).to(dtype)
    wdt = (torch.randn(Z, H, generator=g) * 0.05).to(dtype)
    bias = torch.randn(Z, generator=g).to(dtype)
    for batch in (1, 2, 3, 4):
        x = torch.randn(batch, H, generator=g).to(dtype)
        idx = torch.sort(torch.randperm(Z, generator=g)[:500]).values
        for act in ("id", "relu", "squared_relu", "swish"):
            for b_ in (None, bias):
                got = K.gather_gemv(x.cuda(), w.cuda(), idx.cuda(), None if b_ is None else b_.cuda(), act)
                close(got.cpu(), oracle.torch_gather_gemv(x, w, idx, b_, act), dtype)
        z = (torch.randn(batch, 500, generator=g) * 0.5).to(dtype)
        hb = torch.randn(H, generator=g).to(dtype)
        close(K.gather_transposed_gemv(z.cuda(), wdt.cuda(), idx.cuda()).cpu(), oracle.torch_gather_transposed_gemv(z, wdt, idx), dtype)
        close(K.gather_transposed_gemv(z.cuda(), wdt.cuda(), idx.cuda(), hb.cuda()).cpu(), oracle.torch_gather_transposed_gemv(z, wdt, idx, hb), dtype)
    x = torch.randn(1, H, generator=g).to(dtype)
    x1 = torch.randn(500, generator=g).to(dtype)
    close(K.gather_gemv_elemul_indirect_index_2d(x.cuda(), x1.cuda(), w.cuda(), idx.cuda()).cpu(), oracle.torch_gather_gemv(x, w, idx, scale=x1), dtype)
    z1 = (oracle.torch_gather_gemv(x, w, idx).float() * x1.float()).to(dtype)
    want = oracle.torch_gather_transposed_gemv(z1, wdt, idx)
    close(K.mistral_mlp_partial_sparse(x.cuda(), x1.cuda(), w.cuda(), wdt.cuda(), idx.cuda()).cpu(), want, dtype)
    close(K.mistral_mlp_sparse_direct_index_2d(x.cuda(), x1.cuda(), w.cuda(), wdt.cuda(), idx.cuda()).cpu(), want, dtype)
    # the whole-MLP composites: gate in torch, sorted active list, index-list up and down == the flag-based path
    wg_t = (torch.randn(H, Z, generator=g) * 0.02).to(dtype)
    t = 0.05
    a = fg.flag_gemv_gemv_dejavu(x.cuda(), wg_t.cuda(), w.cuda(), wdt.cuda(), t)
    b = fg.flag_gemv_gemv_fuse_dejavu(x.cuda(), wg_t.cuda(), w.cuda(), wdt.cuda(), t)
    c = fg.flag_gemv_gemv_triton(x.cuda().view(1, 1, H), wg_t.cuda(), w.cuda(), wdt.cuda(), t)
    close(a.cpu(), c.view(1, H).cpu(), dtype)
    close(b.cpu(), c.view(1, H).cpu(), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_mask_boundaries_on_the_device(oracle, dtype):
    """Crafted activations around the threshold, on every copy of the rule the kernels carry.

    With x = e_0 the gate pre-activation of neuron j is exactly wgate[j, 0], so the stored activation a_j =
    round(silu(wgate[j, 0])) can be steered: the first column holds a ladder of values whose activations straddle
    candidate thresholds.  Thresholds are then taken FROM the stored activations of the kernel -- a == t exactly, the
    neighbouring representable values on either side, -t, 0, a value below every |a| and +inf -- and the flags of
    (i) the gate kernel (wave-per-row at 1 and 2 rows, matrix-core at 4 and 8 rows), (ii) the single-pass MLP kernel,
    (iii) the two-kernel MLP path and (iv) cats_up_down, which derives flags from a supplied a, must all equal
    torch.abs(a) > t and the C oracle's comparison, bit for bit (experiments/models/sparse_silu/ugly_utils.py:897,
    flash_gemv/flash_gemv/__init__.py:41,46)."""
    H, I = 4096, 512
    g = torch.Generator().manual_seed(9)
    ladder = torch.cat([torch.linspace(-6, 6, I - 8), torch.tensor([0.0, -0.0, 1e-7, -1e-7, 6e-8, 1.0, -1.0, 0.5])])
    wg = torch.zeros(I, H)
    wg[:, 0] = ladder
    wg = wg.to(dtype)
    wu = (torch.randn(I, H, generator=g) * 0.02).to(dtype)
    wdt = (torch.randn(I, H, generator=g) * 0.02).to(dtype)
    for B in (1, 2, 4, 8):
        x = torch.zeros(B, H)
        x[:, 0] = 1.0
        x = x.to(dtype)
        dx, dwg, dwu, dwdt = x.cuda(), wg.cuda(), wu.cuda(), wdt.cuda()
        ws = _ws(B, H, I)
        a0, _ = capi.gate_flag(dx, dwg, -1.0)
        a0 = a0.cpu()
        torch.testing.assert_close(a0[0].float(), torch.nn.functional.silu(wg[:, 0].float()), **A_TOL[dtype])  # a = round(silu(w)) for x = e_0
        mags = torch.unique(a0[0].float().abs())
        mid = mags[mags.numel() // 2]          # a positive value that some neuron's |a| equals exactly
        itype = torch.int32 if dtype == torch.float32 else torch.int16
        mid_bits = mid.to(dtype).view(itype)
        up1 = (mid_bits + 1).view(dtype).float()   # neighbouring representable values of the storage type
        dn1 = (mid_bits - 1).view(dtype).float()
        small = mags[mags > 0].min()
        cands = [float(mid), float(up1), float(dn1), -float(mid), 0.0, -0.0, float(small), float(small) / 2, -1.0, float(mags.max()), float("inf"),
                 float(mid) * (1 + 1e-4), float(mid) * (1 - 1e-4)]   # the last two are not representable in 16 bits: the threshold itself gets rounded
        for t in cands:
            a, flag = capi.gate_flag(dx, dwg, t)
            want = torch.abs(a) > t                      # torch's own comparison on the kernel's activations, on the device
            assert torch.equal(flag, want), f"gate flags differ from |a| > t at t={t} B={B}"
            tr = oracle.c_round(dtype, t)
            assert torch.equal(flag.cpu(), a.cpu().float().abs() > tr), f"gate flags differ from the C oracle's rule at t={t}"
            _, f_mlp, cnt = capi.mlp(dx, dwg, dwu, dwdt, t, ws, want_flag=True, want_count=True)
            assert torch.equal(f_mlp, want) and int(cnt) == int(want.any(dim=0).sum()), f"MLP flags differ at t={t} B={B}"
            try:
                capi.set_tuning(0, 0, 0, 1)
                _, f_two, cnt2 = capi.mlp(dx, dwg, dwu, dwdt, t, ws, want_flag=True, want_count=True)
                y_two = capi.up_down(dx, a, dwu, dwdt, t, ws)
            finally:
                capi.set_tuning(0, 0, 0, 0)
            assert torch.equal(f_two, want) and int(cnt2) == int(want.any(dim=0).sum()), f"two-kernel MLP flags differ at t={t} B={B}"
            # cats_up_down derives its flags from the supplied a: same output as feeding it a with the dropped entries zeroed
            # and a threshold below everything that is left
            y_a = capi.up_down(dx, a, dwu, dwdt, t, ws)
            a_masked = torch.where(want, a, torch.zeros_like(a))
            flag_masked = a_masked != 0
            z = capi.up_flag(dx, dwu, a_masked, flag_masked)
            y_ref = capi.down_flag(z, dwdt, flag_masked, ws)
            close(y_a.cpu(), y_ref.cpu(), dtype)
            close(y_two.cpu(), y_ref.cpu(), dtype)


def test_sparse_up_and_down_ops(oracle):
    """The stand-alone flag-driven up / down entry points against the oracle's restatement of the Triton pair."""
    for (H, I, B, dtype) in ((512, 1024, 1, torch.float16), (1024, 1000, 3, torch.bfloat16), (256, 512, 2, torch.float32), (4096, 1024, 4, torch.float16),
                             (4096, 1024, 12, torch.bfloat16), (2048, 520, 16, torch.float16)):   # 9..16 rows: gate + up and down in one pass each
        m = make_mlp(H, I, B, dtype, seed=41, corr=0.5)
        d = dev(m)
        t = calibrate(m["wg"], [0.6])[0]
        a, flag = capi.gate_flag(d["x"], d["wg"], t)
        z32 = capi.up_flag(d["x"], d["wu"], a, flag, out_f32=True)
        zt = capi.up_flag(d["x"], d["wu"], a, flag, out_f32=False)
        want_z = oracle.c_sparse_up(m["x"], m["wu"], a, flag)
        torch.testing.assert_close(z32.cpu(), want_z, **TOL[dtype])
        torch.testing.assert_close(zt.cpu().float(), want_z, **TOL[dtype])
        assert torch.count_nonzero(zt[~flag]) == 0
        ws = _ws(B, H, I)
        y = capi.down_flag(zt, d["wdt"], flag, ws)
        want_y = oracle.c_sparse_down(zt, m["wdt"], flag)
        torch.testing.assert_close(y.cpu().float(), want_y, **TOL[dtype])
        acc = torch.ones(B, H, dtype=torch.float32, device="cuda")   # accumulate mode: adds onto what is there
        capi.down_flag(zt, d["wdt"], flag, ws, accumulate_into=acc)
        tol = dict(TOL[dtype]); tol["atol"] = max(tol["atol"], 1e-4)
        torch.testing.assert_close(acc.cpu() - 1.0, want_y, **tol)
        gu, gflag = capi.gate_up(d["x"], d["wg"], d["wu"], t)
        assert torch.equal(gflag, flag)
        torch.testing.assert_close(gu.cpu().float(), want_z, **TOL[dtype])


# ---- the benchmark configurations at full size ---------------------------------------------------------------

@pytest.fixture(scope="module")
def llama_fp16():
    return make_mlp(4096, 11008, 1, torch.float16, seed=0)


def test_config2_llama_fp16_sweep(oracle, llama_fp16):
    m = llama_fp16
    ts = calibrate(m["wg"], [0.0, 0.3, 0.5, 0.7, 0.9])
    ws = _ws(1, 4096, 11008)
    for s, t in zip([0.0, 0.3, 0.5, 0.7, 0.9], ts):
        r = check_mlp_case(oracle, m, t, tag=f"llama-fp16-s{s}", ws=ws)
        got = 1.0 - float(r["flag"].float().mean())
        assert abs(got - s) < 0.03, f"sparsity {got} far from target {s}"


def test_config2_all_active_matches_dense_gemv(oracle, llama_fp16):
    """0 % sparsity reduces to the dense SwiGLU MLP = three library GEMVs (rocBLAS through torch, on the GPU)."""
    d = dev(llama_fp16)
    ws = _ws(1, 4096, 11008)
    y = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], -1.0, ws)
    dense = oracle.torch_dense_mlp(d["x"], d["wg"], d["wu"], d["wd"])
    torch.testing.assert_close(y.float(), dense.float(), **TOL[torch.float16])


def test_config1_llama_fp32(oracle):
    m = make_mlp(4096, 11008, 1, torch.float32, seed=0)
    t = calibrate(m["wg"], [0.5])[0]
    check_mlp_case(oracle, m, t, tag="llama-fp32-s0.5")


def test_config3_mistral_bf16_heavy_tail(oracle):
    m = make_mlp(4096, 14336, 1, torch.bfloat16, seed=3, heavy_tail=True)
    for s, t in zip([0.5, 0.7], calibrate(m["wg"], [0.5, 0.7])):
        check_mlp_case(oracle, m, t, tag=f"mistral-bf16-s{s}")


@pytest.mark.parametrize("B", [2, 4, 8])
def test_config4_small_batch_union(oracle, B):
    m = make_mlp(4096, 11008, B, torch.float16, seed=4, corr=0.5)
    t = calibrate(m["wg"], [0.5])[0]
    r = check_mlp_case(oracle, m, t, tag=f"llama-fp16-B{B}")
    union_sparsity = 1.0 - float(r["flag"].any(dim=0).float().mean())
    row_sparsity = 1.0 - float(r["flag"].float().mean())
    print(f"        B={B} per-row sparsity {row_sparsity:.3f} union sparsity {union_sparsity:.3f}", flush=True)
    assert union_sparsity <= row_sparsity + 1e-6


MATRIX_CORE = [
    # H, I, B, dtype -- 3..8 batch rows in 16-bit types with a row length of 2048 or 4096 take the matrix-core
    # gate / gate+up kernel (one workgroup per CU, each with ceil(I / workgroups) consecutive rows in tiles of 8)
    (4096, 1003, 3, torch.float16),    # 4 rows per workgroup on 256 CUs: half a tile each, the last workgroup has 3 rows
    (4096, 520, 5, torch.bfloat16),
    (2048, 777, 7, torch.float16),
    (2048, 64, 8, torch.bfloat16),
    (4096, 8, 4, torch.float16),       # a single tile
    (4096, 2056, 6, torch.float16),    # 9 rows per workgroup: a full tile and one row of the next
    (2048, 6152, 4, torch.bfloat16),   # 25 rows per workgroup: ranges that start and end inside a mask byte
]


@pytest.mark.parametrize("H,I,B,dtype", MATRIX_CORE)
def test_matrix_core_batches(oracle, H, I, B, dtype):
    m = make_mlp(H, I, B, dtype, seed=H + I + B, corr=0.5)
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    for q in (0.0, 0.5, 0.97):
        t = -1.0 if q == 0.0 else float(torch.quantile(a_abs, q))
        check_mlp_case(oracle, m, t, tag=f"matrix-core-q{q}")
    check_mlp_case(oracle, m, 1e9, tag="matrix-core-all-dead")


def test_matrix_core_and_wave_per_row_kernels_agree(oracle):
    """Same inputs through both gate+up kernels (the tuning knob pins the wave-per-row one): flags may differ only
    where an activation sits within rounding distance of t, outputs agree to the parity tolerance."""
    m = make_mlp(4096, 2048, 8, torch.float16, seed=77, corr=0.5)
    t = calibrate(m["wg"], [0.5])[0]
    d = dev(m)
    ws = _ws(8, 4096, 2048)
    try:
        capi.set_tuning(-1, 0, 0, 0)
        y_w, f_w, _ = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        a_w, _ = capi.gate_flag(d["x"], d["wg"], t)
        capi.set_tuning(0, 0, 0, 0)
        y_m, f_m, _ = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        a_m, _ = capi.gate_flag(d["x"], d["wg"], t)
    finally:
        capi.set_tuning(0, 0, 0, 0)
    torch.cuda.synchronize()
    torch.testing.assert_close(a_m.float().cpu(), a_w.float().cpu(), **A_TOL[torch.float16])
    flips = (f_w != f_m).cpu()
    if int(flips.sum()):
        dist = (a_w.float().cpu().abs() - t).abs()[flips]
        assert float(dist.max()) <= A_TOL[torch.float16]["atol"] + A_TOL[torch.float16]["rtol"] * abs(t)
    if int(flips.sum()) == 0:
        close(y_m.cpu(), y_w.cpu(), torch.float16)


MATRIX_CORE_DOWN = [
    # H, I, B, dtype -- 3..16 rows of a 16-bit type through the stand-alone sparse down entry point
    (4096, 11008, 8, torch.float16),   # the benchmark shape: 32 neuron groups of 344
    (4096, 1003, 3, torch.float16),    # groups of 32 neurons: two steps of sixteen list entries at most
    (520, 1000, 5, torch.bfloat16),    # rows of 65 vectors: the second slab holds one
    (2048, 2049, 7, torch.bfloat16),
    (64, 96, 4, torch.float16),        # one slab of 8 vectors, lists shorter than one step
    (4096, 40, 6, torch.float16),
    (8192, 3584, 5, torch.float16),    # 16 slabs x 16 groups of 224 neurons
    (4096, 2048, 16, torch.bfloat16),  # 9..16 rows: one pass over W_down^T for all of them
    (520, 1000, 11, torch.float16),
]


@pytest.mark.parametrize("H,I,B,dtype", MATRIX_CORE_DOWN)
def test_matrix_core_down_kernel(H, I, B, dtype):
    """The sparse down projection of 3..16 rows on the matrix cores against the spelled-out sum in fp64 and against the
    wave-per-row-pair kernel (an explicit workgroup size pins that one), for mask densities from empty to full, into a
    dtype output and into the caller's fp32 accumulator.  Weight rows that no batch row uses hold infinities: a row
    that is skipped, or that only pads the last step of a list, must not reach the output."""
    g = torch.Generator().manual_seed(H + I + B)
    wdt = (torch.randn(I, H, generator=g) * 0.05).to(dtype)
    z_all = torch.randn(B, I, generator=g).to(dtype)
    ws = _ws(B, H, I)
    for density in (0.0, 0.03, 0.5, 1.0):
        flag = torch.rand(B, I, generator=g) < density
        if density == 0.03:
            flag[:, 0] = False  # row 0 is what the padding of a list reads
        z = torch.where(flag, z_all, torch.zeros_like(z_all))
        w = wdt.clone()
        dead = ~flag.any(dim=0)
        w[dead] = float("inf")
        want = (z.double() @ torch.where(dead[:, None], torch.zeros_like(wdt), wdt).double()).to(dtype)
        dz, dw, df = z.cuda(), w.cuda(), flag.to(torch.uint8).cuda()
        print(f"[case] matrix-core-down H={H} I={I} B={B} {dtype} density={density}", flush=True)
        y = capi.down_flag(dz, dw, df, ws)
        acc = torch.full((B, H), 2.0, dtype=torch.float32, device="cuda")
        capi.down_flag(dz, dw, df, ws, accumulate_into=acc)
        try:
            capi.set_tuning(0, 0, 1024, 0)  # above eight rows: two passes of that kernel
            y_pair = capi.down_flag(dz, dw, df, ws)
        finally:
            capi.set_tuning(0, 0, 0, 0)
        y_again = capi.down_flag(dz, dw, df, ws)
        torch.cuda.synchronize()
        assert torch.isfinite(y.float()).all()
        close(y.cpu(), want, dtype)
        close(y_pair.cpu(), want, dtype)
        close((acc.cpu() - 2.0).to(dtype), want, dtype)
        assert torch.equal(y, y_again), "the matrix-core down kernel is not reproducible call to call"


@pytest.mark.parametrize("H,I,B,dtype", [(2048, 520, 4, torch.float16), (4096, 11008, 8, torch.bfloat16), (4096, 1000, 16, torch.float16),
                                         (2048, 2056, 11, torch.bfloat16)])
def test_rowmajor_down_on_the_matrix_cores(oracle, H, I, B, dtype):
    """cats_mlp_rowmajor_down (flag_gemv_gemv_inner: W_down in nn.Linear's (H, I) layout, read whole) at 3..16 rows runs its
    down projection as a matrix-core GEMV over rows of any length, cut into chunks.  Against the oracle on the kernel's
    own activations and flags; then with infinities in the first bytes of W_down, which the padding loads of that kernel
    re-read: only output column 0, whose weights they are, may see them."""
    m = make_mlp(H, I, B, dtype, seed=H + I + B, corr=0.4)
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    t = float(torch.quantile(a_abs, 0.5))
    d = dev(m)
    ws = _ws(B, H, I)
    y = capi.mlp_rowmajor_down(d["x"], d["wg"], d["wu"], d["wd"], t, ws)
    a, flag = capi.gate_flag(d["x"], d["wg"], t)
    torch.cuda.synchronize()
    ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a.cpu(), flag_in=flag.cpu())
    close(y.cpu(), ref["y"], dtype)
    wd_inf = d["wd"].clone()
    wd_inf[0, :64] = float("inf")
    y_inf = capi.mlp_rowmajor_down(d["x"], d["wg"], d["wu"], wd_inf, t, ws)
    torch.cuda.synchronize()
    assert torch.equal(y_inf[:, 1:], y[:, 1:])
    try:  # and the wave-per-row kernels on the same call
        capi.set_tuning(-1, 0, 0, 0)
        y_w = capi.mlp_rowmajor_down(d["x"], d["wg"], d["wu"], d["wd"], t, ws)
    finally:
        capi.set_tuning(0, 0, 0, 0)
    torch.cuda.synchronize()
    close(y_w.cpu(), ref["y"], dtype)


SINGLE_PASS = [
    # H, I, B, dtype -- every template the single-pass kernel is instantiated for (row length in whole blocks of 512
    # vectors or not, 1 / 2 / 4 vectors of a row per down wave), ranges that end short, fewer neurons than row waves
    (4096, 11008, 1, torch.float16), (4096, 14336, 1, torch.bfloat16), (4096, 2048, 2, torch.float16),
    (520, 1000, 2, torch.float16), (260, 333, 1, torch.float32), (8192, 1024, 1, torch.float16), (8192, 600, 2, torch.bfloat16),
    (4096, 700, 1, torch.float32), (8192, 300, 1, torch.float32), (64, 96, 1, torch.float16), (72, 5, 2, torch.bfloat16), (2048, 4099, 2, torch.float32),
]


@pytest.mark.parametrize("H,I,B,dtype", SINGLE_PASS)
def test_single_pass_and_two_kernel_paths_agree(oracle, H, I, B, dtype):
    """cats_mlp for 1..2 rows runs as one streaming kernel + a reduction; the tuning knob puts the same call on the
    separate gate+up and sparse-down kernels.  Same activations bit for bit (same dot-product order), so the same
    flags and count; outputs agree to the parity tolerance; the single-pass result is bitwise repeatable."""
    m = make_mlp(H, I, B, dtype, seed=H + 3 * I + B, corr=0.5 if B > 1 else 0.0)
    d = dev(m)
    ws = _ws(B, H, I)
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    nw = (torch.rand(H) + 0.5).to(dtype).cuda()
    for q in (0.0, 0.5, 0.93):
        t = -1.0 if q == 0.0 else float(torch.quantile(a_abs, q))
        print(f"[case] single-pass H={H} I={I} B={B} {dtype} q={q}", flush=True)
        try:
            capi.set_tuning(0, 0, 0, 1)
            y2, f2, c2 = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
            n2 = capi.mlp_norm_residual(d["x"], nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws)
            a, _ = capi.gate_flag(d["x"], d["wg"], t)
            u2 = capi.up_down(d["x"], a, d["wu"], d["wdt"], t, ws)
            torch.cuda.synchronize()
        finally:
            capi.set_tuning(0, 0, 0, 0)
        y1, f1, c1 = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        y1b = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws)
        n1 = capi.mlp_norm_residual(d["x"], nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws)
        u1 = capi.up_down(d["x"], a, d["wu"], d["wdt"], t, ws)
        torch.cuda.synchronize()
        assert torch.equal(f1, f2) and int(c1) == int(c2) == int(f1.any(dim=0).sum())
        assert torch.equal(y1, y1b), "single-pass output differs between two calls"
        close(y1.cpu(), y2.cpu(), dtype)
        close(u1.cpu(), u2.cpu(), dtype)
        close(u1.cpu(), y2.cpu(), dtype)
        # the folded norm changes x in its last bits between kernels' staging paths: same tolerance, on the residual sum
        close(n1.cpu(), n2.cpu(), dtype)
        ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a.cpu(), flag_in=f1.cpu())
        close(y1.cpu(), ref["y"], dtype)


def test_mlp_stage_launches_compose_to_the_whole_call():
    """cats_mlp_stage(1) then cats_mlp_stage(2) is cats_mlp, on the single-pass path (1 row) and on the two-kernel path (4 rows)."""
    import ctypes

    L = capi.lib()
    for B in (1, 4):
        m = make_mlp(4096, 1536, B, torch.float16, seed=5 + B)
        d = dev(m)
        t = calibrate(m["wg"], [0.5])[0]
        ws = _ws(B, 4096, 1536)
        want = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws)
        got = torch.zeros_like(want)
        p = lambda x: ctypes.c_void_p(x.data_ptr())
        s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for stage in (1, 2):
            capi.check(L.cats_mlp_stage(stage, p(d["x"]), p(d["wg"]), p(d["wu"]), p(d["wdt"]), p(got), B, 4096, 1536, capi.F16,
                                        ctypes.c_float(t), p(ws.buf), ws.nbytes, s), "cats_mlp_stage")
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    assert L.cats_mlp_stage(3, None, None, None, None, None, 1, 64, 64, 0, ctypes.c_float(0), None, 0, None) != 0


@pytest.mark.parametrize("B", [1, 2, 4])
def test_active_count_does_not_disturb_the_down_kernel_output(B):
    """The sparse down kernel totals the mask in the LDS it has just folded its partial sums through: asking for the
    count must not change a single output bit."""
    m = make_mlp(4096, 4096, B, torch.float16, seed=91 + B, corr=0.5)
    d = dev(m)
    t = calibrate(m["wg"], [0.5])[0]
    ws = _ws(B, 4096, 4096)
    try:
        capi.set_tuning(0, 0, 0, 1)  # two-kernel path at every batch size
        y_plain = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws)
        for _ in range(5):
            y_cnt, flag, cnt = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
            torch.cuda.synchronize()
            assert torch.equal(y_cnt, y_plain)
            assert int(cnt) == int(flag.any(dim=0).sum())
    finally:
        capi.set_tuning(0, 0, 0, 0)


def _gap_threshold(a_abs, q):
    """A threshold near the q-quantile of |a| that sits in the middle of the widest gap between neighbouring values
    there, so that a last-bit difference in the normalised input cannot move a neuron across it."""
    v = torch.sort(a_abs.flatten().float()).values
    k = int(q * (v.numel() - 1))
    lo, hi = max(k - 40, 0), min(k + 40, v.numel() - 1)
    gaps = v[lo + 1:hi + 1] - v[lo:hi]
    i = int(torch.argmax(gaps)) + lo
    return float((v[i] + v[i + 1]) / 2)


LAYER_TAIL = [
    # H, I, B, dtype
    (64, 96, 1, torch.float16), (72, 100, 2, torch.bfloat16), (260, 333, 3, torch.float32),
    (4096, 1000, 1, torch.float16), (4096, 1003, 5, torch.float16), (2048, 520, 8, torch.bfloat16),
    (4096, 11008, 1, torch.float16),
]


@pytest.mark.parametrize("H,I,B,dtype", LAYER_TAIL)
def test_norm_and_residual_folded_into_the_mlp(oracle, H, I, B, dtype):
    """cats_mlp_norm_residual against  h + MLP(norm(h))  spelled out with the oracle's restatements."""
    m = make_mlp(H, I, B, dtype, seed=H + 3 * I + B)
    g = torch.Generator().manual_seed(H + I)
    h = (m["x"].float() * 2.5 + 0.3).to(dtype)                      # not unit-variance, not zero-mean
    nw = (1.0 + 0.2 * torch.randn(H, generator=g)).to(dtype)
    eps = 1e-5
    x_ref = oracle.torch_rms_norm(h, nw, eps)
    a_abs = oracle.c_gate(x_ref, m["wg"], -1.0)[0].float().abs()
    d = dev(dict(h=h, nw=nw, wg=m["wg"], wu=m["wu"], wdt=m["wdt"]))
    ws = _ws(B, H, I)
    for q in (0.0, 0.5, 0.9):
        t = -1.0 if q == 0.0 else _gap_threshold(a_abs, q)
        print(f"[case] layer-tail dtype={dtype} B={B} H={H} I={I} q={q} t={t}", flush=True)
        ref = oracle.c_mlp(x_ref, m["wg"], m["wu"], m["wd"], t)
        want = h + ref["y"].to(dtype)
        got = capi.mlp_norm_residual(d["h"], d["nw"], eps, d["wg"], d["wu"], d["wdt"], t, ws)
        # the same thing in two steps on the GPU: torch's norm, the unfused entry point, torch's add
        two_step = d["h"] + capi.mlp(oracle.torch_rms_norm(d["h"], d["nw"], eps), d["wg"], d["wu"], d["wdt"], t, ws)
        torch.cuda.synchronize()
        close(got.cpu(), want, dtype)
        close(got.cpu(), two_step.cpu(), dtype)
    # in place: out aliases h
    h2 = d["h"].clone()
    capi.mlp_norm_residual(h2, d["nw"], eps, d["wg"], d["wu"], d["wdt"], t, ws, out=h2)
    torch.cuda.synchronize()
    assert torch.equal(h2, got)


@pytest.mark.parametrize("H,I,B,dtype", [(4096, 11008, 1, torch.float16), (4096, 1000, 2, torch.bfloat16), (512, 768, 4, torch.float16),
                                         (1024, 640, 8, torch.bfloat16), (256, 333, 3, torch.float32), (2048, 512, 12, torch.float16),
                                         (256, 200, 10, torch.float32), (1056, 300, 9, torch.bfloat16)])   # the last two: two passes of <= 8 rows
def test_next_norm_written_by_the_finishing_launch(oracle, H, I, B, dtype):
    """cats_mlp_norm_residual_norm: `out` carries the bits of cats_mlp_norm_residual (same launches), and `next` is the
    RMS norm of exactly those stored values -- checked against the restated HF norm evaluated on the kernel's own `out`
    (one fp32 sum of squares per row: the only difference is the order the squares are added in).  Twice on one
    workspace (the arrival counter must be back at zero), then under a graph."""
    m = make_mlp(H, I, B, dtype, seed=5 * H + I + B)
    g = torch.Generator().manual_seed(H + I + 1)
    h = (m["x"].float() * 1.7 - 0.2).to(dtype)
    nw = (1.0 + 0.2 * torch.randn(H, generator=g)).to(dtype)
    nw2 = (0.8 + 0.3 * torch.randn(H, generator=g)).to(dtype)
    eps, eps2 = 1e-5, 1e-6
    x_ref = oracle.torch_rms_norm(h, nw, eps)
    t = float(torch.quantile(oracle.c_gate(x_ref, m["wg"], -1.0)[0].float().abs().flatten(), 0.5))
    d = dev(dict(h=h, nw=nw, nw2=nw2, wg=m["wg"], wu=m["wu"], wdt=m["wdt"]))
    ws = _ws(B, H, I)
    want_out = capi.mlp_norm_residual(d["h"], d["nw"], eps, d["wg"], d["wu"], d["wdt"], t, ws)
    tol = {torch.float16: dict(rtol=2e-3, atol=2e-3), torch.bfloat16: dict(rtol=1.6e-2, atol=1.6e-2), torch.float32: dict(rtol=1e-5, atol=1e-5)}[dtype]
    for rep in range(2):
        print(f"[case] next-norm dtype={dtype} B={B} H={H} I={I} rep={rep}", flush=True)
        out, nxt = capi.mlp_norm_residual_norm(d["h"], d["nw"], eps, d["wg"], d["wu"], d["wdt"], t, d["nw2"], eps2, ws)
        torch.cuda.synchronize()
        assert torch.equal(out, want_out)
        want_next = oracle.torch_rms_norm(out.cpu(), nw2, eps2)
        torch.testing.assert_close(nxt.cpu().float(), want_next.float(), **tol)
    # the whole chain against the oracle's restatement of the layer tail
    ref = oracle.c_mlp(x_ref, m["wg"], m["wu"], m["wd"], t)
    close(out.cpu(), h + ref["y"].to(dtype), dtype)
    if B <= 8:
        gr = torch.cuda.CUDAGraph()
        hs = d["h"].clone()
        with torch.cuda.graph(gr):
            o_g, n_g = capi.mlp_norm_residual_norm(hs, d["nw"], eps, d["wg"], d["wu"], d["wdt"], t, d["nw2"], eps2, ws)
        for rep in range(3):
            capi.mlp(d["h"], d["wg"], d["wu"], d["wdt"], t, ws)   # eager work on the same workspace between replays
            torch.cuda.synchronize()
            gr.replay()
            torch.cuda.synchronize()
            assert torch.equal(o_g, out) and torch.equal(n_g, nxt), f"replay {rep}"


def test_next_norm_needs_rows_of_whole_reduction_blocks():
    z = lambda *s: torch.zeros(*s, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="shape"):
        capi.mlp_norm_residual_norm(z(1, 72), z(72), 1e-5, z(64, 72), z(64, 72), z(64, 72), 0.1, z(72), 1e-5, _ws(1, 72, 64))


def test_norm_residual_rejects_rows_that_do_not_fit_in_lds():
    H, I, B = 16384, 64, 8   # 8 x 32 KiB of fp16 activations
    z = lambda *s: torch.zeros(*s, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="shape"):
        capi.mlp_norm_residual(z(B, H), z(H), 1e-5, z(I, H), z(I, H), z(I, H), 0.1, _ws(B, H, I))


@pytest.mark.parametrize("B", [1, 4])
def test_llama70b_shape(oracle, B):
    """8192 -> 28672, the larger shape the reference smoke-tests (flash_gemv/test/test_fuse_gemv_cmp.py:662-676).
    Rows of 16 KiB: two passes of 8 chunks per row in the wave-per-row kernel, 16 column slabs in the down kernel;
    batch 4 stays on the wave-per-row kernel (the matrix-core one takes rows of 2048 or 4096 elements)."""
    m = make_mlp(8192, 28672, B, torch.float16, seed=70, corr=0.5 if B > 1 else 0.0)
    t = calibrate(m["wg"], [0.5], n_vec=64)[0]
    check_mlp_case(oracle, m, t, tag=f"llama70b-fp16-B{B}")


@pytest.mark.parametrize("H,I,B,dtype", [(4096, 1000, 16, torch.float16), (512, 333, 11, torch.bfloat16), (260, 96, 9, torch.float32),
                                         (2048, 1536, 9, torch.bfloat16), (4096, 11008, 12, torch.float16), (4096, 2048, 16, torch.bfloat16)])
def test_batches_of_nine_to_sixteen_rows(oracle, H, I, B, dtype):
    """The reference's kernels are instantiated up to 16 rows (fuse_gemv_cmp_cuda.cu:2368-2400).  Here 16-bit rows of 2048
    or 4096 elements take one matrix-core gate + up pass and one matrix-core down pass over all rows (every matrix read
    once, over the union mask of all rows); every other case is two passes of at most 8 rows.  Either way: the full
    parity case, and rows 8.. of the big batch against the same rows run as a batch of their own (same flags, bit for
    bit; outputs to the parity tolerance -- the union of sixteen rows orders the down sums differently)."""
    m = make_mlp(H, I, B, dtype, seed=B + H, corr=0.3)
    a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
    t = float(torch.quantile(a_abs, 0.5))
    check_mlp_case(oracle, m, t, tag=f"rows-9-to-16-B{B}")
    d = dev(m)
    ws = _ws(B, H, I)
    y_all, f_all, _ = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
    y_hi, f_hi, _ = capi.mlp(d["x"][8:].contiguous(), d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
    torch.cuda.synchronize()
    if B - 8 >= 3 or dtype == torch.float32 or H not in (2048, 4096):   # same gate kernel in both calls: same activations
        assert torch.equal(f_all[8:], f_hi)
    close(y_all[8:].cpu(), y_hi.cpu(), dtype)
    # the layer tail through the same path, in place and with the next norm
    g = torch.Generator().manual_seed(B)
    nw = (1.0 + 0.2 * torch.randn(H, generator=g)).to(dtype).cuda()
    h = (d["x"].float() * 1.5).to(dtype)
    want = capi.mlp_norm_residual(h[:8].contiguous(), nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws)
    want_hi = capi.mlp_norm_residual(h[8:].contiguous(), nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws)
    got = capi.mlp_norm_residual(h, nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws)
    torch.cuda.synchronize()
    close(got[:8].cpu(), want.cpu(), dtype)
    close(got[8:].cpu(), want_hi.cpu(), dtype)
    if H % 32 == 0:
        out, nxt = capi.mlp_norm_residual_norm(h, nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, nw, 1e-6, ws)
        torch.cuda.synchronize()
        assert torch.equal(out, got)
        ntol = {torch.float16: dict(rtol=2e-3, atol=2e-3), torch.bfloat16: dict(rtol=1.6e-2, atol=1.6e-2), torch.float32: dict(rtol=1e-5, atol=1e-5)}[dtype]
        torch.testing.assert_close(nxt.cpu().float(), oracle.torch_rms_norm(out.cpu(), nw.cpu(), 1e-6).float(), **ntol)
    h2 = h.clone()
    capi.mlp_norm_residual(h2, nw, 1e-5, d["wg"], d["wu"], d["wdt"], t, ws, out=h2)
    torch.cuda.synchronize()
    assert torch.equal(h2, got)


def test_batch_above_sixteen_is_an_error_not_a_crash():
    z = lambda *s: torch.zeros(*s, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="batch"):
        capi.mlp(z(17, 512), z(64, 512), z(64, 512), z(64, 512), 0.1, _ws(8, 512, 64))


def test_active_count_above_eight_rows_is_the_union_over_both_passes(oracle):
    """9..16 rows run as two passes of 8; the count must still be the number of neurons active in any row, whether or
    not the caller asks for the flags (without them the passes write the flags into the workspace)."""
    for B, H, I in ((9, 512, 200), (16, 1024, 333), (12, 4096, 11008)):
        m = make_mlp(H, I, B, torch.float16, seed=B)
        d = dev(m)
        t = float(torch.quantile(torch.nn.functional.silu(m["x"].float() @ m["wg"].float().t()).abs().flatten()[::7], 0.95))
        ws = _ws(B, H, I)
        y, flag, count = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws, want_flag=True, want_count=True)
        cnt_only = torch.full((1,), -1, dtype=torch.int32, device="cuda")
        y2 = torch.empty_like(y)
        L = capi.lib()
        st = L.cats_mlp(capi._p(d["x"]), capi._p(d["wg"]), capi._p(d["wu"]), capi._p(d["wdt"]), capi._p(y2), None, None, capi._p(cnt_only),
                        B, H, I, capi.F16, t, capi._p(ws.buf), ws.nbytes, capi._stream(d["x"]))
        assert st == 0
        torch.cuda.synchronize()
        want = int(flag.cpu().bool().any(dim=0).sum())
        assert 0 < want < I
        assert int(count.item()) == want
        assert int(cnt_only.item()) == want
        assert torch.equal(y, y2)


def test_reference_recipe_shapes(oracle):
    """The reference's own test recipe: U(-0.5, 0.5) data, (4096 -> 14336), t = 0.2 / 0.3, B = 1 and 2
    (flash_gemv/test/test_fuse_gemv_cmp.py:173-187, 442-524).  Only the gate / mask part is checked at t = 0.2;
    the full pipeline at t = 0.3 in all three dtypes."""
    m = make_mlp(4096, 14336, 1, torch.float16, seed=0, dist="uniform")
    d = dev(m)
    a, flag = capi.gate_flag(d["x"], d["wg"], 0.2)
    assert torch.equal(flag, torch.abs(a) > 0.2)
    for dtype in (torch.float16, torch.float32, torch.bfloat16):
        m = make_mlp(4096, 14336, 2, dtype, seed=0, dist="uniform")
        check_mlp_case(oracle, m, 0.3, tag=f"ref-recipe-{dtype}")


def test_error_codes_on_device():
    x = torch.zeros(1, 64, dtype=torch.float16, device="cuda")
    w = torch.zeros(96, 64, dtype=torch.float16, device="cuda")
    ws = _ws(1, 64, 96)
    L = capi.lib()
    p = capi._p
    s = capi._stream(x)
    small = torch.empty(256, dtype=torch.uint8, device="cuda")
    y = torch.empty(1, 64, dtype=torch.float16, device="cuda")
    assert L.cats_mlp(p(x), p(w), p(w), p(w), p(y), None, None, None, 1, 64, 96, 0, 0.1, p(small), 256, s) == 6  # workspace
    assert L.cats_mlp(p(x), p(w), p(w), p(w), p(y), None, None, None, 17, 64, 96, 0, 0.1, p(ws.buf), ws.nbytes, s) == 4  # batch
    assert L.cats_mlp(p(x), p(w), p(w), p(w), p(y), None, None, None, 1, 60, 96, 0, 0.1, p(ws.buf), ws.nbytes, s) == 3  # align
    assert L.cats_mlp(p(x), p(w), p(w), p(w), p(y), None, None, None, 1, 64, 96, 7, 0.1, p(ws.buf), ws.nbytes, s) == 1  # dtype
    assert L.cats_mlp(p(x), None, p(w), p(w), p(y), None, None, None, 1, 64, 96, 0, 0.1, p(ws.buf), ws.nbytes, s) == 5  # null
    torch.cuda.synchronize()
