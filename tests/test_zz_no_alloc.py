"""cats_mlp_noalloc: the whole MLP with the library's built-in device scratch instead of a caller workspace.
Called through the C ABI and compared with cats_mlp (same kernels, same summation order: same bits) and with the CPU
oracle (parity tolerance), twice in a row, the second time on a smaller problem -- the scratch keeps the first call's
contents.  A second test captures the call into a HIP graph after one eager call and replays it."""
import pytest
import torch

from tests.util import TOL, calibrate, dev, make_mlp

pytestmark = pytest.mark.gpu


def test_mlp_noalloc_matches_cats_mlp_on_two_calls_in_a_row(oracle):
    assert torch.cuda.is_available(), "this test needs the GPU"
    from cats_amd import capi

    capi.lib()
    cases = [(4096, 11008, 2, torch.float16, 31), (2048, 1000, 1, torch.bfloat16, 32)]  # the second is smaller in every dimension
    for H, I, B, dtype, seed in cases:
        print(f"[case] noalloc H={H} I={I} B={B} {dtype}", flush=True)
        m = make_mlp(H, I, B, dtype, seed=seed, corr=0.5 if B > 1 else 0.0)
        d = dev(m)
        t = calibrate(m["wg"], [0.5])[0]
        ws = capi.Workspace(B, H, I)
        want = capi.mlp(d["x"], d["wg"], d["wu"], d["wdt"], t, ws)
        got = torch.full_like(want, float("nan"))
        before = torch.cuda.memory_allocated()
        capi.mlp_noalloc(d["x"], d["wg"], d["wu"], d["wdt"], t, got)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(got, want), f"max |diff| {float((got.float() - want.float()).abs().max())}"
        # and against the CPU oracle on the kernel's own gate values (torch's allocator counters above cannot see a
        # hipMalloc; that the entry point makes none is a property of its source: it calls no allocating routine)
        a, flag = capi.gate_flag(d["x"], d["wg"], t)
        ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t, a_in=a.cpu(), flag_in=flag.cpu())
        torch.testing.assert_close(got.cpu().float(), ref["y"].float(), **TOL[dtype])
    # beyond the built-in scratch: a clear error, no launch
    x = torch.zeros(4, 4096, dtype=torch.float16, device="cuda")
    w = torch.zeros(64, 4096, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="scratch"):
        capi.mlp_noalloc(x, w, w, w, 0.0, torch.empty_like(x))
    x = torch.zeros(2, 8192, dtype=torch.float16, device="cuda")   # B * H = 16384 > 8192
    w = torch.zeros(64, 8192, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="scratch"):
        capi.mlp_noalloc(x, w, w, w, 0.0, torch.empty_like(x))


def test_mlp_noalloc_in_a_hip_graph():
    """The callers this entry point is for include code under graph capture: one eager call first (it resolves the
    scratch address and the kernel's LDS attribute), then capture, then replays with eager work in between, each
    compared bit for bit with cats_mlp on the same input."""
    from cats_amd import capi

    capi.lib()
    H, I, B, dtype = 4096, 11008, 1, torch.float16
    m = make_mlp(H, I, B, dtype, seed=41)
    d = dev(m)
    t = calibrate(m["wg"], [0.5])[0]
    ws = capi.Workspace(B, H, I)
    x = d["x"].clone()
    y = torch.empty_like(x)
    capi.mlp_noalloc(x, d["wg"], d["wu"], d["wdt"], t, y)   # eager warm-up
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        capi.mlp_noalloc(x, d["wg"], d["wu"], d["wdt"], t, y)
    for rep in range(3):
        x.copy_(torch.randn(B, H, device="cuda", generator=torch.Generator(device="cuda").manual_seed(rep)).to(dtype))
        want = capi.mlp(x, d["wg"], d["wu"], d["wdt"], t, ws)   # eager work between the replays
        torch.cuda.synchronize()
        y.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {rep}: max |diff| {float((y.float() - want.float()).abs().max())}"
