"""cats_mlp_noalloc: the whole MLP with the library's built-in device scratch instead of a caller workspace.
Called through the C ABI and compared with cats_mlp (same kernels, same summation order: same bits), twice in a
row, the second time on a smaller problem -- the scratch keeps the first call's contents."""
import pytest
import torch

from tests.util import calibrate, dev, make_mlp

pytestmark = pytest.mark.gpu


def test_mlp_noalloc_matches_cats_mlp_on_two_calls_in_a_row():
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
    # beyond the built-in scratch: a clear error, no launch
    x = torch.zeros(4, 4096, dtype=torch.float16, device="cuda")
    w = torch.zeros(64, 4096, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="scratch"):
        capi.mlp_noalloc(x, w, w, w, 0.0, torch.empty_like(x))
    x = torch.zeros(2, 8192, dtype=torch.float16, device="cuda")   # B * H = 16384 > 8192
    w = torch.zeros(64, 8192, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.CatsError, match="scratch"):
        capi.mlp_noalloc(x, w, w, w, 0.0, torch.empty_like(x))
