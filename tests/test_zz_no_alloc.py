"""The allocation-free dispatch plan (ats_dispatch_plan_static) against ats_dispatch_plan, through the C ABI:
same integer outputs bit for bit on two calls in a row, the second with a smaller input (the fixed scratch
array keeps the first call's contents), then a plan small enough for the single-block kernel, then the first
size again.  Also: the size limit is refused with a clear error and without touching the device."""
import pytest
import torch

from oracle import c_oracle


def _plan(lib, fn_static, idx, E, C, dev):
    from adaptivetrainingsystem_amd._lib import check
    T, k = idx.shape
    n = T * k
    i32 = dict(dtype=torch.int32, device=dev)
    outs = {"slot": torch.full((n,), -7, **i32), "token_map": torch.full((E * C,), -7, **i32),
            "hist": torch.full((E,), -7, **i32), "kept": torch.full((E,), -7, **i32),
            "offsets": torch.full((E + 1,), -7, **i32), "row_src": torch.full((max(1, min(n, E * C)),), -7, **i32),
            "row_of": torch.full((n,), -7, **i32), "status": torch.full((1,), -7, **i32)}
    ptrs = [outs[name].data_ptr() for name in ("slot", "token_map", "hist", "kept", "offsets", "row_src", "row_of",
                                               "status")]
    stream = torch.cuda.current_stream().cuda_stream
    if fn_static:
        check(lib.ats_dispatch_plan_static(idx.data_ptr(), 0, T, k, E, C, *ptrs, stream), "ats_dispatch_plan_static")
    else:
        nbytes = lib.ats_dispatch_plan_workspace(T, k, E)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        check(lib.ats_dispatch_plan(idx.data_ptr(), 0, T, k, E, C, *ptrs, ws.data_ptr(), nbytes, stream),
              "ats_dispatch_plan")
    torch.cuda.synchronize()
    return outs


@pytest.mark.gpu
def test_static_plan_equals_workspace_plan_on_consecutive_calls(gpu):
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    # plans above 32768 assignments run the three-kernel form, whose chunk histograms live in the fixed array
    # (smaller ones are done in one launch that needs no scratch at all): large, smaller, tiny, large again
    cases = [(40000, 2, 8, 9000, 11), (17000, 2, 8, 4000, 12), (100, 3, 16, 20, 13), (40000, 2, 8, 9000, 11),
             (8192, 6, 64, 1000, 14), (5000, 2, 8, 1000, 15)]
    for T, k, E, C, seed in cases:
        print("case static plan", T, k, E, C, flush=True)
        g = torch.Generator().manual_seed(seed)
        idx = torch.topk(torch.randn(T, E, generator=g), k, -1)[1].int()
        idx_dev = idx.to(gpu)
        got = _plan(lib, True, idx_dev, E, C, gpu)
        want = _plan(lib, False, idx_dev, E, C, gpu)
        for name in want:
            assert torch.equal(got[name], want[name]), (name, T, k, E, C)
        tm, slot, hist, kept, dropped = c_oracle.fcfs_dispatch(idx.long().numpy(), E, C)
        assert (got["token_map"].cpu().view(E, C).numpy() == tm).all() and (got["slot"].cpu().numpy() == slot).all()
        assert got["status"].item() == 0


def test_static_plan_refuses_oversized_plans_on_the_host():
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    # 2^30 assignments over 1024 experts would need 16 GiB of chunk histograms
    rc = lib.ats_dispatch_plan_static(None, 0, 1 << 29, 2, 1024, 4, *([None] * 8), None)
    assert rc == -4
    msg = lib.ats_last_error_string().decode()
    assert "ats_dispatch_plan_static" in msg and "scratch" in msg and "ats_dispatch_plan" in msg
    assert lib.ats_dispatch_plan_static(None, 0, 4, 0, 8, 4, *([None] * 8), None) == -1
