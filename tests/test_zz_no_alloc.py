"""clt_threshold_count_static (the entry point that allocates nothing) against clt_threshold_count,
through the C ABI: two calls in a row on one GPU, the second on a smaller input, so that whatever
the first call left in the library's device array must not leak into the second result."""
import pytest
import torch

from crosslayer_coding_amd import _native as nat

pytestmark = pytest.mark.gpu


def _count(lib, fn_static, pre, theta, pred):
    L, T, F = pre.shape
    dev = pre.device
    dt = nat.dtype_code(pre.dtype)
    stream = nat.current_stream(dev)
    row_ptr = torch.full((L * T + 1,), -7, dtype=torch.int32, device=dev)
    if fn_static:
        code = lib.clt_threshold_count_static(nat.ptr(pre), T, F, L, pre.stride(0), nat.ptr(theta), pred, dt,
                                              nat.ptr(row_ptr), stream)
    else:
        ws = torch.empty(max(L * T * 4, 256), dtype=torch.uint8, device=dev)
        code = lib.clt_threshold_count(nat.ptr(pre), T, F, L, pre.stride(0), nat.ptr(theta), pred, dt,
                                       nat.ptr(row_ptr), nat.ptr(ws), ws.numel(), stream)
    nat.check(code, "threshold_count")
    torch.cuda.synchronize()
    return row_ptr


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_count_matches_the_workspace_variant_on_two_calls_in_a_row(dev, dtype):
    lib = nat.load()
    g = torch.Generator().manual_seed(11)
    # first call: many rows with many survivors; second call: fewer, shorter rows with few survivors
    for (L, T, F, pred, shift) in ((3, 640, 1024, nat.PRED_GE_THETA, 0.0), (2, 96, 264, nat.PRED_GE_THETA, 1.5),
                                   (1, 33, 100, nat.PRED_GT_ZERO, 0.0)):
        pre = torch.randn(L, T, F, generator=g).to(dtype).to(dev)
        theta = (torch.rand(L, F, generator=g) + shift).to(dtype).to(dev)
        want = _count(lib, False, pre, theta, pred)
        got = _count(lib, True, pre, theta, pred)
        assert torch.equal(got, want)
        # and against the definition
        keep = (pre >= theta[:, None, :]) if pred == nat.PRED_GE_THETA else (pre > 0)
        counts = keep.sum(dim=2).reshape(-1).to(torch.int64)
        assert torch.equal(got[1:].long(), torch.cumsum(counts, 0)) and int(got[0]) == 0


def test_static_count_rejects_sizes_beyond_its_array(dev):
    lib = nat.load()
    pre = torch.zeros(1, 8, 8, device=dev)
    row_ptr = torch.zeros(2 ** 20 + 2, dtype=torch.int32, device=dev)
    code = lib.clt_threshold_count_static(nat.ptr(pre), 2 ** 20 + 1, 8, 1, 8, None, nat.PRED_GT_ZERO, 0, nat.ptr(row_ptr),
                                          nat.current_stream(dev))
    assert code == -6
    # an empty input needs neither the array nor a kernel over rows
    code = lib.clt_threshold_count_static(None, 0, 8, 1, 0, None, nat.PRED_GT_ZERO, 0, nat.ptr(row_ptr), nat.current_stream(dev))
    assert code == 0
    torch.cuda.synchronize()
    assert int(row_ptr[0]) == 0
