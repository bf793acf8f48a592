"""GPU: the entry point that allocates nothing (llmc_sumsq_accumulate_noalloc) against the existing
llmc_sumsq_accumulate, through the C ABI, bit for bit, on two calls in a row (the second smaller, so that
it runs over what the first left in the library's device array)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(x, K):
    from llmcompressor_amd import _lib

    lib = _lib.lib()
    dev = x.device
    dt = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[x.dtype]
    base = torch.rand(K, device=dev, dtype=torch.float32)
    want, got = base.clone(), base.clone()
    nws = int(lib.llmc_sumsq_workspace_bytes(K))
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    rc = lib.llmc_sumsq_accumulate(x.data_ptr(), dt, x.shape[0], K, x.stride(0), want.data_ptr(), ws.data_ptr(), nws, st)
    assert rc == 0
    torch.cuda.synchronize()
    # torch's allocator counter sees torch allocations only; the driver's free-byte figure also sees a hipMalloc made
    # inside the library (the array's address was resolved by the first call of the process, before these figures)
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info(dev)[0]
    rc = lib.llmc_sumsq_accumulate_noalloc(x.data_ptr(), dt, x.shape[0], K, x.stride(0), got.data_ptr(), st)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
    if _both.warm:
        assert torch.cuda.mem_get_info(dev)[0] >= free_before
    _both.warm = True
    return want.cpu(), got.cpu(), base.cpu()


_both.warm = False


def _check_sum(x, got, base):
    ref = (x.double() ** 2).sum(0).cpu()
    err = ((got.double() - base.double()) - ref).abs().max().item()
    # fp32 sums of up to 4096 squares in 64 slices against the fp64 sum
    assert err <= 1e-5 * ref.abs().max().item() + 1e-6, err


def test_no_alloc_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    from llmcompressor_amd import _lib

    lib = _lib.lib()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    # first call: wide and long (fills 64 slices x 14336 columns of the array)
    x1 = torch.randn(4096, 14336, device=dev).bfloat16()
    want, got, base = _both(x1, 14336)
    assert torch.equal(want, got)
    _check_sum(x1, got, base)
    # second call, smaller in both directions (fewer slices than 64, fewer columns, odd width -> scalar loads)
    x2 = torch.randn(37, 1001, device=dev).half()
    want2, got2, base2 = _both(x2, 1001)
    assert torch.equal(want2, got2)
    _check_sum(x2, got2, base2)
    # third: fp32 rows with a row stride, again over stale contents
    x3 = torch.randn(300, 4096, device=dev)[:, :2048]
    want3, got3, base3 = _both(x3, 2048)
    assert torch.equal(want3, got3)
    _check_sum(x3, got3, base3)
    # beyond the array's capacity: refused, nothing written
    K = 16384 + 8
    xb = torch.ones(8, K, device=dev, dtype=torch.bfloat16)
    out = torch.zeros(K, device=dev)
    rc = lib.llmc_sumsq_accumulate_noalloc(xb.data_ptr(), 0, 8, K, K, out.data_ptr(),
                                           torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    assert rc == -4 and not out.any()
    # the largest width it takes
    xm = torch.randn(128, 16384, device=dev).bfloat16()
    wantm, gotm, basem = _both(xm, 16384)
    assert torch.equal(wantm, gotm)
    _check_sum(xm, gotm, basem)
