"""The non-allocating sort/bin entry point (mi_moe_sort_bin_static) against the workspace-taking one.

Called through the C ABI with caller-allocated inputs and outputs only; results must be bit-identical to
mi_moe_sort_bin on the same input (integer work), on two calls in a row, the second with a smaller input that
leaves most of the library's scratch array holding the first call's contents."""

import pytest
import torch

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


def _selection(T, k, E, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.rand(T, E, generator=g).argsort(dim=1)[:, :k].to(torch.int32).contiguous()


def _run_static(lib, sel, E, device, check_no_alloc=False):
    """The call through the C ABI.  With ``check_no_alloc`` the device's free memory and torch's reserved memory
    are read right before the call and after it has finished: the entry point exists for callers that cannot
    allocate, so neither may move (the library's code object and the scratch address are set up by the first call
    of the process, which is why the first call is not checked)."""
    T, k = sel.shape
    ids = sel.to(device)
    L = T * k
    se = torch.full((L,), -1, dtype=torch.int32, device=device)
    ss = torch.full((L,), -1, dtype=torch.int32, device=device)
    off = torch.full((E,), -1, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    free0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    rc = lib.mi_moe_sort_bin_static(ids.data_ptr(), T, k, E, se.data_ptr(), ss.data_ptr(), off.data_ptr(), stream)
    torch.cuda.synchronize()
    free1, reserved1 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    assert rc == 0, lib.mi_moe_strerror(rc).decode()
    if check_no_alloc:
        assert free1 == free0 and reserved1 == reserved0, "mi_moe_sort_bin_static changed the device's free memory"
    return se, ss, off


def test_sort_bin_static_matches_workspace_entry_point(device):
    from dolomite_engine_amd import _lib, ops

    lib = _lib.load()
    # first a large input (scratch: 40 experts x 128 chunks), then smaller ones; the last fits one block and
    # touches no scratch at all
    for n, (T, k, E) in enumerate([(32768, 8, 40), (5000, 3, 1000), (2100, 6, 64), (64, 6, 64)]):
        sel = _selection(T, k, E, seed=T + k + E)
        print(f"sort_bin_static T={T} k={k} E={E}", flush=True)
        se, ss, off = _run_static(lib, sel, E, device, check_no_alloc=n > 0)
        rse, rss, roff = ops.sort_bin(sel.to(device), E)
        torch.cuda.synchronize()
        assert torch.equal(off, roff)
        assert torch.equal(se, rse)
        assert torch.equal(ss, rss)
        ose, oss, ooff = oracle.sort_bin(sel.long(), E)
        assert torch.equal(off.cpu().long(), ooff) and torch.equal(se.cpu().long(), ose)
        assert torch.equal(ss.cpu().long(), oss)


def test_sort_bin_static_refuses_what_does_not_fit(device):
    from dolomite_engine_amd import _lib

    lib = _lib.load()
    # 1000 experts x 4096 chunks of 2048 slots need 16 MB of histograms: more than the fixed array
    T, k, E = 1 << 20, 8, 1000
    assert lib.mi_moe_sort_bin_workspace_bytes(T * k, E) > (1 << 20)
    dummy = torch.zeros(16, dtype=torch.int32, device=device)
    p = dummy.data_ptr()
    rc = lib.mi_moe_sort_bin_static(p, T, k, E, p, p, p, None)
    assert rc == _lib.MI_MOE_ETOOLARGE
    assert "scratch" in lib.mi_moe_strerror(rc).decode()


def test_sort_bin_static_at_the_limit_of_its_scratch(device):
    """An input whose histograms need exactly the fixed array (512 experts x 511 chunks + one row = 2^20 bytes) runs
    and equals the workspace entry point; one more chunk is refused."""
    from dolomite_engine_amd import _lib, ops

    lib = _lib.load()
    E, k = 512, 1
    T_fit, T_over = 511 * 2048, 511 * 2048 + 1
    assert lib.mi_moe_sort_bin_workspace_bytes(T_fit * k, E) == (1 << 20)
    assert lib.mi_moe_sort_bin_workspace_bytes(T_over * k, E) > (1 << 20)
    g = torch.Generator().manual_seed(511)
    sel = torch.randint(0, E, (T_over, k), generator=g, dtype=torch.int32)
    print(f"sort_bin_static at the limit T={T_fit} k={k} E={E}", flush=True)
    _run_static(lib, _selection(5000, 3, 64, seed=5), 64, device)   # the process's first call sets the library up
    se, ss, off = _run_static(lib, sel[:T_fit].contiguous(), E, device, check_no_alloc=True)
    rse, rss, roff = ops.sort_bin(sel[:T_fit].to(device), E)
    torch.cuda.synchronize()
    assert torch.equal(off, roff) and torch.equal(se, rse) and torch.equal(ss, rss)
    order = torch.sort(sel[:T_fit, 0].long(), stable=True)
    assert torch.equal(ss.cpu().long(), order.indices) and torch.equal(se.cpu().long(), order.values)
    ids = sel.to(device)
    p = ids.data_ptr()
    rc = lib.mi_moe_sort_bin_static(p, T_over, k, E, p, p, p, None)   # refused on the host, before any launch
    assert rc == _lib.MI_MOE_ETOOLARGE
