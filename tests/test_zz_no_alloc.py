"""mxq_quantize_v2_noalloc (reduction partials in the library's own device array, nothing
allocated) against mxq_quantize_v2 with a caller workspace: bit-identical outputs and
ranges, on two calls in a row, the second with a smaller input."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, entry, x, out_type, workspace):
    dt = torch.int8 if out_type == 5 else torch.uint8
    out = torch.empty(x.numel(), dtype=dt, device="cuda")
    mn = torch.empty(1, device="cuda")
    mx = torch.empty(1, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [st, P(x), P(out), P(mn), P(mx), x.numel(), out_type, 0, 0.0, 0.0]
    if workspace is not None:
        args += [P(workspace), workspace.numel()]
    rc = getattr(lib, entry)(*args)
    assert rc == 0, lib.mxq_last_error()
    return out, mn, mx


@pytest.mark.parametrize("out_type", [5, 3])
def test_no_alloc_matches_workspace_entry_point(out_type):
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    g = torch.Generator(device="cuda").manual_seed(7)
    big = torch.randn(5_000_003, device="cuda", generator=g) * 3.0
    small = torch.randn(70_001, device="cuda", generator=g) * 0.25
    ws = torch.empty(lib.mxq_quantize_v2_workspace(big.numel()), dtype=torch.uint8,
                     device="cuda")
    # everything the calls need exists before the first of them; the entry point itself
    # must not allocate, so the allocator's counters may not move across the two calls
    outs = []
    for x in (big, small):          # second call: fewer partials than the first left behind
        want = _run(lib, "mxq_quantize_v2", x, out_type, ws)
        torch.cuda.synchronize()
        dt = torch.int8 if out_type == 5 else torch.uint8
        out = torch.empty(x.numel(), dtype=dt, device="cuda")
        mn, mx = torch.empty(1, device="cuda"), torch.empty(1, device="cuda")
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        mid = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        rc = lib.mxq_quantize_v2_noalloc(st, P(x), P(out), P(mn), P(mx), x.numel(), out_type, 0,
                                         0.0, 0.0)
        assert rc == 0, lib.mxq_last_error()
        torch.cuda.synchronize()
        # neither torch's allocator nor the driver handed out memory during the call
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == mid
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(out, want[0])
        assert (mn.item(), mx.item()) == (want[1].item(), want[2].item())
        xn = x.cpu().numpy()
        if out_type == 3:
            assert (mn.item(), mx.item()) == (float(xn.min()), float(xn.max()))
        else:
            r = float(np.abs(xn).max())
            assert (mn.item(), mx.item()) == (-r, r)
        outs.append(out)


def test_no_alloc_calibrated_and_limits():
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    x = torch.linspace(-2.0, 2.0, 4099, device="cuda")
    out = torch.empty(x.numel(), dtype=torch.int8, device="cuda")
    ref = torch.empty(x.numel(), dtype=torch.int8, device="cuda")
    sc = [torch.empty(1, device="cuda") for _ in range(4)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.mxq_quantize_v2_noalloc(st, P(x), P(out), P(sc[0]), P(sc[1]), x.numel(), 5, 1,
                                       -1.5, 1.0) == 0
    assert lib.mxq_quantize_v2(st, P(x), P(ref), P(sc[2]), P(sc[3]), x.numel(), 5, 1, -1.5, 1.0,
                               None, 0) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    assert (sc[0].item(), sc[1].item()) == (sc[2].item(), sc[3].item()) == (-1.5, 1.5)
    # beyond the stated maximum: refused before anything is launched
    rc = lib.mxq_quantize_v2_noalloc(st, P(x), P(out), P(sc[0]), P(sc[1]), (1 << 31) + 1, 5, 0,
                                     0.0, 0.0)
    assert rc == -1 and "at most" in mxnet_amd._lib.last_error()
