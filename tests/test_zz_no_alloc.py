"""The entry point that allocates nothing (tfcc_rocm_gemv_u8s8s32_noalloc) against the ordinary one
(tfcc_rocm_gemv_u8s8s32): same int32 sums and same dequantized floats, bit for bit, on two calls in a row that
share the workspace inside the library, the second one smaller than the first."""
import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu


def _case(rng, m, n, k):
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    scale_b = rng.uniform(0.001, 0.01, n).astype(np.float32)
    return a, b, O.reduce_sum(a, True), O.reduce_sum(b, False), scale_b


def test_no_alloc_entry_point_matches_the_ordinary_one(pkg, T):
    import torch
    rng = np.random.default_rng(77)
    # K-split kernel (workspace in use) at the decode size, then a smaller product of the same kind, then one
    # small enough for the kernel without a workspace
    for m, n, k in ((8, 11008, 4096), (3, 4096, 2048), (5, 260, 80)):
        print("no-alloc gemv", m, n, k, flush=True)
        a, b, rs, cs, scale_b = _case(rng, m, n, k)
        ta, tb, trs, tcs, tsb = T.t(a), T.t(b), T.t(rs), T.t(cs), T.t(scale_b)
        out = torch.empty((m, n), dtype=torch.float32, device=ta.device)
        acc = torch.empty((m, n), dtype=torch.int32, device=ta.device)
        # the new entry point first: in a fresh process this is the library's first launch
        pkg.gemv_dequant(ta, tb, trs, tcs, -57, 93, 0.02, tsb, out=out, acc=acc, no_alloc=True)
        got_out, got_acc = T.n(out).copy(), T.n(acc).copy()
        want_out, want_acc = pkg.gemv_dequant(ta, tb, trs, tcs, -57, 93, 0.02, tsb)
        assert np.array_equal(got_acc, T.n(want_acc))
        assert np.array_equal(got_out.view(np.uint32), T.n(want_out).view(np.uint32))
        assert np.array_equal(got_acc, O.qgemm(a, b, -57, 93, rs, cs))
        # again on the same workspace (it was left clean), and this time watching the free device memory: it drops
        # with any allocation, the library's own included
        acc.zero_()
        out.zero_()
        torch.cuda.synchronize()
        before = torch.cuda.mem_get_info()[0]
        pkg.gemv_dequant(ta, tb, trs, tcs, -57, 93, 0.02, tsb, out=out, acc=acc, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before
        assert np.array_equal(T.n(acc), T.n(want_acc))
        assert np.array_equal(T.n(out).view(np.uint32), T.n(want_out).view(np.uint32))


def test_no_alloc_entry_point_beyond_its_workspace(pkg, T):
    """Wider than the workspace inside the library: the kernel that needs no workspace takes the product (same sums);
    what neither kernel takes is refused with a clear error instead of being routed to a path that allocates."""
    import torch
    rng = np.random.default_rng(78)
    m, n, k = 2, 32768 + 256, 1024
    a, b, rs, cs, scale_b = _case(rng, m, n, k)
    ta, tb, trs, tcs = T.t(a), T.t(b), T.t(rs), T.t(cs)
    acc = torch.empty((m, n), dtype=torch.int32, device="cuda")
    pkg.gemv_dequant(ta, tb, trs, tcs, -57, 93, 1.0, None, acc=acc, no_alloc=True)
    assert np.array_equal(T.n(acc), O.qgemm(a, b, -57, 93, rs, cs))
    # nine rows: not a skinny product
    a9 = torch.zeros((9, k), dtype=torch.uint8, device="cuda")
    rs9 = torch.zeros((9,), dtype=torch.int32, device="cuda")
    acc9 = torch.empty((9, n), dtype=torch.int32, device="cuda")
    with pytest.raises(Exception, match="without allocation"):
        pkg.gemv_dequant(a9, tb, rs9, tcs, 0, 0, 1.0, None, acc=acc9, no_alloc=True)
