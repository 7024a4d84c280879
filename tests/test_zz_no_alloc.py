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
    # What the entry point cannot help is the HIP runtime loading a kernel's code onto the GPU at that kernel's first
    # launch in the process, so one call per kernel involved comes first, on operands of zeros (callers that must not
    # allocate - a stream being recorded, for one - warm up the same way); from then on nothing may be allocated.
    for m, n, k in ((1, 4096, 2048), (4, 4096, 2048), (8, 4096, 2048), (1, 64, 64)):
        za = torch.zeros((m, k), dtype=torch.uint8, device="cuda")
        zb = torch.zeros((k, n), dtype=torch.int8, device="cuda")
        zr, zc = torch.zeros((m,), dtype=torch.int32, device="cuda"), torch.zeros((n,), dtype=torch.int32, device="cuda")
        zacc = torch.empty((m, n), dtype=torch.int32, device="cuda")
        pkg.gemv_dequant(za, zb, zr, zc, 0, 0, 1.0, None, acc=zacc, no_alloc=True)
        assert int(zacc.abs().max()) == 0
    for m, n, k in ((8, 11008, 4096), (3, 4096, 2048), (5, 260, 80)):
        print("no-alloc gemv", m, n, k, flush=True)
        a, b, rs, cs, scale_b = _case(rng, m, n, k)
        ta, tb, trs, tcs, tsb = T.t(a), T.t(b), T.t(rs), T.t(cs), T.t(scale_b)
        out = torch.empty((m, n), dtype=torch.float32, device=ta.device)
        acc = torch.empty((m, n), dtype=torch.int32, device=ta.device)
        # The new entry point before the ordinary one has run on this product: the free device memory is read on
        # both sides of the call (it drops with any allocation, the library's own included).
        torch.cuda.synchronize()
        before_first = torch.cuda.mem_get_info()[0]
        pkg.gemv_dequant(ta, tb, trs, tcs, -57, 93, 0.02, tsb, out=out, acc=acc, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before_first
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
