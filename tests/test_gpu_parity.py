"""GPU parity tests: every compute entry point of the C ABI against the CPU oracle and the committed
outputs of the reference's own kernels.  Integer and byte results must be bit-exact; fp32 matmul
must be within a relative Frobenius error of 1e-5 of the float64 result."""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from golden.make_golden import BENCH_RANGES, SMALL_CASES, bench_out_range, gen_inputs

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FP32_TOL = 1e-5  # relative Frobenius error allowed for fp32 matmul


def wrap32(x):
    return (np.asarray(x, np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


from conftest import rel_fro  # noqa: E402



# ---- quantized matmul ----------------------------------------------------------------------------

@pytest.mark.parametrize("seed,shape_a,shape_b", SMALL_CASES)
def test_qgemm_golden_vectors(pkg, T, seed, shape_a, shape_b):
    """All shape families (matrix, batched x batched, batched x matrix, matrix x batched, N == 1)
    with float ranges in device memory, against the reference kernel's stored outputs."""
    print("case", seed, shape_a, shape_b, flush=True)
    z = np.load(os.path.join(GOLDEN, "qgemm_ref_vectors.npz"))
    p = "case%d/" % seed
    a, b = z[p + "a"], z[p + "b"]
    ranges = [float(v) for v in z[p + "ranges"]]
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    r = [T.f1(v) for v in ranges]
    c, mn_c, mx_c = pkg.quantization_matmul(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3])
    assert np.array_equal(T.n(c), z[p + "c"])
    assert (float(T.n(mn_c)[0]), float(T.n(mx_c)[0])) == O.qmatmul_range(*ranges)
    mn_o, mx_o = [float(v) for v in z[p + "out_range"]]
    q, c2, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                     T.f1(mn_o), T.f1(mx_o), want_acc=True)
    assert np.array_equal(T.n(c2), z[p + "c"])
    assert np.array_equal(T.n(q), z[p + "q"])
    q_promised, _, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                              T.f1(mn_o), T.f1(mx_o), colsum_exact=True)
    assert np.array_equal(T.n(q_promised), T.n(q))  # cs holds the true column sums: the promise changes nothing
    q_only, none, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2],
                                                            r[3], T.f1(mn_o), T.f1(mx_o), want_acc=False)
    assert none is None and np.array_equal(T.n(q_only), z[p + "q"])
    # the stand-alone requantize pass gives the same bytes
    q_sep = pkg.requantize(c, mn_c, mx_c, T.f1(mn_o), T.f1(mx_o), __import__("torch").uint8)
    assert np.array_equal(T.n(q_sep), z[p + "q"])


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 16, 16), (5, 7, 3), (31, 33, 15), (64, 64, 64), (100, 260, 72),
                                   (257, 129, 130), (128, 128, 2048), (300, 516, 1040), (512, 768, 256),
                                   (1000, 1012, 1040), (2048, 2048, 512), (768, 4096, 1024)])
def test_qgemm_shapes_against_oracle(pkg, T, m, n, k):
    """Ragged, unaligned, tail-in-K and multi-tile shapes; both tile configurations and the
    unaligned path are exercised.  Offsets wrap around int32 on purpose in one case."""
    print("shape", m, n, k, flush=True)
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    for oa, ob in ((-128, 0), (-57, 93), (70000, -90000)):
        want = O.qgemm(a, b, oa, ob, rs, cs)
        got = pkg.quantization_matmul_offsets(T.t(a), T.t(rs), T.t(b), T.t(cs), oa, ob)
        assert np.array_equal(T.n(got), want), (oa, ob)


def test_qgemm_uses_caller_sums_as_given(pkg, T):
    """rowsum / colsum tensors that are NOT the true sums, and a rank-1 sum shared by a batch."""
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (3, 70, 48), dtype=np.uint8)
    b = rng.integers(-128, 128, (3, 48, 36), dtype=np.int8)
    rs = rng.integers(-10000, 10000, 70).astype(np.int32)      # rank 1: shared by the batch
    cs = rng.integers(-10000, 10000, (3, 36)).astype(np.int32)
    oa, ob = -31, 17
    want = wrap32(48 * oa * ob + rs[None, :, None].astype(np.int64) * ob + cs[:, None, :].astype(np.int64) * oa +
                  np.matmul(a.astype(np.int64), b.astype(np.int64)))
    assert np.array_equal(O.qgemm(a, b, oa, ob, rs, cs), want)
    got = pkg.quantization_matmul_offsets(T.t(a), T.t(rs), T.t(b), T.t(cs), oa, ob)
    assert np.array_equal(T.n(got), want)


@pytest.mark.parametrize("name", ["c3_1024_ragged", "c3_4096"])
def test_qgemm_full_size_hash(pkg, T, name):
    """The benchmark configuration at full size: SHA-256 of the int32 accumulators and of the fused
    uint8 output against the reference kernel's (int32 matmul + AVX2 requantize) on the same seeded inputs."""
    print("hash case", name, flush=True)
    h = json.load(open(os.path.join(GOLDEN, "qgemm_ref_hashes.json")))[name]
    a, b = gen_inputs(h["seed"], h["shape_a"], h["shape_b"])
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    r = [T.f1(v) for v in h["ranges"]]
    mn_o, mx_o = h["out_range"]
    q, c, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                    T.f1(mn_o), T.f1(mx_o), want_acc=True)
    assert hashlib.sha256(T.n(c).tobytes()).hexdigest() == h["sha256_c"]
    assert hashlib.sha256(T.n(q).tobytes()).hexdigest() == h["sha256_q"]
    q2, _, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                     T.f1(mn_o), T.f1(mx_o), want_acc=False)
    assert hashlib.sha256(T.n(q2).tobytes()).hexdigest() == h["sha256_q"]
    # with the promise that the column sums passed in are the true ones (they are) the kernel skips its own
    for want_acc in (False, True):
        q3, c3, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                          T.f1(mn_o), T.f1(mx_o), want_acc=want_acc, colsum_exact=True)
        assert hashlib.sha256(T.n(q3).tobytes()).hexdigest() == h["sha256_q"]
        assert c3 is None or hashlib.sha256(T.n(c3).tobytes()).hexdigest() == h["sha256_c"]
    # sums computed on the device equal the oracle's
    assert np.array_equal(T.n(pkg.reduce_sum(T.t(a), True)), rs)
    assert np.array_equal(T.n(pkg.reduce_sum(T.t(b), False)), cs)


def test_qgemm_requant_immediate_scalars(pkg, T):
    """The fused kernel with host-computed scalars (the kernel-level form of the C ABI)."""
    import ctypes as C
    import torch
    rng = np.random.default_rng(6)
    m, n, k = 300, 272, 208
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    oa, ob = O.qmatmul_offsets(*BENCH_RANGES)
    want_c = O.qgemm(a, b, oa, ob, rs, cs)
    mn_c, mx_c = O.qmatmul_range(*BENCH_RANGES)
    mn_o, mx_o = bench_out_range(k)
    want_q = O.requantize_s32_u8(want_c, mn_c, mx_c, mn_o, mx_o)
    in_s, in_m = O.dequantized_scale_info(32, mn_c, mx_c)
    out_s, out_o = O.quantized_scale_info(8, mn_o, mx_o)
    ta, tb, trs, tcs = T.t(a), T.t(b), T.t(rs), T.t(cs)
    d = pkg.QGemmDesc()
    d.a, d.b, d.rowsum_a, d.colsum_b = ta.data_ptr(), tb.data_ptr(), trs.data_ptr(), tcs.data_ptr()
    d.m, d.n, d.k, d.batch, d.stride_c = m, n, k, 1, m * n
    d.offset_a, d.offset_b = oa, ob
    q = torch.empty((m, n), dtype=torch.uint8, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_gemm_u8s8s32_requant_u8(torch.cuda.current_stream().cuda_stream, C.byref(d), None,
                                                           q.data_ptr(), in_s, in_m, out_s, out_o, None, None))
    assert np.array_equal(T.n(q), want_q)
    # a range pair that takes the exact int64 epilogue (the double shortcut is not provably exact there)
    mn_o2, mx_o2 = 0.0, 1e-30
    want_q2 = O.requantize_s32_u8(want_c, mn_c, mx_c, mn_o2, mx_o2)
    out_s2, out_o2 = O.quantized_scale_info(8, mn_o2, mx_o2)
    pkg.check(pkg.lib().tfcc_rocm_gemm_u8s8s32_requant_u8(torch.cuda.current_stream().cuda_stream, C.byref(d), None,
                                                           q.data_ptr(), in_s, in_m, out_s2, out_o2, None, None))
    assert np.array_equal(T.n(q), want_q2)


# ---- skinny (decode) shapes -------------------------------------------------------------------------

@pytest.mark.parametrize("m", [1, 4, 8])
@pytest.mark.parametrize("n,k", [(11008, 4096), (128, 64), (260, 80), (4096, 4000), (176, 272), (1024, 8192), (512, 8320)])
def test_gemv_against_oracle(pkg, T, m, n, k):
    print("gemv", m, n, k, flush=True)
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    scale_b = rng.uniform(0.001, 0.01, n).astype(np.float32)
    scale_a = float(np.float32(0.02))
    for oa, ob in ((-128, 0), (-57, 93)):
        want = O.qgemm(a, b, oa, ob, rs, cs)
        out, acc = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(cs), oa, ob, scale_a, T.t(scale_b))
        assert np.array_equal(T.n(acc), want), (oa, ob)
        assert np.array_equal(T.n(out), O.dequant_per_channel(want, scale_a, scale_b))
        # second call in a row reuses the workspace and the tickets
        out2, _ = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(cs), oa, ob, scale_a, T.t(scale_b), want_acc=False)
        assert np.array_equal(T.n(out2), T.n(out))
    # the general entry point routes these shapes to the same kernel
    got = pkg.quantization_matmul_offsets(T.t(a), T.t(rs), T.t(b), T.t(cs), -128, 0)
    assert np.array_equal(T.n(got), O.qgemm(a, b, -128, 0, rs, cs))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 4000), (1024, 8192), (2048, 16448)])
def test_gemv_with_column_sums_declared_exact(pkg, T, m, n, k):
    """Every row count of the K-split kernel (rows padded to 1, 4 or 8; one or several parts of K; two rows per
    workspace word or one), with the kernel's own column sums and with the caller's promise that colsum_b holds them."""
    print("gemv exact", m, n, k, flush=True)
    rng = np.random.default_rng(1000 * m + n + k)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    if m == 8:  # extreme operands: every partial sum at its bound
        a[:4] = 255
        b[:, ::2] = -128
        b[:, 1::4] = 127
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    scale_b = rng.uniform(0.001, 0.01, n).astype(np.float32)
    want = O.qgemm(a, b, -57, 93, rs, cs)
    for exact in (False, True):
        for rep in range(2):  # the second call finds the workspace as the first one left it
            out, acc = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(cs), -57, 93, 0.02, T.t(scale_b), colsum_exact=exact)
            assert np.array_equal(T.n(acc), want), (exact, rep)
            assert np.array_equal(T.n(out), O.dequant_per_channel(want, float(np.float32(0.02)), scale_b))
    # without the promise the caller's sums are used as given, as the reference uses them
    wrong = (cs - 5).astype(np.int32)
    _, acc = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(wrong), -57, 93, 1.0, None)
    assert np.array_equal(T.n(acc), O.qgemm(a, b, -57, 93, rs, wrong))


def test_gemv_beyond_one_round_of_workgroups(pkg, T):
    """A B so wide that sixteen-wavefront workgroups of one step each would be more than a thousand: the kernel of
    four wavefronts that walk several steps takes it."""
    m, n, k = 3, 69632, 4096
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    want = O.qgemm(a, b, -128, 0, rs, cs)
    for exact in (False, True):
        _, acc = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(cs), -128, 0, 1.0, None, colsum_exact=exact)
        assert np.array_equal(T.n(acc), want), exact


def test_gemv_recorded_into_a_graph(pkg, T):
    """A skinny product recorded into a HIP graph: with a workspace from an earlier call the K-split kernel is
    recorded; on a stream that has none yet nothing may be allocated while recording, and the kernel without a
    workspace takes the launch.  Either way every replay gives the oracle's sums, also after a wider product on the
    same stream has outgrown the workspace the graph was recorded with."""
    import ctypes
    import torch
    lib = pkg.lib()
    m, n, k = 4, 4096, 4096
    rng = np.random.default_rng(9)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    want = O.qgemm(a, b, -57, 93, rs, cs)
    ta, tb, trs, tcs = T.t(a), T.t(b), T.t(rs), T.t(cs)
    for warm in (False, True):
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            stream = side.cuda_stream
            acc = torch.zeros((m, n), dtype=torch.int32, device=ta.device)
            call = lambda: pkg.check(lib.tfcc_rocm_gemv_u8s8s32(stream, ta.data_ptr(), tb.data_ptr(), trs.data_ptr(),  # noqa: E731
                                                                tcs.data_ptr(), -57, 93, m, n, k, acc.data_ptr(), 1.0, None, None))
            if warm:
                call()
                torch.cuda.synchronize()
            graph = ctypes.c_void_p()
            pkg.check(lib.tfcc_rocm_stream_begin_capture(stream))
            call()
            pkg.check(lib.tfcc_rocm_stream_end_capture(stream, ctypes.byref(graph)))
            for replay in range(3):
                acc.zero_()
                torch.cuda.synchronize()
                pkg.check(lib.tfcc_rocm_graph_launch(graph, stream))
                torch.cuda.synchronize()
                assert np.array_equal(T.n(acc), want), (warm, replay)
                if replay == 0:
                    # a wider product on the same stream: the workspace grows, the one recorded stays valid
                    n2 = 8192
                    b2 = torch.zeros((k, n2), dtype=torch.int8, device=ta.device)
                    cs2 = torch.zeros((n2,), dtype=torch.int32, device=ta.device)
                    acc2 = torch.empty((m, n2), dtype=torch.int32, device=ta.device)
                    pkg.check(lib.tfcc_rocm_gemv_u8s8s32(stream, ta.data_ptr(), b2.data_ptr(), trs.data_ptr(), cs2.data_ptr(),
                                                         0, 0, m, n2, k, acc2.data_ptr(), 1.0, None, None))
                    torch.cuda.synchronize()
                    assert int(acc2.abs().max()) == 0
            pkg.check(lib.tfcc_rocm_graph_destroy(graph))
            pkg.check(lib.tfcc_rocm_stream_release(stream))


@pytest.mark.parametrize("m", [1, 5, 8])
@pytest.mark.parametrize("n,k", [(11008, 4096), (16, 16), (100, 80), (260, 4000), (4096, 8320), (64, 12352)])
def test_gemv_on_packed_weights(pkg, T, m, n, k):
    print("gemv packed", m, n, k, flush=True)
    rng = np.random.default_rng(m * 7 + n + k)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    scale_b = rng.uniform(0.001, 0.01, n).astype(np.float32)
    scale_a = float(np.float32(0.02))
    packed = pkg.gemv_pack(T.t(b))
    for oa, ob in ((-128, 0), (-57, 93)):
        want = O.qgemm(a, b, oa, ob, rs, cs)
        out, acc = pkg.gemv_dequant_packed(T.t(a), packed, n, T.t(rs), T.t(cs), oa, ob, scale_a, T.t(scale_b))
        assert np.array_equal(T.n(acc), want), (oa, ob)
        assert np.array_equal(T.n(out), O.dequant_per_channel(want, scale_a, scale_b))
    # column sums as given by the caller, as the reference uses them
    wrong = (cs + 3).astype(np.int32)
    _, acc = pkg.gemv_dequant_packed(T.t(a), packed, n, T.t(rs), T.t(wrong), -57, 93, 1.0, None)
    assert np.array_equal(T.n(acc), O.qgemm(a, b, -57, 93, rs, wrong))


def test_gemv_full_size_hash(pkg, T):
    h = json.load(open(os.path.join(GOLDEN, "qgemm_ref_hashes.json")))["c5_m8"]
    a, b = gen_inputs(h["seed"], h["shape_a"], h["shape_b"])
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    _, acc = pkg.gemv_dequant(T.t(a), T.t(b), T.t(rs), T.t(cs), h["offsets"][0], h["offsets"][1], 1.0, None)
    assert hashlib.sha256(T.n(acc).tobytes()).hexdigest() == h["sha256_c"]


# ---- sums, quantize, requantize, dequantize ----------------------------------------------------------

@pytest.mark.parametrize("shape", [
    (1, 1), (17, 29), (3, 64, 256), (2, 100, 1000), (4096, 512), (5, 7, 16),
    # 16-byte column groups: the wide column-sum kernel; row counts on both sides of its 16-row rounds and 64-row slabs,
    # column counts that leave part of the last 1024-column block empty, extreme values (all -128 / 127 / 255)
    (64, 16), (65, 1040), (2, 130, 2064), (4096, 4096), (1000, 11008), (3, 63, 32), (127, 48)])
def test_reduce_sum(pkg, T, shape):
    rng = np.random.default_rng(sum(shape))
    cases = [rng.integers(0, 256, shape, dtype=np.uint8), rng.integers(-128, 128, shape, dtype=np.int8)]
    if shape[-2] >= 64 and shape[-2] * shape[-1] <= 1 << 21:
        cases += [np.full(shape, 255, np.uint8), np.full(shape, -128, np.int8), np.full(shape, 127, np.int8)]
    for x in cases:
        assert np.array_equal(T.n(pkg.reduce_sum(T.t(x), True)), O.reduce_sum(x, True))
        got = T.n(pkg.reduce_sum(T.t(x), False))
        assert np.array_equal(got, O.reduce_sum(x, False))
        assert np.array_equal(got, x.astype(np.int64).sum(axis=-2))  # the closed form, independent of the oracle


def test_requantize_known_answer_and_fma_cases(pkg, T):
    import torch
    # tfcc/test/quantization.cpp:88-101 (int8 -> uint16; torch has no uint16 arithmetic: use int16 storage)
    a = np.array([23, -115, -128, 127, -20, -11], np.int8)
    ta = T.t(a)
    out = torch.empty(6, dtype=torch.int16, device=ta.device)
    r = [T.f1(-2.5), T.f1(3.4), T.f1(-12.7), T.f1(24.5)]  # kept alive until the kernel has run
    pkg.check(pkg.lib().tfcc_rocm_requantize(torch.cuda.current_stream().cuda_stream, ta.data_ptr(), pkg.S8,
                                              out.data_ptr(), pkg.U16, 6, r[0].data_ptr(), r[1].data_ptr(),
                                              r[2].data_ptr(), r[3].data_ptr()))
    assert T.n(out).view(np.uint16).tolist() == [24125, 18500, 17970, 28364, 22372, 22739]
    # inputs on which the fused multiply-add decides: outputs of the reference's AVX2 kernel
    for c in json.load(open(os.path.join(GOLDEN, "requantize_fma_cases.json")))["cases"]:
        acc = np.asarray(c["acc"], np.int32)
        got = pkg.requantize(T.t(acc), T.f1(c["minIn"]), T.f1(c["maxIn"]), T.f1(c["minOut"]), T.f1(c["maxOut"]),
                             torch.uint8)
        assert T.n(got).tolist() == c["ref_avx2"]


def test_requantize_against_oracle(pkg, T):
    import torch
    rng = np.random.default_rng(40)
    for total in (1, 3, 4, 1000, 4099, 1 << 16):
        acc = rng.integers(-2 ** 31, 2 ** 31, total).astype(np.int32)
        for (mi, ma, mo, mxo) in ((-1000.0, 1000.0, -300.0, 310.0), (-2147483648.0, 2147483648.0, -33554432.0, 33292288.0),
                                  (-1.0, 1.0, 2.0, 2.0), (1.5, 1.5, -4.0, 4.0), (-3.0, 5.0, 0.5, -0.5),
                                  # output scale so large that the int64 conversion overflows: exact integer path
                                  (-1000.0, 1000.0, 0.0, 1e-30), (-1e30, 1e30, -1e-3, 1e-3),
                                  # output offset near 2^31: the double shortcut, not the int32 one
                                  (8388607.5, 8388610.0, 8388608.0, 8388609.0)):
            got = pkg.requantize(T.t(acc), T.f1(mi), T.f1(ma), T.f1(mo), T.f1(mxo), torch.uint8)
            assert np.array_equal(T.n(got), O.requantize_s32_u8(acc, mi, ma, mo, mxo)), (total, mi, ma, mo, mxo)
    # ties: nearest-even like the reference's AVX2 kernel
    a8 = np.arange(-128, 128).astype(np.int8)
    out = torch.empty(256, dtype=torch.int16, device=T.t(a8).device)
    ta = T.t(a8)
    r = [T.f1(-128.0), T.f1(127.0), T.f1(-65535.0), T.f1(65535.0)]
    pkg.check(pkg.lib().tfcc_rocm_requantize(torch.cuda.current_stream().cuda_stream, ta.data_ptr(), pkg.S8,
                                              out.data_ptr(), pkg.U16, 256, r[0].data_ptr(), r[1].data_ptr(),
                                              r[2].data_ptr(), r[3].data_ptr()))
    assert np.array_equal(T.n(out).view(np.uint16), O.requantize_s8_u16(a8, -128.0, 127.0, -65535.0, 65535.0))


def test_dequantize_and_quantize_against_oracle(pkg, T):
    import torch
    rng = np.random.default_rng(41)
    a = np.array([23, -115, -128, 127, -20, -11], np.int8)
    got = T.n(pkg.dequantize(T.t(a), T.f1(-2.5), T.f1(3.4)))
    assert np.array_equal(got, O.dequantize(a, -2.5, 3.4))
    q = rng.integers(-2 ** 31, 2 ** 31, 5000).astype(np.int32)
    assert np.array_equal(T.n(pkg.dequantize(T.t(q), T.f1(-3.25), T.f1(7.5))), O.dequantize(q, -3.25, 7.5))
    assert np.array_equal(T.n(pkg.dequantize(T.t(q), T.f1(3.0), T.f1(3.0))), np.full(5000, 3.0, np.float32))
    u = rng.integers(0, 256, 777, dtype=np.uint8)
    assert np.array_equal(T.n(pkg.dequantize(T.t(u), T.f1(-1.0), T.f1(2.0))), O.dequantize(u, -1.0, 2.0))
    x = rng.uniform(-5, 5, 4097).astype(np.float32)
    x[:50] = np.float32(np.arange(50) * 0.5 - 12)
    for dtype, tdt in ((np.uint8, torch.uint8), (np.int8, torch.int8)):
        for mn, mx in ((-5.0, 5.0), (-8.0, 7.9375), (3.0, 3.0)):
            got = pkg.quantize(T.t(x), tdt, T.f1(mn), T.f1(mx))
            assert np.array_equal(T.n(got), O.quantize(x, mn, mx, dtype))
        got, mn_t, mx_t = pkg.quantize(T.t(x), tdt)
        mn, mx = float(x.min()), float(x.max())
        assert (float(T.n(mn_t)[0]), float(T.n(mx_t)[0])) == (mn, mx)
        assert np.array_equal(T.n(got), O.quantize(x, mn, mx, dtype))
    const = np.full(100, 1.25, np.float32)
    got, _, _ = pkg.quantize(T.t(const), torch.int8)
    assert np.array_equal(T.n(got), np.full(100, -128, np.int8))


@pytest.mark.parametrize("total", [4096, 65540, 9_000_004])
def test_streaming_quantization_kernels_at_size(pkg, T, total):
    """The four-loads-in-flight kernels over sizes of one pass, a partial pass and several passes of the capped
    grid: requantize int32 -> uint8 (both the general and the folded arithmetic), dequantize int32, quantize with
    a given range and with the range found by the two-step reduction that parks its partial results in the
    output buffer."""
    import torch
    rng = np.random.default_rng(total)
    acc = rng.integers(-2 ** 26, 2 ** 26, total).astype(np.int32)
    acc[:8] = (-2 ** 31, 2 ** 31 - 1, 0, -1, 1, 131072, -131072, 393216)
    mn_c, mx_c = O.qmatmul_range(-128.0, 127.0, -128.0, 127.0)
    for mn_o, mx_o in ((-128.0 * 2 ** 18, 127.0 * 2 ** 18), (-3.1e7, 2.9e7)):  # power-of-two scale / general
        got = pkg.requantize(T.t(acc), T.f1(mn_c), T.f1(mx_c), T.f1(mn_o), T.f1(mx_o), torch.uint8)
        assert np.array_equal(T.n(got), O.requantize_s32_u8(acc, mn_c, mx_c, mn_o, mx_o))
    assert np.array_equal(T.n(pkg.dequantize(T.t(acc), T.f1(-3.25), T.f1(7.5))), O.dequantize(acc, -3.25, 7.5))
    x = rng.normal(0, 2, total).astype(np.float32)
    x[total // 3] = 11.5     # the extremes away from the ends
    x[total // 2] = -13.25
    for dtype, tdt in ((np.uint8, torch.uint8), (np.int8, torch.int8)):
        got = pkg.quantize(T.t(x), tdt, T.f1(-6.0), T.f1(6.5))
        assert np.array_equal(T.n(got), O.quantize(x, -6.0, 6.5, dtype))
        got, mn_t, mx_t = pkg.quantize(T.t(x), tdt)
        assert (float(T.n(mn_t)[0]), float(T.n(mx_t)[0])) == (-13.25, 11.5)
        assert np.array_equal(T.n(got), O.quantize(x, -13.25, 11.5, dtype))


def test_quantized_matmul_round_trip(pkg, T):
    """tfcc/test/quantization.cpp:105-189: quantize -> reduce_sum -> matmul -> dequantize gives 5, 11, 17."""
    import torch
    for shape_a, shape_b in (((2, 3, 2), (2, 2, 1)), ((3, 2), (2, 2, 1)), ((2, 3, 2), (2, 1))):
        v1 = np.array([1, 2, 3, 4, 5, 6] * (2 if len(shape_a) == 3 else 1), np.float32).reshape(shape_a)
        v2 = np.array([1, 2] * (2 if len(shape_b) == 3 else 1), np.float32).reshape(shape_b)
        qa, mn_a, mx_a = pkg.quantize(T.t(v1), torch.uint8)
        qb, mn_b, mx_b = pkg.quantize(T.t(v2), torch.int8)
        ra, rb = pkg.reduce_sum(qa, True), pkg.reduce_sum(qb, False)
        qc, mn_c, mx_c = pkg.quantization_matmul(qa, ra, mn_a, mx_a, qb, rb, mn_b, mx_b)
        out = T.n(pkg.dequantize(qc, mn_c, mx_c))
        assert out.astype(np.int64).reshape(-1).tolist() == [5, 11, 17, 5, 11, 17]


# ---- fp32 matmul -------------------------------------------------------------------------------------

def test_sgemm_config_c1(pkg, T):
    """[128,768] x [768,3072] + bias[3072], U[-1,1) / U[-0.1,0.1): relative Frobenius error <= 1e-5."""
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, (128, 768)).astype(np.float32)
    b = rng.uniform(-1, 1, (768, 3072)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, 3072).astype(np.float32)
    _, want = O.sgemm(a, b, bias, want64=True)
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b), T.t(bias)))
    assert got.shape == (128, 3072) and rel_fro(got, want) <= FP32_TOL
    _, want2 = O.sgemm(a, b, want64=True)
    assert rel_fro(T.n(pkg.blas_matmul(T.t(a), T.t(b))), want2) <= FP32_TOL


@pytest.mark.parametrize("shape_a,shape_b", [
    ((16, 12, 128, 64), (1, 12, 64, 64)),   # one weight per head, shared by the batch
    ((1, 12, 128, 64), (16, 12, 64, 64)), ((2, 3, 1, 7, 8), (2, 3, 4, 8, 6)), ((5, 1, 3, 4), (1, 1, 4, 2)),
    ((3, 1, 33, 20), (1, 4, 20, 17)),
])
def test_matmul_broadcast_of_leading_dimensions(pkg, T, shape_a, shape_b):
    """Leading dimensions of extent 1 stand for every index of the other operand's (the reference raises for
    unequal leading dimensions, tfcc/core/operations/tfcc_blas.cpp:36-42).  Checked against the oracle's
    two-dimensional product, one batch entry at a time."""
    rng = np.random.default_rng(sum(shape_a) * 3 + sum(shape_b))
    a = rng.normal(0, 1, shape_a).astype(np.float32)
    b = rng.normal(0, 1, shape_b).astype(np.float32)
    bias = rng.uniform(-1, 1, shape_b[-1]).astype(np.float32)
    lead = tuple(max(x, y) for x, y in zip(shape_a[:-2], shape_b[:-2]))
    ab = np.broadcast_to(a, lead + shape_a[-2:]).reshape((-1,) + shape_a[-2:])
    bb = np.broadcast_to(b, lead + shape_b[-2:]).reshape((-1,) + shape_b[-2:])
    want = np.stack([O.sgemm(np.ascontiguousarray(x), np.ascontiguousarray(y), bias, want64=True)[1] for x, y in zip(ab, bb)])
    want = want.reshape(lead + (shape_a[-2], shape_b[-1]))
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b), T.t(bias)))
    assert got.shape == want.shape and rel_fro(got, want) <= FP32_TOL
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b)))
    assert rel_fro(got, want - bias) <= FP32_TOL


def test_sgemm_exact_cases(pkg, T):
    rng = np.random.default_rng(20)
    a = rng.uniform(-1, 1, (137, 253)).astype(np.float32)
    eye = np.eye(253, dtype=np.float32)
    mm = lambda x, y, *b: T.n(pkg.blas_matmul(T.t(x), T.t(y), *[T.t(v) for v in b]))
    assert np.array_equal(mm(a, eye), a)
    perm = rng.permutation(253)
    assert np.array_equal(mm(a, eye[:, perm]), a[:, perm])
    assert np.array_equal(mm(eye[perm], a.T.copy()), a.T[perm])
    assert np.array_equal(mm(np.ones((5, 64), np.float32), np.ones((64, 7), np.float32)), np.full((5, 7), 64, np.float32))
    assert np.array_equal(mm(a * 4, eye * 0.5), a * 2)
    x = np.arange(6, dtype=np.float32).reshape(2, 3)
    y = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert mm(x, y).tolist() == [[20, 23, 26, 29], [56, 68, 80, 92]]
    assert mm(x, y, np.array([1, 2, 3, 4], np.float32)).tolist() == [[21, 25, 29, 33], [57, 70, 83, 96]]


@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (128, 96, 40), (256, 512, 512), (8, 128, 64), (1, 4096, 512),
                                   (1024, 768, 768)])
def test_sgemm_keeps_subnormal_operands_and_results(pkg, T, m, n, k):
    """fp32 values below 2^-126.  The reference's dispatch thread sets flush-to-zero and denormals-are-zero before it
    runs any kernel (tfcc/mkl/framework/tfcc_mkldevice.cpp:126-128), so on the CPU a subnormal operand counts as 0 and a
    subnormal result becomes 0.  The fp32 matrix ops and the streaming kernel of this backend follow IEEE gradual
    underflow instead: operands are taken as they are and subnormal results are produced.  Pinned here on all tile
    families (register-staged, direct-to-LDS with and without K groups, few-rows streaming kernel) with powers of two,
    whose products and sums are exact whatever the order; the two oracles differ in exactly the elements named."""
    a = np.zeros((m, k), np.float32)
    b = np.zeros((k, n), np.float32)
    a[0, 0], b[0, :] = np.float32(2.0 ** -130), np.float32(2.0 ** 10)        # subnormal operand, normal product
    ieee = np.zeros((m, n), np.float64)
    flushed = np.zeros((m, n), np.float64)
    ieee[0, :] = 2.0 ** -120                                                   # DAZ: the operand is 0
    if m > 1:
        a[1, 1], b[1, :] = np.float32(2.0 ** -70), np.float32(2.0 ** -70)      # normal operands, subnormal product
        ieee[1, :] = 2.0 ** -140                                               # FTZ: the result is 0
    if m > 2:
        a[2, 2:], b[2:, :] = np.float32(2.0 ** -100), np.float32(2.0 ** -30)   # k - 2 subnormal products of 2^-130
        ieee[2, :] = (k - 2) * 2.0 ** -130
        flushed[2, :] = np.nan  # depends on where an implementation flushes its partial sums: not compared
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b))).astype(np.float64)
    assert np.array_equal(got, ieee)
    rows = slice(0, min(m, 2))
    assert np.all(got[rows] != flushed[rows]) and np.all(flushed[rows] == 0.0)
    # the oracle (fp64 accumulation, one rounding to fp32) is the IEEE flavour too
    want32, _ = O.sgemm(a, b, None, want64=True)
    assert np.array_equal(want32.astype(np.float64), ieee)


@pytest.mark.parametrize("shape_a,shape_b", [
    ((1, 1), (1, 1)), ((5, 7), (7, 3)), ((33, 65), (65, 31)), ((99, 98), (98, 97)),
    ((3, 50, 20), (3, 20, 30)), ((4, 25, 40), (40, 24)), ((31, 48), (2, 48, 52)), ((2, 3, 17, 9), (2, 3, 9, 33)),
    ((16, 12, 128, 64), (16, 12, 64, 128)),      # attention scores Q.K^T
    ((16, 12, 128, 128), (16, 12, 128, 64)),     # attention P.V
    ((8, 128, 768), (768, 3072)), ((8, 128, 3072), (3072, 768)),   # BERT-base FFN
    ((1024, 1024), (1024, 4096)),                # enough tiles for the 128x128 configuration
    ((130, 36), (36, 516)), ((257, 100), (100, 260)),
    # few tiles and a long K: several K groups per workgroup (x4, x2), with ragged K and edges
    ((1024, 768), (768, 768)), ((200, 1000), (1000, 300)), ((300, 300), (300, 500)), ((64, 516), (516, 64)),
    ((3, 70, 1028), (1028, 90)),
    ((100, 600), (600, 200)), ((128, 768), (768, 3072)),   # 32x96 tiles, ragged edges
])
def test_sgemm_shapes_against_oracle(pkg, T, shape_a, shape_b):
    """The four shape families of tfcc/test/blas.cpp:34-61 plus the benchmark's batched shapes."""
    print("sgemm", shape_a, shape_b, flush=True)
    rng = np.random.default_rng(sum(shape_a) + sum(shape_b))
    a = rng.normal(0, 1, shape_a).astype(np.float32)
    b = rng.normal(0, 1, shape_b).astype(np.float32)
    bias = rng.uniform(-1, 1, shape_b[-1]).astype(np.float32)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b)))
    assert got.shape == want.shape and rel_fro(got, want) <= FP32_TOL
    got_b = T.n(pkg.blas_matmul(T.t(a), T.t(b), T.t(bias)))
    assert rel_fro(got_b, want + bias) <= FP32_TOL
    # the reference's own element-wise tolerance (tfcc/core/utils/tfcc_debugutils.cpp:102-111), at the
    # sizes its generator draws (m, n, k < 100): larger K makes near-zero sums fail it for any fp32 order
    if shape_a[-1] < 100:
        ref32 = O.sgemm(a, b)
        assert np.all((np.abs(got - ref32) < 1e-3 * np.abs(got + ref32)) | (np.abs(got - ref32) < 1e-5))


@pytest.mark.parametrize("b,s,h,d", [(8, 128, 12, 64), (2, 50, 3, 20), (3, 33, 2, 18), (1, 7, 1, 4)])
def test_sgemm_general_multiplies_permuted_views_in_place(pkg, T, b, s, h, d):
    """attention without materialised transposes: Q, K, V and the context in [batch, seq, heads, size] order"""
    import torch
    rng = np.random.default_rng(b + s + h + d)
    q, k, v = (rng.normal(0, 1, (b, s, h, d)).astype(np.float32) for _ in range(3))
    tq, tk, tv = T.t(q), T.t(k), T.t(v)
    scores = torch.empty((b, h, s, s), dtype=torch.float32, device=tq.device)
    pkg.sgemm_general(tq, tk, scores, s, s, d, h * d, h * d, s, trans_b=True, batch_outer=b, batch_inner=h,
                      strides=(s * h * d, s * h * d, h * s * s), inner_strides=(d, d, s * s))
    want = np.einsum("bshd,bthd->bhst", q.astype(np.float64), k.astype(np.float64))
    assert rel_fro(T.n(scores), want) <= FP32_TOL
    p = np.ascontiguousarray(T.n(scores))
    ctx = torch.full((b, s, h, d), float("nan"), dtype=torch.float32, device=tq.device)
    pkg.sgemm_general(T.t(p), tv, ctx, s, d, s, s, h * d, h * d, batch_outer=b, batch_inner=h,
                      strides=(h * s * s, s * h * d, s * h * d), inner_strides=(s * s, d, d))
    want_ctx = np.einsum("bhst,bthd->bshd", p.astype(np.float64), v.astype(np.float64))
    got_ctx = T.n(ctx)
    assert not np.isnan(got_ctx).any() and rel_fro(got_ctx, want_ctx) <= FP32_TOL
    # the same product through the dense entry point after explicit transposes: bit-identical
    dense = T.n(pkg.blas_matmul(T.t(np.ascontiguousarray(q.transpose(0, 2, 1, 3))),
                                T.t(np.ascontiguousarray(k.transpose(0, 2, 3, 1)))))
    assert np.array_equal(dense, T.n(scores))


@pytest.mark.parametrize("m,n,k,groups", [
    (1024, 768, 768, 3), (100, 52, 36, 4), (64, 64, 1028, 2), (7, 4, 4, 1),
    # 128 x 96 tiles shared by the products (four and two K groups' worth of sums per tile), ragged edges
    (1000, 760, 768, 3), (2048, 768, 768, 2), (2040, 764, 512, 2)])
def test_sgemm_grouped_equals_separate_launches(pkg, T, m, n, k, groups):
    rng = np.random.default_rng(m + n + k + groups)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    bs = [rng.normal(0, 1, (k, n)).astype(np.float32) for _ in range(groups)]
    biases = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(groups)]
    outs = pkg.sgemm_grouped(T.t(a), [T.t(b) for b in bs], [T.t(b) for b in biases])
    for b, bias, out in zip(bs, biases, outs):
        single = T.n(pkg.blas_matmul(T.t(a), T.t(b), T.t(bias)))
        assert np.array_equal(T.n(out), single)
        assert rel_fro(T.n(out), a.astype(np.float64) @ b.astype(np.float64) + bias) <= FP32_TOL


def test_matmul_validation_and_empty(pkg, T):
    """Error behaviour of tfcc::blas::matmul (tfcc/core/operations/tfcc_blas.cpp:26-54)."""
    z = lambda *s: T.t(np.zeros(s, np.float32))
    with pytest.raises(pkg.InvalidArgumentError, match="two or more dimensions"):
        pkg.blas_matmul(z(3), z(3, 4))
    for sa, sb in (((2, 3, 4), (5, 6, 4, 7)), ((3, 4), (5, 6)), ((2, 3, 4), (3, 4, 5))):
        with pytest.raises(pkg.InvalidArgumentError, match="shape invalid"):
            pkg.blas_matmul(z(*sa), z(*sb))
    with pytest.raises(pkg.InvalidArgumentError, match="shape invalid"):
        pkg.blas_matmul(z(3, 4), z(4, 5), z(4))
    assert tuple(pkg.blas_matmul(z(2, 0, 4), z(2, 4, 5)).shape) == (2, 0, 5)
    assert tuple(pkg.blas_matmul(z(6, 3, 4), z(4, 5)).shape) == (6, 3, 5)


# ---- element-wise neighbours --------------------------------------------------------------------------

def test_unary_functions_against_numpy_float64(pkg, T):
    """tfcc_rocm_unary_f32 against the expressions of tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:48-110,222-228,
    284-291 evaluated in float64; sizes on both sides of the grid-stride loop's first pass."""
    import math
    rng = np.random.default_rng(12)
    ref = {"sigmoid": lambda x: 1 / (1 + np.exp(-x)), "tanh": np.tanh, "relu": lambda x: np.maximum(x, 0),
           "softplus": lambda x: np.log(np.exp(x) + 1), "log": np.log, "rsqrt": lambda x: 1 / np.sqrt(x),
           "erf": np.vectorize(math.erf), "abs": np.abs, "sign": np.sign, "neg": lambda x: -x,
           "reciprocal": lambda x: 1 / x, "sqrt": np.sqrt}
    assert set(ref) == set(pkg.UNARY)
    for total in (1, 255, 70001):
        x = rng.normal(0, 3, total).astype(np.float32)
        pos = rng.uniform(1e-4, 100, total).astype(np.float32)
        for name, f in ref.items():
            src = pos if name in ("log", "rsqrt", "sqrt") else x
            got = T.n(pkg.unary(name, T.t(src)))
            assert np.allclose(got, f(src.astype(np.float64)), rtol=2e-6, atol=1e-7), (name, total)
    with pytest.raises(pkg.TfccRocmError):
        pkg.check(pkg.lib().tfcc_rocm_unary_f32(None, 99, 16, 1, 16))


@pytest.mark.parametrize("batch,units,input_size", [(1, 1, 1), (3, 67, 5), (4, 256, 64), (2, 511, 130), (64, 1024, 8)])
def test_recurrent_cells_against_oracle(pkg, T, batch, units, input_size):
    """The four cells of CellInterface against the scalar restatement of tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:
    same expressions, device expf / tanhf instead of libm's (a few ulp)."""
    rng = np.random.default_rng(batch * 1000 + units)
    u = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)  # noqa: E731
    state, c = u(batch, units), u(batch, units)
    x4, h4, b4 = u(batch, 4 * units) * 3, u(batch, 4 * units) * 3, u(4 * units)
    x3, h3, b2 = u(batch, 3 * units) * 3, u(batch, 3 * units) * 3, u(2 * units)
    v2, inputs, cv, cb, bi, bh = u(batch, 2 * units) * 3, u(batch, input_size), u(batch, units) * 3, u(units), u(units), u(units)
    tol = dict(rtol=2e-6, atol=2e-7)
    for forget in (0.0, 1.0):
        h, cs = pkg.lstm_cell(T.t(c), T.t(x4), T.t(h4), T.t(b4), forget)
        wh, wc = O.lstm_cell(c, x4, h4, b4, forget)
        assert np.allclose(T.n(h), wh, **tol) and np.allclose(T.n(cs), wc, **tol)
    got = T.n(pkg.gru_cell_gates(T.t(state), T.t(inputs), T.t(v2), T.t(b2)))
    assert np.array_equal(got[:, :input_size], inputs)
    assert np.allclose(got, O.gru_cell_gates(state, inputs, v2, b2), **tol)
    assert np.allclose(T.n(pkg.gru_cell_candidate(T.t(state), T.t(v2), T.t(b2), T.t(cv), T.t(cb))),
                       O.gru_cell_candidate(state, v2, b2, cv, cb), **tol)
    assert np.allclose(T.n(pkg.pytorch_gru_cell(T.t(state), T.t(x3), T.t(h3), T.t(b2), T.t(bi), T.t(bh))),
                       O.pytorch_gru_cell(state, x3, h3, b2, bi, bh), **tol)
    with pytest.raises(pkg.InvalidArgumentError, match="invalid inputValue"):
        pkg.lstm_cell(T.t(c), T.t(x3), T.t(h4), T.t(b4), 0.0)
    with pytest.raises(pkg.InvalidArgumentError, match="invalid cBias"):
        pkg.gru_cell_candidate(T.t(state), T.t(v2), T.t(b2), T.t(cv), T.t(b2))


def test_lstm_cell_in_place_state_and_sequence(pkg, T):
    """The cell may write cs over stateC (each thread reads its element before writing it): a short sequence
    driven through the C ABI the way tfcc::rnn::lstm_forward (tfcc/core/operations/tfcc_rnn.cpp:29-81) is,
    against the oracle's sequence."""
    import torch
    rng = np.random.default_rng(8)
    seq, batch, length, hidden = 6, 3, 48, 40
    u = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)  # noqa: E731
    a, wi, wh, bias, ih, ic = u(seq, batch, length), u(length, 4 * hidden), u(hidden, 4 * hidden), u(4 * hidden), \
        u(batch, hidden), u(batch, hidden)
    want_out, want_h, want_c = O.lstm_sequence(a, wi, wh, bias, ih, ic)
    xw = pkg.blas_matmul(T.t(a.reshape(seq * batch, length)), T.t(wi))
    out = torch.empty((seq, batch, hidden), dtype=torch.float32, device=xw.device)
    c, h, dwh, dbias = T.t(ic.copy()), T.t(ih), T.t(wh), T.t(bias)
    for t in range(seq):
        hv = pkg.blas_matmul(h, dwh)
        pkg.check(pkg.lib().tfcc_rocm_lstm_cell_f32(None, batch, hidden, c.data_ptr(), xw[t * batch:].data_ptr(),
                                                    hv.data_ptr(), dbias.data_ptr(), 0.0, out[t].data_ptr(), c.data_ptr()))
        h = out[t]
    for got, want in ((T.n(out), want_out), (T.n(h), want_h), (T.n(c), want_c)):
        assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)


def test_gather_slice_concat_cast_equal_numpy(pkg, T):
    """Row gather (out-of-range indices give zeros, tfcc/mkl/interfaces/tfcc_mklgatherinterface.cpp:35-39), slice and
    concat along every axis (byte, 4-byte and 16-byte copy paths), casts between element types: numpy bit for bit."""
    import torch
    rng = np.random.default_rng(13)
    table = rng.normal(size=(50, 768)).astype(np.float32)
    for idx_type in (np.int32, np.int64):
        idx = rng.integers(-3, 55, (4, 9)).astype(idx_type)
        want = np.where(((idx >= 0) & (idx < 50))[..., None], table[np.clip(idx, 0, 49)], 0).astype(np.float32)
        assert np.array_equal(T.n(pkg.gather(T.t(table), T.t(idx))), want)
    small = rng.integers(-100, 100, (7, 3), dtype=np.int8)          # 3-byte rows: the byte path
    assert np.array_equal(T.n(pkg.gather(T.t(small), T.t(np.array([6, 0, 7, 2], np.int32)))),
                          np.concatenate([small[[6, 0]], np.zeros((1, 3), np.int8), small[[2]]]))
    odd = rng.normal(size=(5, 3, 6)).astype(np.float32)             # 72-byte rows: the 4-byte path
    assert np.array_equal(T.n(pkg.gather(T.t(odd), T.t(np.array([[4], [1]], np.int64)))), odd[[[4], [1]]])
    x = rng.normal(size=(3, 10, 8, 4)).astype(np.float32)
    for axis, start, end in ((0, 1, 3), (1, 0, 10), (1, 3, 4), (2, 5, 99), (3, 1, 3)):
        assert np.array_equal(T.n(pkg.slice_axis(T.t(x), axis, start, end)), np.take(x, range(start, min(end, x.shape[axis])), axis))
    for bad, text in (((4, 0, 1), "invalid axis"), ((1, 3, 3), "start large than end"), ((1, 10, 12), "invalid start")):
        with pytest.raises(pkg.InvalidArgumentError, match=text):
            pkg.slice_axis(T.t(x), *bad)
    for axis in range(4):
        parts = [rng.normal(size=[d if i != axis else n for i, d in enumerate(x.shape)]).astype(np.float32) for n in (1, 5, 2)]
        assert np.array_equal(T.n(pkg.concat([T.t(p) for p in parts], axis)), np.concatenate(parts, axis))
    bytes_ = [rng.integers(0, 255, (3, n), dtype=np.uint8) for n in (5, 2, 9)]
    assert np.array_equal(T.n(pkg.concat([T.t(b) for b in bytes_], 1)), np.concatenate(bytes_, 1))
    with pytest.raises(pkg.InvalidArgumentError, match="invalid shape"):
        pkg.concat([T.t(x), T.t(x[:, :, :7])], 1)
    ints = rng.integers(-1000, 1000, (33, 7)).astype(np.int32)
    floats = (rng.normal(size=(33, 7)) * 50).astype(np.float32)
    for src, dtype, np_dtype in ((ints, torch.float32, np.float32), (floats, torch.int32, np.int32), (ints, torch.int64, np.int64),
                                 (floats, torch.float64, np.float64), (ints, torch.int8, np.int8), (floats, torch.int64, np.int64)):
        assert np.array_equal(T.n(pkg.cast(T.t(src), dtype)), src.astype(np_dtype))


def test_reductions_pow_max_min_clip_leaky_relu(pkg, T):
    """Reductions over the trailing dimensions (tfcc/mkl/interfaces/tfcc_mklreduceinterface.cpp:107-230) against numpy
    float64 (sum, mean, product) and exactly (maximum, minimum); rows shorter and longer than a wavefront's and a
    workgroup's share; pow / max / min of two tensors, clip and leaky relu of one."""
    rng = np.random.default_rng(41)
    for shape, keep in (((7, 33), 1), ((3, 5, 64), 1), ((2, 3, 4100), 2), ((5, 9000), 1), ((4, 1), 1), ((6, 2, 3), 0)):
        x = rng.uniform(0.5, 1.5, shape).astype(np.float32) * rng.choice([-1.0, 1.0], shape).astype(np.float32)
        axes = tuple(range(keep, len(shape)))
        x64 = x.astype(np.float64)
        for op, ref in (("sum", np.sum), ("mean", np.mean), ("max", np.max), ("min", np.min)):
            got = T.n(pkg.reduce_trailing(op, T.t(x), keep))
            want = ref(x64, axis=axes, keepdims=True)
            assert got.shape == want.shape
            if op in ("max", "min"):
                assert np.array_equal(got, want.astype(np.float32))
            else:
                assert np.allclose(got, want, rtol=1e-5, atol=1e-4), (op, shape)
        small = rng.uniform(0.9, 1.1, shape).astype(np.float32)
        got = T.n(pkg.reduce_trailing("prod", T.t(small), keep))
        assert np.allclose(got, np.prod(small.astype(np.float64), axis=axes, keepdims=True), rtol=1e-4)
    with pytest.raises(pkg.InvalidArgumentError, match="invalid keep dims"):
        pkg.reduce_trailing("sum", T.t(np.zeros((2, 3), np.float32)), 2)
    a = rng.uniform(0.1, 3, (5, 7, 33)).astype(np.float32)
    b = rng.uniform(-2, 2, (5, 7, 33)).astype(np.float32)
    row = rng.uniform(-2, 2, 33).astype(np.float32)
    assert np.allclose(T.n(pkg.binary("pow", T.t(a), T.t(b))), np.power(a.astype(np.float64), b), rtol=2e-6)
    assert np.allclose(T.n(pkg.binary("pow", T.t(a), T.t(row))), np.power(a.astype(np.float64), row), rtol=2e-6)
    assert np.array_equal(T.n(pkg.binary("max", T.t(b), T.t(row))), np.maximum(b, row))
    assert np.array_equal(T.n(pkg.binary("min", T.t(b), T.t(a))), np.minimum(b, a))
    assert np.array_equal(T.n(pkg.clip(T.t(b), -0.5, 1.25)), np.clip(b, np.float32(-0.5), np.float32(1.25)))
    assert np.array_equal(T.n(pkg.leaky_relu(T.t(b), 0.1)), np.where(b > 0, b, b * np.float32(0.1)))


def test_comparisons_and_argmax(pkg, T):
    """tfcc::relation's six comparisons: tensor against value (tfcc/core/interfaces/tfcc_comparisoninterface.h:38-83) and
    tensor against tensor, where the reference compares the difference with 0 in the element type
    (tfcc/core/operations/tfcc_relation.cpp:101-115): unsigned differences wrap, so `less` never holds for them.
    tfcc::math::argmax: first position of the largest element (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:469-485)."""
    rng = np.random.default_rng(47)
    refs = {"equal": np.equal, "unequal": np.not_equal, "greater": np.greater, "greater_equal": np.greater_equal,
            "less": np.less, "less_equal": np.less_equal}
    for dtype in (np.float32, np.int32, np.int64, np.uint8, np.int8, np.float64):
        a = rng.integers(0, 5, (3, 4, 33)).astype(dtype)
        b = rng.integers(0, 5, (4, 1)).astype(dtype)
        for op, ref in refs.items():
            got = T.n(pkg.compare(op, T.t(a), 2))
            assert got.dtype == np.uint8 and np.array_equal(got, ref(a, dtype(2)).astype(np.uint8)), (op, dtype)
            with np.errstate(over="ignore"):
                diff = (a - b).astype(dtype)
            got = T.n(pkg.compare(op, T.t(a), T.t(b)))
            assert np.array_equal(got, ref(diff, dtype(0)).astype(np.uint8)), (op, dtype)
    inf = np.array([np.inf, 1.0], np.float32)
    assert T.n(pkg.compare("equal", T.t(inf), T.t(inf))).tolist() == [0, 1]       # inf - inf is not 0
    assert T.n(pkg.compare("equal", T.t(inf), float("inf"))).tolist() == [1, 0]
    with pytest.raises(pkg.InvalidArgumentError):
        pkg.compare("equal", T.t(np.zeros((0, 3), np.float32)), 1.0)
    for shape, axis in (((5, 7, 9), 0), ((5, 7, 9), 1), ((5, 7, 9), 2), ((6, 300), 1), ((3, 64), 1), ((2, 5000), 1),
                        ((1, 1), 0)):
        x = rng.integers(0, 12, shape).astype(np.float32)       # many ties: the first position must win
        got = T.n(pkg.argmax(T.t(x), axis))
        assert got.dtype == np.int64 and np.array_equal(got, np.argmax(x, axis=axis, keepdims=True)), (shape, axis)
    x = rng.normal(size=(4, 200)).astype(np.float32)
    x[1, 0] = np.nan            # a NaN in the first place stays: nothing is greater
    x[2, 77] = np.nan           # elsewhere it is never taken
    want = np.array([np.argmax(x[0]), 0, np.nanargmax(x[2]), np.argmax(x[3])]).reshape(4, 1)
    assert np.array_equal(T.n(pkg.argmax(T.t(x), 1)), want)
    # the same along the first axis, which is cut into ranges that each start from the axis' first element
    xt = np.ascontiguousarray(x.T)
    assert np.array_equal(T.n(pkg.argmax(T.t(xt), 0)), want.reshape(1, 4))
    with pytest.raises(pkg.InvalidArgumentError, match="invalid axis"):
        pkg.argmax(T.t(x), 2)


def test_where_and_triangles(pkg, T):
    """tfcc::nn::where with tensor / value operands and tfcc::base::tril / triu
    (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:398-466) against numpy, on several element types."""
    rng = np.random.default_rng(59)
    for dtype in (np.float32, np.int64, np.uint8, np.int16, np.float64):
        cond = rng.integers(0, 3, (3, 5, 17)).astype(np.uint8)
        x = rng.integers(-50, 50, cond.shape).astype(dtype)
        y = rng.integers(-50, 50, cond.shape).astype(dtype)
        assert np.array_equal(T.n(pkg.where(T.t(cond), T.t(x), T.t(y))), np.where(cond != 0, x, y))
        assert np.array_equal(T.n(pkg.where(T.t(cond), 7, T.t(y))), np.where(cond != 0, dtype(7), y))
        assert np.array_equal(T.n(pkg.where(T.t(cond), T.t(x), 9)), np.where(cond != 0, x, dtype(9)))
        for rows, cols in ((5, 5), (3, 9), (9, 3), (1, 1)):
            m = rng.integers(1, 50, (rows, cols)).astype(dtype)
            for k in (0, 1, -1, 4, -4, 100, -100):
                assert np.array_equal(T.n(pkg.triangle(T.t(m), k, False)), np.tril(m, k)), (rows, cols, k)
                assert np.array_equal(T.n(pkg.triangle(T.t(m), k, True)), np.triu(m, k)), (rows, cols, k)
    with pytest.raises(pkg.InvalidArgumentError, match="different shape"):
        pkg.where(T.t(np.zeros((2, 3), np.uint8)), T.t(np.zeros((3, 2), np.float32)), 1.0)
    with pytest.raises(pkg.InvalidArgumentError, match="invalid shape"):
        pkg.triangle(T.t(np.zeros((2, 3, 4), np.float32)), 0, True)


def test_top_k(pkg, T):
    """tfcc::math::top_k (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:159-260, :779-800): the k largest of each row,
    descending.  Values are checked exactly against a sort; positions against a stable sort (equal values in ascending
    position: the reference leaves that order to its heaps), also with ties, negative zero and infinities."""
    rng = np.random.default_rng(67)
    cases = [((3, 50), 5), ((2, 4, 300), 17), ((1, 30000), 8), ((5, 7), 7), ((4, 1), 1), ((6, 64), 64)]
    for shape, k in cases:
        for ties in (False, True):
            x = (rng.integers(-4, 5, shape) if ties else rng.normal(size=shape)).astype(np.float32)
            if ties and x.shape[-1] > 3:
                x[..., 1] = np.inf
                x[..., 2] = -np.inf
                x[..., 0] = -0.0
            values, positions = pkg.top_k(T.t(x), k)
            order = np.argsort(-x.astype(np.float64), axis=-1, kind="stable")[..., :k]
            assert np.array_equal(T.n(positions), order), (shape, k, ties)
            assert np.array_equal(T.n(values).view(np.uint32), np.take_along_axis(x, order, axis=-1).view(np.uint32))
    with pytest.raises(pkg.InvalidArgumentError, match="invalid k"):
        pkg.top_k(T.t(np.zeros((2, 3), np.float32)), 4)
    # a deliberate choice where the reference's heap comparison leaves the order open: a NaN counts as the largest,
    # several of them in ascending position, +inf next
    x = np.array([[1.0, np.nan, np.inf, -2.0, np.nan, 7.0]], np.float32)
    values, positions = pkg.top_k(T.t(x), 4)
    assert T.n(positions).tolist() == [[1, 4, 2, 5]]
    assert np.isnan(T.n(values)[0, :2]).all() and T.n(values)[0, 2:].tolist() == [np.inf, 7.0]
    # the selection makes one pass per element: beyond 1024 it is refused
    with pytest.raises(pkg.TfccRocmError, match="beyond the 1024"):
        pkg.top_k(T.t(np.zeros((1, 4096), np.float32)), 1025)


BROADCAST_PAIRS = [
    ((2, 4, 8, 8), (2, 1, 1, 8)),        # attention scores + mask
    ((3, 1, 5), (1, 4, 1)),              # both sides broadcast
    ((5, 6), (1,)), ((1,), (5, 6)),      # a one-element tensor on either side
    ((7, 33), (33,)), ((33,), (7, 33)),  # bias forms, either order
    ((2, 3, 4, 5, 6, 7), (2, 1, 4, 1, 6, 1)),  # six groups
    ((4, 1, 6), (4, 5, 6)), ((1, 1, 9), (8, 1, 1)), ((16, 12, 128, 128), (16, 1, 1, 128)),
]


@pytest.mark.parametrize("sa,sb", BROADCAST_PAIRS)
def test_broadcast_arithmetic_equals_numpy(pkg, T, sa, sb):
    """tfcc::math::add / sub / mul / div with the broadcasting of tfcc/core/operations/tfcc_math.cpp:38-104: one
    rounding per element, so the results are numpy's bit for bit."""
    rng = np.random.default_rng(len(sa) * 100 + len(sb))
    a = rng.normal(0, 2, sa).astype(np.float32)
    b = rng.uniform(0.5, 3, sb).astype(np.float32) * rng.choice([-1, 1], sb).astype(np.float32)
    for op, ref in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        got = T.n(pkg.math_binary(op, T.t(a), T.t(b)))
        want = ref(a, b)
        assert got.shape == want.shape and np.array_equal(got, want), op


def test_broadcast_arithmetic_rejects_what_the_reference_rejects(pkg, T):
    a = T.t(np.zeros((2, 3), np.float32))
    with pytest.raises(pkg.InvalidArgumentError, match="broadcast failed"):
        pkg.math_binary("add", a, T.t(np.zeros((2, 2), np.float32)))
    with pytest.raises(pkg.InvalidArgumentError, match="broadcast failed"):
        pkg.math_binary("mul", a, T.t(np.zeros((4, 1, 3, 3), np.float32)))
    assert tuple(pkg.math_binary("add", T.t(np.zeros((0, 3), np.float32)), T.t(np.zeros((1, 3), np.float32))).shape) == (0, 3)


@pytest.mark.parametrize("seq,batch,length,hidden", [(6, 3, 48, 40), (3, 1, 32, 513), (4, 8, 64, 128), (2, 5, 16, 7)])
def test_lstm_step_in_one_launch(pkg, T, seq, batch, length, hidden):
    """tfcc_rocm_lstm_step_f32 (state product and cell in one launch, state kernel with interleaved gates) driven as
    tfcc::rnn::lstm_forward drives its steps, against the oracle's sequence and against product + cell launches."""
    import torch
    rng = np.random.default_rng(hidden)
    u = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)  # noqa: E731
    a, wi, wh, bias, ih, ic = u(seq, batch, length), u(length, 4 * hidden), u(hidden, 4 * hidden), u(4 * hidden), \
        u(batch, hidden), u(batch, hidden)
    want_out, want_h, want_c = O.lstm_sequence(a, wi, wh, bias, ih, ic)
    xw = pkg.blas_matmul(T.t(a.reshape(seq * batch, length)), T.t(wi))
    inter = pkg.transpose(T.t(wh.reshape(hidden, 4, hidden)), (0, 2, 1)).reshape(hidden, 4 * hidden)
    assert np.array_equal(T.n(inter)[:, 4 * 3 + 2], wh[:, 2 * hidden + 3]) if hidden > 3 else True
    out = torch.empty((seq, batch, hidden), dtype=torch.float32, device=xw.device)
    c, h, dbias = T.t(ic.copy()), T.t(ih), T.t(bias)
    for t in range(seq):
        pkg.check(pkg.lib().tfcc_rocm_lstm_step_f32(None, batch, hidden, h.data_ptr(), inter.data_ptr(),
                                                    xw[t * batch:].data_ptr(), dbias.data_ptr(), 0.0, c.data_ptr(),
                                                    out[t].data_ptr(), c.data_ptr()))
        h = out[t]
    for got, want in ((T.n(out), want_out), (T.n(h), want_h), (T.n(c), want_c)):
        assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    # one step against the separate launches on the same operands: the same expressions on sums that differ only in
    # the order of their partial sums
    tih, tic = T.t(ih), T.t(ic)
    hv = pkg.blas_matmul(tih, T.t(wh))
    h2, c2 = pkg.lstm_cell(tic, xw[:batch].contiguous(), hv, dbias, 0.0)
    h1 = torch.empty_like(h2)
    c1 = torch.empty_like(c2)
    pkg.check(pkg.lib().tfcc_rocm_lstm_step_f32(None, batch, hidden, tih.data_ptr(), inter.data_ptr(), xw.data_ptr(),
                                                dbias.data_ptr(), 0.0, tic.data_ptr(), h1.data_ptr(), c1.data_ptr()))
    assert np.allclose(T.n(h1), T.n(h2), rtol=1e-4, atol=1e-5) and np.allclose(T.n(c1), T.n(c2), rtol=1e-4, atol=1e-5)
    with pytest.raises(pkg.TfccRocmError):
        pkg.check(pkg.lib().tfcc_rocm_lstm_step_f32(None, 9, hidden, h.data_ptr(), inter.data_ptr(), xw.data_ptr(),
                                                    dbias.data_ptr(), 0.0, c.data_ptr(), out.data_ptr(), c.data_ptr()))


def test_gelu_and_softmax_at_the_edges_of_their_ranges(pkg, T):
    """GELU goes through a fit of erfc and softmax through the hardware's exp2 where the reference calls erff / exp:
    the oracle's values at the ends of the ranges, where an approximation would go wrong first."""
    x = np.array([0.0, -0.0, 1e-40, -1e-40, 1e-10, -1e-10, 0.5, -0.5, 1.0, -1.0, 3.0, -3.0, 5.5, -5.5, 7.0, -7.0, 7.1, -7.1,
                  10.0, -10.0, 14.0, -14.0, 100.0, -100.0, 1e30, -1e30, 3e38, -3e38, np.inf, -np.inf, np.nan],
                 dtype=np.float32)
    x = np.concatenate([x, np.linspace(-8, 8, 4001, dtype=np.float32)])
    got, want = T.n(pkg.gelu_accurate(T.t(x))), O.gelu_accurate(x)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
    assert np.allclose(got[ok], want[ok], rtol=1e-6, atol=1e-7)
    rows = np.stack([
        np.linspace(-200, 0, 128), np.linspace(0, 88, 128), np.full(128, -3e38), np.full(128, 3e38),
        np.concatenate([np.full(64, -np.inf), np.linspace(-5, 5, 64)]), np.full(128, -np.inf),
        np.concatenate([[np.nan], np.zeros(127)]), np.concatenate([[0.0], np.full(127, -104.5)]),
    ]).astype(np.float32)
    for cols in (128, 100, 300, 1500):  # one wavefront per row with the row in registers; a workgroup per long row
        r = np.ascontiguousarray(np.resize(rows, (rows.shape[0], cols))) if cols != 128 else rows
        with np.errstate(invalid="ignore", over="ignore"):
            want = O.softmax(r)
        got = T.n(pkg.softmax(T.t(r)))
        assert np.array_equal(np.isnan(got), np.isnan(want)), cols
        ok = ~np.isnan(want)
        assert np.allclose(got[ok], want[ok], rtol=2e-6, atol=1e-8), cols


def test_elementwise_against_oracle(pkg, T):
    rng = np.random.default_rng(50)
    for shape in ((8, 12, 128, 128), (7, 33), (5, 1000)):
        x = rng.normal(0, 2, shape).astype(np.float32)
        assert np.allclose(T.n(pkg.softmax(T.t(x))), O.softmax(x), rtol=2e-6, atol=1e-8)
    x = rng.normal(0, 1, (1024, 768)).astype(np.float32)
    g, b = rng.normal(1, 0.1, 768).astype(np.float32), rng.normal(0, 0.1, 768).astype(np.float32)
    assert np.allclose(T.n(pkg.layer_norm(T.t(x), T.t(g), T.t(b), 1e-12)), O.layer_norm(x, g, b, 1e-12), rtol=1e-5, atol=1e-5)
    for rows, cols in ((3, 1), (5, 255), (4, 1024), (2, 1025), (3, 3000)):  # register-resident rows and long rows
        xr = rng.normal(0.5, 2, (rows, cols)).astype(np.float32)
        gr, br = rng.normal(1, 0.1, cols).astype(np.float32), rng.normal(0, 0.1, cols).astype(np.float32)
        assert np.allclose(T.n(pkg.layer_norm(T.t(xr), T.t(gr), T.t(br), 1e-5)), O.layer_norm(xr, gr, br, 1e-5),
                           rtol=1e-5, atol=1e-5)
    for op, ref in (("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        assert np.array_equal(T.n(pkg.binary(op, T.t(x), T.t(g))), ref(x, g))
    assert np.array_equal(T.n(pkg.transform2(T.t(x), 3.0, 0.5)), x / np.float32(3.0) + np.float32(0.5))
    assert np.allclose(T.n(pkg.gelu_accurate(T.t(x))), O.gelu_accurate(x), rtol=1e-6, atol=1e-7)
    assert np.array_equal(T.n(pkg.transform(T.t(x), 0.125, 0.0)), x * np.float32(0.125))
    assert np.array_equal(T.n(pkg.add(T.t(x), T.t(g))), x + g)
    assert np.array_equal(T.n(pkg.add(T.t(x), T.t(x))), x + x)
    y = rng.normal(0, 1, (8, 128, 12, 64)).astype(np.float32)
    for perm in ((0, 2, 1, 3), (0, 1, 3, 2), (3, 2, 1, 0), (0, 2, 3, 1)):
        assert np.array_equal(T.n(pkg.transpose(T.t(y), perm)), np.transpose(y, perm))
    assert np.array_equal(T.n(pkg.transpose(T.t(x), (1, 0))), x.T)


@pytest.mark.gpu
def test_max_min_clip_relu_keep_the_reference_comparison_order(pkg, T):
    """std::max(a, b) = a < b ? b : a and std::min(a, b) = b < a ? b : a, as the reference's kernels call them
    (tfcc/mkl/interfaces/tfcc_mklminmaxinterface.cpp:37-61, tfcc_mklbasicinterface.cpp:152-153,
    tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:67-83): the first argument comes back when either is a NaN, a clip
    with its bounds the wrong way round gives the lower bound, a leaky relu with alpha > 1 gives max(v, alpha v)."""
    nan = np.float32(np.nan)

    def std_max(a, b):
        return np.where(a < b, b, a)

    def std_min(a, b):
        return np.where(b < a, b, a)

    a = np.array([1.0, nan, -2.0, 0.0, -0.0, 5.0, nan, -3.5], np.float32)
    b = np.array([nan, 2.0, -1.0, -0.0, 0.0, 4.0, nan, 7.25], np.float32)
    with np.errstate(invalid="ignore"):
        for op, ref in (("max", std_max), ("min", std_min)):
            got = T.n(pkg.binary(op, T.t(a), T.t(b)))
            want = ref(a, b)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (op, got, want)
        v = np.array([-3.0, -1.0, 0.5, 2.0, nan, 9.0], np.float32)
        for lo, hi in ((-1.0, 2.0), (2.0, -1.0)):  # the second pair: lower bound above the upper one
            want = std_max(std_min(v, np.float32(hi)), np.float32(lo))
            got = T.n(pkg.clip(T.t(v), lo, hi))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (lo, hi, got, want)
        for alpha in (0.1, 1.5, -0.5):
            want = std_max(v, np.float32(alpha) * v)
            got = T.n(pkg.leaky_relu(T.t(v), alpha))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (alpha, got, want)
        want = std_max(v, np.float32(0))
        got = T.n(pkg.unary("relu", T.t(v)))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
