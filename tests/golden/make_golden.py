"""Writes the golden fixtures of this directory from the REFERENCE's own kernels.

Runs only where oracle/_ref/libtfcc_ref.so exists (the build container, where the reference tree
is mounted and `make -C oracle` compiled its AVX2 quantized-matmul / quantization kernels with the
reference's Release flags).  The fixtures are data only: seeded inputs (or the seed that makes
them) and what the reference's kernels returned.

  qgemm_ref_vectors.npz        small ragged / batched uint8 x int8 products: inputs, offsets, int32
                               result of the reference kernel, and its AVX2 requantize to uint8
  qgemm_ref_hashes.json        SHA-256 of the reference's int32 and uint8 results for seeded inputs
                               too large to store (incl. the 4096^3 benchmark case)
  requantize_fma_cases.json    inputs on which fusing the multiply-add changes the result
                               (found by random search, see find_fma_cases)

usage: python tests/golden/make_golden.py [--fma-search N]
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as O  # noqa: E402


def gen_inputs(seed, shape_a, shape_b):
    """Seeded operands; the tests regenerate them from the seed with this same function."""
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 256, shape_a, dtype=np.uint8)
    b = rng.integers(-127, 128, shape_b, dtype=np.int8)
    return a, b


def gen_ranges(seed):
    """Float ranges like the reference's generator draws them
    (tfcc/test/python/testcase/quantization/mklquantizationmatmul.py:35-43)."""
    rng = np.random.default_rng(seed + 1000)
    a_min = np.float32(rng.uniform(-5.0, 5.0))
    a_max = np.float32(a_min + rng.uniform(0.05, 5.0))
    b_min = np.float32(rng.uniform(-5.0, 5.0))
    b_max = np.float32(b_min + rng.uniform(0.05, 5.0))
    return float(a_min), float(a_max), float(b_min), float(b_max)


SMALL_CASES = [
    # (seed, shapeA, shapeB)
    (1, (7, 5), (5, 3)),
    (2, (33, 17), (17, 1)),       # N == 1: the reference's GEMV path
    (3, (100, 64), (64, 96)),
    (4, (129, 130), (130, 131)),
    (5, (3, 50, 20), (3, 20, 30)),  # batched x batched
    (6, (4, 25, 40), (40, 24)),     # batched x matrix (batch folds into M)
    (7, (31, 48), (2, 48, 52)),     # matrix x batched
    (8, (256, 256), (256, 256)),
]

HASH_CASES = [
    # (name, seed, shapeA, shapeB, ranges or None for the benchmark ranges)
    ("c3_4096", 0, (4096, 4096), (4096, 4096), None),
    ("c3_1024_ragged", 11, (1000, 1040), (1040, 1012), None),
    ("c5_m8", 12, (8, 4096), (4096, 11008), None),
]

# the benchmark's quantization: A zero-point 128, B symmetric, levels of 1
BENCH_RANGES = (-128.0, 127.0, -128.0, 127.0)


def bench_out_range(k):
    """requantize scale 1/(K*64) with zero-point 128: one output level = K*64 accumulator units."""
    return -128.0 * k * 64.0, 127.0 * k * 64.0


def main():
    ref = O.ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libtfcc_ref.so is missing: run `make -C oracle` where the reference tree is mounted")
    out = {}
    for seed, sa, sb in SMALL_CASES:
        a, b = gen_inputs(seed, sa, sb)
        ranges = gen_ranges(seed)
        oa, ob = O.qmatmul_offsets(*ranges, lib=ref)
        c = O.qgemm(a, b, oa, ob, lib=ref)
        mn_c, mx_c = O.qmatmul_range(*ranges, lib=ref)
        # an output range (in real units) that spreads this case's accumulators over most of the
        # uint8 levels and saturates a few at both ends
        in_s, in_m = O.dequantized_scale_info(32, mn_c, mx_c)
        real = in_m + (c.astype(np.float64) + 2.0 ** 31) * in_s
        lo, hi = np.quantile(real, 0.02), np.quantile(real, 0.98)
        mn_o, mx_o = float(np.float32(lo)), float(np.float32(hi))
        q = np.empty(c.shape, np.uint8)
        ref.ref_requantize_s32_u8(np.ascontiguousarray(c).reshape(-1), c.size, mn_c, mx_c, mn_o, mx_o, 1, q.reshape(-1))
        p = "case%d/" % seed
        out[p + "a"], out[p + "b"] = a, b
        out[p + "ranges"] = np.asarray(ranges, np.float32)
        out[p + "offsets"] = np.asarray([oa, ob], np.int32)
        out[p + "c"] = c
        out[p + "out_range"] = np.asarray([mn_o, mx_o], np.float32)
        out[p + "q"] = q
        print(p, sa, sb, "offsets", oa, ob, "levels used", np.unique(q).size)
    np.savez_compressed(os.path.join(HERE, "qgemm_ref_vectors.npz"), **out)

    hashes = {}
    for name, seed, sa, sb, _ in HASH_CASES:
        a, b = gen_inputs(seed, sa, sb)
        oa, ob = O.qmatmul_offsets(*BENCH_RANGES, lib=ref)
        c = O.qgemm(a, b, oa, ob, lib=ref)
        mn_c, mx_c = O.qmatmul_range(*BENCH_RANGES, lib=ref)
        mn_o, mx_o = bench_out_range(sa[-1])
        q = np.empty(c.shape, np.uint8)
        ref.ref_requantize_s32_u8(np.ascontiguousarray(c).reshape(-1), c.size, mn_c, mx_c, mn_o, mx_o, 1, q.reshape(-1))
        hashes[name] = dict(seed=seed, shape_a=list(sa), shape_b=list(sb), ranges=list(BENCH_RANGES),
                            offsets=[oa, ob], out_range=[mn_o, mx_o],
                            sha256_c=hashlib.sha256(c.tobytes()).hexdigest(),
                            sha256_q=hashlib.sha256(q.tobytes()).hexdigest(),
                            levels_used=int(np.unique(q).size))
        print(name, hashes[name])
    json.dump(hashes, open(os.path.join(HERE, "qgemm_ref_hashes.json"), "w"), indent=1)


def find_fma_cases(n_sets, seed=11, want=4):
    """Random search for int32 -> uint8 requantize inputs on which a fused multiply-add in
    real = minIn + (x - lowest) * inScale changes the result, and what the reference's AVX2 kernel
    gives for them.  About one parameter set in 5e4 has such an input."""
    ref = O.ref()
    rng = np.random.default_rng(seed)
    j = np.arange(0, 255)
    hits = []
    for _ in range(n_sets):
        mi = float(np.float32(rng.uniform(-1, 0)))
        ma = float(np.float32(rng.uniform(2, 4)))
        mo = float(np.float32(rng.uniform(1, 2)))
        mxo = float(np.nextafter(np.float32(mo), np.float32(10)))
        in_s, in_m = O.dequantized_scale_info(32, mi, ma)
        out_s, out_o = O.quantized_scale_info(8, mo, mxo)
        real = (j + 0.5 + out_o) / out_s
        acc0 = np.round((real - in_m) / in_s - 2 ** 31).astype(np.int64)
        acc = np.unique((acc0[:, None] + np.arange(-1, 2)[None, :]).reshape(-1)).astype(np.int32)
        o0 = O.requantize_s32_u8(acc, mi, ma, mo, mxo, 0, 0)
        o1 = O.requantize_s32_u8(acc, mi, ma, mo, mxo, 0, 1)
        d = np.nonzero(o0 != o1)[0]
        if len(d):
            sel = np.ascontiguousarray(acc[d])
            r = np.empty(sel.shape, np.uint8)
            ref.ref_requantize_s32_u8(sel, sel.size, mi, ma, mo, mxo, 1, r)
            hits.append(dict(minIn=mi, maxIn=ma, minOut=mo, maxOut=mxo, acc=sel.tolist(), nofma=o0[d].tolist(),
                             fma=o1[d].tolist(), ref_avx2=r.tolist()))
            if len(hits) >= want:
                break
    return hits


if __name__ == "__main__":
    if len(sys.argv) > 2 and sys.argv[1] == "--fma-search":
        found = find_fma_cases(int(sys.argv[2]))
        print(json.dumps(found, indent=1))
    else:
        main()
