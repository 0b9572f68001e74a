"""Pins of the oracle's GEMM (oracle_ref_gemm_naive / oracle_ref_gemm / _points).

The reference holds no golden vectors for this path (its only check is check.cu:174, one
shape, absolute tolerance 100), so the oracle is pinned by what the mathematics fixes:
exact integer block sums, numpy matmul for unit scales, one-hot inputs that isolate every
index formula, exact-rational brute force on tiny cases, linearity and permutation
invariants, and -- where it was built in this checkout -- the reference's own gemmCPU and
genMat compiled from its utils.h.
"""
from fractions import Fraction

import numpy as np
import pytest

import oracle


def _rand_inputs(m, n, k, seed, scale_lo=0.5, scale_hi=2.0):
    rng = np.random.RandomState(seed)
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    a = codes[rng.randint(0, len(codes), (k, m))]
    b = codes[rng.randint(0, len(codes), (k, n))]
    sa = rng.uniform(scale_lo, scale_hi, (k // 128, m)).astype(np.float32)
    sb = rng.uniform(scale_lo, scale_hi, (k // 128, (n + 127) // 128)).astype(np.float32)
    return a, b, sa, sb


@pytest.mark.parametrize("m,n,k", [(1, 1, 128), (5, 7, 256), (16, 200, 384), (33, 129, 256),
                                   (64, 576, 512)])
def test_fast_loop_is_bit_identical_to_naive(m, n, k):
    a, b, sa, sb = _rand_inputs(m, n, k, m + n + k)
    c0 = oracle.ref_gemm_naive(a, b, sa, sb, m, n, k)
    c1, f1 = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    assert np.array_equal(c0, c1)
    c2 = oracle.ref_gemm(a, b, sa, sb, m, n, k, nthreads=1)
    assert np.array_equal(c0, c2)
    rows, cols = np.divmod(np.arange(m * n, dtype=np.int32), n)
    f, h = oracle.ref_gemm_points(a, b, sa, sb, rows, cols, m, n, k)
    assert np.array_equal(h.reshape(m, n), c0)
    assert np.array_equal(f.reshape(m, n), f1)


def test_against_exact_integer_block_sums():
    m, n, k = 24, 150, 768
    a, b, sa, sb = oracle.make_inputs(m, n, k, 21)
    _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    exact = oracle.ref_gemm_f64(a, b, sa, sb, m, n, k)
    # independent numpy restatement of the exact value: integer products, float64 scaling
    ai = np.round(oracle.e4m3fn_decode(a).astype(np.float64) * 512).astype(np.int64)
    bi = np.round(oracle.e4m3fn_decode(b).astype(np.float64) * 512).astype(np.int64)
    want = np.zeros((m, n))
    for kb in range(k // 128):
        blk = ai[kb * 128:(kb + 1) * 128].T @ bi[kb * 128:(kb + 1) * 128]
        want += blk / 2.0 ** 18 * sa[kb][:, None].astype(np.float64) * np.repeat(sb[kb], 128)[:n][None, :]
    assert np.allclose(exact, want, rtol=1e-14, atol=0)
    # fp32 sequential accumulation error bound: 128 + K/128 roundings of ~2^-24 on sum |terms|
    assert np.max(np.abs(f - exact)) <= 2e-5 * np.max(np.abs(exact)) + 1e-6


def test_unit_scales_reduce_to_plain_matmul():
    m, n, k = 17, 130, 256
    a, b, _, _ = _rand_inputs(m, n, k, 4)
    # keep magnitudes small so that every partial sum is exact in fp32
    a &= 0xB7
    b &= 0xB7
    sa = np.ones((k // 128, m), np.float32)
    sb = np.ones((k // 128, 2), np.float32)
    _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    want = oracle.e4m3fn_decode(a).astype(np.float64).T @ oracle.e4m3fn_decode(b).astype(np.float64)
    assert np.max(np.abs(f - want)) <= 1e-6 * np.max(np.abs(want))


def test_one_hot_pins_every_index_formula():
    m, n, k = 20, 300, 384
    sn = 3
    rng = np.random.RandomState(9)
    sa = rng.uniform(1, 2, (k // 128, m)).astype(np.float32)
    sb = rng.uniform(1, 2, (k // 128, sn)).astype(np.float32)
    one = 0x38  # 1.0
    for (mi, ni, ki, code) in [(0, 0, 0, 0x40), (19, 299, 383, 0x44), (7, 128, 130, 0x3C),
                               (3, 255, 127, 0x48), (11, 256, 256, 0xC0)]:
        a = np.zeros((k, m), np.uint8)
        b = np.zeros((k, n), np.uint8)
        a.reshape(-1)[mi + ki * m] = code        # a element (m,k) lives at m + k*M
        b.reshape(-1)[ni + ki * n] = one         # b element (n,k) lives at n + k*N
        _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
        val = float(oracle.e4m3fn_decode(np.array([code], np.uint8))[0])
        want = np.float32(np.float32(val * sa.reshape(-1)[mi + (ki // 128) * m]) *
                          sb.reshape(-1)[ni // 128 + (ki // 128) * sn])
        assert f[mi, ni] == want
        f[mi, ni] = 0
        assert not f.any()
        cn = oracle.ref_gemm_naive(a, b, sa, sb, m, n, k)
        assert cn.reshape(-1)[mi * n + ni] == oracle.bf16_encode(np.array([want]))[0]


def test_tiny_brute_force_with_fractions():
    m, n, k = 3, 4, 256
    a, b, sa, sb = _rand_inputs(m, n, k, 12)
    a &= 0xAF  # small exponents: every fp32 partial sum stays exact, so order cannot matter
    b &= 0xAF
    sa = (2.0 ** np.random.RandomState(1).randint(-3, 4, sa.shape)).astype(np.float32)
    sb = (2.0 ** np.random.RandomState(2).randint(-3, 4, sb.shape)).astype(np.float32)
    _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    da, db = oracle.e4m3fn_decode(a), oracle.e4m3fn_decode(b)
    for i in range(m):
        for j in range(n):
            tot = Fraction(0)
            for kk in range(k):
                tot += Fraction(float(da[kk, i])) * Fraction(float(db[kk, j])) * \
                    Fraction(float(sa[kk // 128, i])) * Fraction(float(sb[kk // 128, j // 128]))
            assert Fraction(float(f[i, j])) == tot


def test_linearity_in_one_a_scale():
    m, n, k = 8, 140, 384
    a, b, sa, sb = oracle.make_inputs(m, n, k, 33)
    base = oracle.ref_gemm_f64(a, b, sa, sb, m, n, k)
    sa2 = sa.copy()
    sa2[1, 5] *= 2
    doubled = oracle.ref_gemm_f64(a, b, sa2, sb, m, n, k)
    # only row 5 changes, by exactly the contribution of K block 1
    sa_only = np.zeros_like(sa)
    sa_only[1, 5] = sa[1, 5]
    contrib = oracle.ref_gemm_f64(a, b, sa_only, sb, m, n, k)
    assert np.allclose(doubled - base, contrib, rtol=1e-12, atol=1e-12)
    assert not (doubled - base)[np.arange(m) != 5].any()


def test_permuting_k_inside_a_block_keeps_the_exact_result():
    m, n, k = 6, 130, 256
    a, b, sa, sb = oracle.make_inputs(m, n, k, 44)
    perm = np.concatenate([np.random.RandomState(0).permutation(128), 128 + np.random.RandomState(1).permutation(128)])
    x = oracle.ref_gemm_f64(a, b, sa, sb, m, n, k)
    y = oracle.ref_gemm_f64(np.ascontiguousarray(a[perm]), np.ascontiguousarray(b[perm]), sa, sb, m, n, k)
    assert np.array_equal(x, y)


def test_n576_equals_first_columns_of_zero_padded_n640():
    m, k = 32, 256
    a, b, sa, sb = oracle.make_inputs(m, 576, k, 55)
    c = oracle.ref_gemm(a, b, sa, sb, m, 576, k)
    bp = np.zeros((k, 640), np.uint8)
    bp[:, :576] = b
    cp = oracle.ref_gemm(a, bp, sa, sb, m, 640, k)
    assert np.array_equal(c, cp[:, :576])


def test_reference_gemmCPU_single_block():
    """With unit scales and K = 128 the block-scaled GEMM is the reference's gemmCPU
    (utils.h:65-76) term for term: identical fp32 sequence, so identical bits."""
    ref = oracle.refutils()
    if ref is None:
        pytest.skip("oracle/_ref not built here (reference checkout absent)")
    m, n, k = 9, 70, 128
    a, b, _, _ = _rand_inputs(m, n, k, 6)
    sa = np.ones((1, m), np.float32)
    sb = np.ones((1, 1), np.float32)
    _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    A = np.ascontiguousarray(oracle.e4m3fn_decode(a).T)  # M x K row-major
    B = oracle.e4m3fn_decode(b)                          # K x N row-major
    C = np.empty((m, n), np.float32)
    ref.ref_gemmCPU(C.ctypes.data, A.ctypes.data, B.ctypes.data, m, n, k)
    assert np.array_equal(C, f)


def test_reference_gemmCPU_multi_block_close():
    ref = oracle.refutils()
    if ref is None:
        pytest.skip("oracle/_ref not built here (reference checkout absent)")
    m, n, k = 5, 40, 512
    a, b, _, _ = _rand_inputs(m, n, k, 8)
    sa = np.ones((4, m), np.float32)
    sb = np.ones((4, 1), np.float32)
    _, f = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    A = np.ascontiguousarray(oracle.e4m3fn_decode(a).T)
    B = oracle.e4m3fn_decode(b)
    C = np.empty((m, n), np.float32)
    ref.ref_gemmCPU(C.ctypes.data, A.ctypes.data, B.ctypes.data, m, n, k)
    exact = A.astype(np.float64) @ B.astype(np.float64)
    # both are fp32 summations of the same exact products, only the grouping differs
    assert np.max(np.abs(C - f)) <= 2e-5 * np.max(np.abs(exact))


def test_compare_rule():
    ref = oracle.bf16_encode(np.array([100.0, -50.0, 0.0, 1.0], np.float32))
    ok = oracle.bf16_encode(np.array([100.5, -50.5, 0.5, 1.0], np.float32))
    bad = oracle.bf16_encode(np.array([100.0, -50.0, 2.0, 1.0], np.float32))
    assert oracle.compare_bf16(ok, ref)["bad"] == 0          # bound = 1e-2*100 + 1e-3
    r = oracle.compare_bf16(bad, ref)
    assert r["bad"] == 1 and abs(r["bound"] - 1.001) < 1e-9
    nanv = ref.copy()
    nanv[1] = 0x7FC0
    assert oracle.compare_bf16(nanv, ref)["bad"] == 1
