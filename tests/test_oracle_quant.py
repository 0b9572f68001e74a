"""Pins of the oracle's input producers (quantisers and the seeded generator).

Two kinds of pins: the closed-form invariants that quantize.py's arithmetic implies
(quantize.py:26-41, 53-67) with FP8 max = 448, and the reference's own outputs
(tests/golden/quantize_reference.npz, written by tests/golden/make_quantize_golden.py, which
imports quantize.py where the reference checkout exists), which fix what the invariants leave
open: the evaluation order and rounding of the scale and of the scaled values, for fp32 and for
bf16 sources.
"""
import os

import numpy as np
import pytest

import oracle


def test_a_quantiser_invariants_and_layout():
    m, k = 48, 512
    x = oracle.gen_normal_bf16(m, k, 77)
    q, s = oracle.quantize_a_1x128(x)
    assert q.shape == (k, m) and s.shape == (k // 128, m)
    deq = oracle.e4m3fn_decode(q)            # [k, m]
    g = x.reshape(m, k // 128, 128)
    amax = np.abs(g).max(-1)                 # [m, kb]
    # returned value is the inverse scale amax/448 (two fp32 roundings away at most)
    assert np.allclose(s.T, amax / 448.0, rtol=3e-7)
    # the largest element of every group maps to code 448 exactly
    assert np.all(np.abs(deq).reshape(k // 128, 128, m).max(1).T == 448.0)
    # reconstruction error within half an fp8 ulp of the scaled value (relative 2^-4) plus
    # the subnormal step
    rec = deq.T.reshape(m, k // 128, 128) * s.T[:, :, None]
    err = np.abs(rec - g)
    assert np.all(err <= np.abs(g) * 2.0 ** -4 * 1.001 + s.T[:, :, None] * 2.0 ** -10 * 1.001)
    # layout: element (m, k) at m + k*M
    assert q.reshape(-1)[5 + 130 * m] == q[130, 5]


def test_b_quantiser_invariants_partial_block():
    n, k = 200, 256                         # second n-block has 72 rows only
    x = oracle.gen_normal_bf16(n, k, 78)
    q, s = oracle.quantize_b_128x128(x)
    assert q.shape == (k, n) and s.shape == (2, 2)
    for nb in range(2):
        for kb in range(2):
            blk = x[nb * 128:min(n, nb * 128 + 128), kb * 128:kb * 128 + 128]
            assert np.isclose(s[kb, nb], np.abs(blk).max() / 448.0, rtol=3e-7)
            d = oracle.e4m3fn_decode(q[kb * 128:kb * 128 + 128, nb * 128:min(n, nb * 128 + 128)])
            assert np.abs(d).max() == 448.0
            assert np.all(np.abs(d.T * s[kb, nb] - blk) <= np.abs(blk) * 2.0 ** -4 * 1.001 + s[kb, nb] * 2.0 ** -10 * 1.001)


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantize_reference.npz")


def _bf16_round(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32).view(np.float32)


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_quantisers_reproduce_the_reference_outputs_bit_for_bit(tag):
    """quantize.py's outputs are row-major [rows, K] bytes and [rows(/128), K/128] inverse
    scales; the oracle writes the kernel layouts, i.e. their transposes (check.cu:164-167)."""
    d = np.load(GOLDEN)
    x = d["x_f32"] if tag == "f32" else _bf16_round(d["x_f32"])
    q, s = oracle.quantize_a_1x128(x, bf16_arith=(tag == "bf16"))
    assert np.array_equal(q.T, d[f"rowwise_{tag}_q"])
    assert np.array_equal(s.T.view(np.uint32), d[f"rowwise_{tag}_s"].view(np.uint32))
    q, s = oracle.quantize_b_128x128(x, bf16_arith=(tag == "bf16"))
    assert np.array_equal(q.T, d[f"block_{tag}_q"])
    assert np.array_equal(s.T.view(np.uint32), d[f"block_{tag}_s"].view(np.uint32))


def test_bf16_source_with_fp32_arithmetic_is_not_the_reference():
    """the two arithmetics differ on a few percent of the bytes: the vectors tell them apart"""
    d = np.load(GOLDEN)
    q, _ = oracle.quantize_a_1x128(_bf16_round(d["x_f32"]), bf16_arith=False)
    assert 0.001 < (q.T != d["rowwise_bf16_q"]).mean() < 0.2


def test_zero_group_gets_tiny_scale_and_zero_codes():
    x = np.zeros((2, 128), np.float32)
    x[1, 3] = 1.0
    q, s = oracle.quantize_a_1x128(x)
    assert not q[:, 0].any()
    assert s[0, 0] == np.float32(1.0) / ((np.float32(1.0) / np.float32(1e-12)) * np.float32(448.0))
    assert oracle.e4m3fn_decode(q[3:4, 1:2])[0, 0] == 448.0


def test_generator_is_seeded_order_independent_and_normal():
    x = oracle.gen_normal_bf16(64, 1000, 5)
    y = oracle.gen_normal_bf16(64, 1000, 5)
    z = oracle.gen_normal_bf16(64, 1000, 6)
    assert np.array_equal(x, y) and not np.array_equal(x, z)
    assert abs(x.mean()) < 0.02 and abs(x.std() - 1.0) < 0.02
    # values are bf16-representable
    assert np.array_equal(oracle.bf16_decode(oracle.bf16_encode(x)), x)
    # the first rows of a taller matrix with the same width are the same stream
    t = oracle.gen_normal_bf16(128, 1000, 5)
    assert np.array_equal(t[:64], x)


def test_outlier_mask_rate():
    x = oracle.gen_normal_bf16(256, 1024, 9)
    y = oracle.gen_normal_bf16(256, 1024, 9, 1.0, 50.0)
    changed = x != y
    rate = changed.mean()
    assert 0.007 < rate < 0.013
    assert np.allclose(y[changed], oracle.bf16_decode(oracle.bf16_encode(x[changed] * 50.0)), rtol=2 ** -7)


def test_config_shapes():
    for name, (m, n, k, *_rest) in oracle.CONFIGS.items():
        assert k % 128 == 0
    m, n, k, a, b, sa, sb = oracle.make_config_inputs("cfg5")
    assert (m, n, k) == (32, 7168, 2048)
    assert a.shape == (2048, 32) and b.shape == (2048, 7168) and sa.shape == (16, 32) and sb.shape == (16, 56)


def test_reference_genMat_stream():
    """utils.h:25-33 built from the reference header: seed-7 uniform(-5,5); the stream is
    compared with the committed fixture (first 4096 values) so that the fixture itself is
    known to come from the reference's generator."""
    import os
    ref = oracle.refutils()
    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "genmat_seed7_4096.npy"))
    if ref is None:
        pytest.skip("oracle/_ref not built here (reference checkout absent)")
    out = np.empty(4096, np.float32)
    ref.ref_genMat(out.ctypes.data, out.size)
    assert np.array_equal(out, fx)
    assert out.min() >= -5 and out.max() < 5
