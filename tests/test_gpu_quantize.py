"""GPU parity of the device-side quantisers against the CPU oracle, through the C ABI.

Bar: bit-exact.  fp8 bytes and fp32 scales are the results of a handful of IEEE fp32
operations (max, a reciprocal, two multiplications, a clamp, one rounding to e4m3fn, a
reciprocal; with a bf16 source a rounding to bf16 after each) that are the same on both sides,
so every byte and every scale bit must agree -- with the oracle, and with the reference's own
quantize.py outputs held in tests/golden/quantize_reference.npz.
"""
import sys

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _bf16_bits(x):
    """fp32 array holding bf16-representable values -> their bf16 bit patterns"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    assert not (u & 0xFFFF).any()
    return (u >> 16).astype(np.uint16)


def _quantize_gpu(pkg, x, which, dtype):
    import torch
    rows, k = x.shape
    src = np.ascontiguousarray(x, np.float32) if dtype == pkg.DTYPE_F32 else _bf16_bits(x).view(np.int16)
    dx = torch.from_numpy(src).cuda()
    dq = torch.full((k, rows), 0x7F, dtype=torch.uint8, device="cuda")          # NaN code sentinel
    ncol = rows if which == "a" else (rows + 127) // 128
    ds = torch.full((k // 128, ncol), float("nan"), dtype=torch.float32, device="cuda")
    _say(f"[gpu case] quantize_{which} rows={rows} k={k} dtype={dtype}")
    fn = pkg.quantize_a_1x128 if which == "a" else pkg.quantize_b_128x128
    fn(dx, dq, ds, rows, k, dtype, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dq.cpu().numpy(), ds.cpu().numpy()


def _check(pkg, x, which, dtype):
    q, s = _quantize_gpu(pkg, x, which, dtype)
    rq, rs = (oracle.quantize_a_1x128 if which == "a" else oracle.quantize_b_128x128)(
        x, bf16_arith=(dtype == pkg.DTYPE_BF16))
    assert np.array_equal(s.view(np.uint32), rs.view(np.uint32)), (which, x.shape, "scales differ")
    bad = np.argwhere(q != rq)
    assert bad.size == 0, (which, x.shape, bad[:4], q[tuple(bad[0])], rq[tuple(bad[0])])


# (row counts off the 16-byte grid leave through dword stores shifted into place: odd, 2 mod 4, 0 mod 4;
# 20001 x 2048 is past the tile count up to which the 1 x 128 quantiser works in 64-row tiles)
SHAPES_A = [(32, 2048), (1024, 2048), (2048, 7168), (16, 128), (1, 128), (130, 256), (77, 384),
            (200, 128), (1001, 512), (259, 256), (3, 256), (20001, 2048), (16384, 2560)]
SHAPES_B = [(512, 2048), (576, 7168), (7168, 2048), (128, 128), (64, 128), (1, 256), (130, 256),
            (300, 384)]


@pytest.mark.parametrize("rows,k", SHAPES_A)
def test_quantize_a_bf16_matches_oracle(pkg, rows, k):
    x = oracle.gen_normal_bf16(rows, k, 31 + rows + k, 1.0, 50.0)
    _check(pkg, x, "a", pkg.DTYPE_BF16)
    _check(pkg, x, "a", pkg.DTYPE_BF16_F32MATH)


@pytest.mark.parametrize("rows,k", SHAPES_B)
def test_quantize_b_bf16_matches_oracle(pkg, rows, k):
    x = oracle.gen_normal_bf16(rows, k, 57 + rows + k)
    _check(pkg, x, "b", pkg.DTYPE_BF16)
    _check(pkg, x, "b", pkg.DTYPE_BF16_F32MATH)


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_quantize_reproduces_the_reference_outputs(pkg, tag):
    """the reference's own quantize.py outputs (tests/golden/quantize_reference.npz), bit for bit"""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantize_reference.npz"))
    x = d["x_f32"]
    if tag == "bf16":
        u = x.view(np.uint32)
        x = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32).view(np.float32)
    dtype = pkg.DTYPE_F32 if tag == "f32" else pkg.DTYPE_BF16
    q, s = _quantize_gpu(pkg, x, "a", dtype)
    assert np.array_equal(q.T, d[f"rowwise_{tag}_q"])
    assert np.array_equal(s.T.view(np.uint32), d[f"rowwise_{tag}_s"].view(np.uint32))
    q, s = _quantize_gpu(pkg, x, "b", dtype)
    assert np.array_equal(q.T, d[f"block_{tag}_q"])
    assert np.array_equal(s.T.view(np.uint32), d[f"block_{tag}_s"].view(np.uint32))


@pytest.mark.parametrize("which,rows,k", [("a", 256, 512), ("a", 48, 256), ("b", 256, 512),
                                           ("b", 200, 256)])
def test_quantize_fp32_source_matches_oracle(pkg, which, rows, k):
    rs = np.random.RandomState(rows * 7 + k)
    x = (rs.standard_normal((rows, k)) * np.exp(rs.uniform(-6, 6, (rows, 1)))).astype(np.float32)
    _check(pkg, x, which, pkg.DTYPE_F32)


def test_quantize_special_groups(pkg):
    """all-zero groups (scale = 1e-12 / 448, codes 0), a group whose amax is tiny, one with a
    huge amax, and values whose scaled magnitude rounds past 448 before the clamp"""
    rs = np.random.RandomState(5)
    x = oracle.gen_normal_bf16(256, 512, 99)
    x[3, 128:256] = 0.0
    x[128:256, 0:128] = 0.0
    x[7, 256:384] *= np.float32(2.0 ** -100)
    x[9, 0:128] *= np.float32(2.0 ** 100)
    x[11, 384:512] = np.float32(3.0)
    x[11, 385] = np.float32(-3.0)
    for which in ("a", "b"):
        _check(pkg, x, which, pkg.DTYPE_BF16)
        _check(pkg, x, which, pkg.DTYPE_BF16_F32MATH)
        _check(pkg, x * np.float32(1.0 + 2.0 ** -20), which, pkg.DTYPE_F32)
    q, s = _quantize_gpu(pkg, x, "a", pkg.DTYPE_BF16_F32MATH)
    assert (q[128:256, 3] == 0).all()
    assert s[1, 3] == np.float32(1.0) / ((np.float32(1.0) / np.float32(1e-12)) * np.float32(448.0))
    assert (q[384:512, 11] & 0x7F == 0x7E).all()          # +-448 everywhere


def test_gemm_on_device_quantised_inputs_equals_gemm_on_oracle_inputs(pkg):
    """cfg3's shape end to end on the device: quantise bf16 A and B, multiply; the fp8 bytes
    and scales equal the oracle's, so C is compared with the oracle GEMM on the oracle's
    quantised inputs under the GEMM tolerance."""
    import torch
    m, n, k = 512, 576, 1024
    xa = oracle.gen_normal_bf16(m, k, 4001)
    xb = oracle.gen_normal_bf16(n, k, 4002)
    st = torch.cuda.current_stream().cuda_stream
    dxa = torch.from_numpy(_bf16_bits(xa).view(np.int16)).cuda()
    dxb = torch.from_numpy(_bf16_bits(xb).view(np.int16)).cuda()
    da = torch.empty((k, m), dtype=torch.uint8, device="cuda")
    db = torch.empty((k, n), dtype=torch.uint8, device="cuda")
    dsa = torch.empty((k // 128, m), dtype=torch.float32, device="cuda")
    dsb = torch.empty((k // 128, (n + 127) // 128), dtype=torch.float32, device="cuda")
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    _say(f"[gpu case] quantise + gemm m={m} n={n} k={k}")
    pkg.quantize_a_1x128(dxa, da, dsa, m, k, pkg.DTYPE_BF16, st)
    pkg.quantize_b_128x128(dxb, db, dsb, n, k, pkg.DTYPE_BF16, st)
    pkg.gemm(da, db, dsa, dsb, dc, m, n, k, st)
    torch.cuda.synchronize()
    a, sa = oracle.quantize_a_1x128(xa, bf16_arith=True)
    b, sb = oracle.quantize_b_128x128(xb, bf16_arith=True)
    assert np.array_equal(da.cpu().numpy(), a) and np.array_equal(db.cpu().numpy(), b)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    r = oracle.compare_bf16(dc.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)
    assert r["bad"] == 0, r
