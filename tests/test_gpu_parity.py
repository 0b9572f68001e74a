"""GPU parity tests: every kernel family, through the C ABI, against the CPU oracle.

Bars: the scalar definition kernel and the fp32->fp8 converter are bit-exact; the MFMA
kernels satisfy max|C - ref| <= 1e-2 * max|ref| + 1e-3 (bf16 output rounding plus a
different fp32 accumulation order inside a 128-wide block).
"""
import os
import subprocess
import sys

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _dev(*arrs):
    import torch
    return [torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in arrs]


def _run(pkg, a, b, sa, sb, m, n, k, kernel=0, variant=-1, ksplit=0, scalar=False, persistent=-1, fused=-1):
    import torch
    da, db, dsa, dsb = _dev(a, b, sa, sb)
    dc = torch.full((m, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)  # NaN sentinel
    _say(f"[gpu case] m={m} n={n} k={k} kernel={kernel} variant={variant} ksplit={ksplit} scalar={scalar} "
         f"persistent={persistent} fused={fused}")
    pkg.select(kernel)
    pkg.force_config(variant, ksplit)
    pkg.set_persistent(persistent)
    pkg.set_fused_reduction(fused)
    try:
        if scalar:
            pkg.gemm_scalar(da, db, dsa, dsb, dc, m, n, k)
        else:
            pkg.gemm(da, db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        name = pkg.last_kernel()
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
        pkg.set_persistent(-1)
        pkg.set_fused_reduction(-1)
    return dc.cpu().numpy().view(np.uint16), name


def _assert_close(got, ref, what):
    r = oracle.compare_bf16(got, ref, RTOL, ATOL)
    assert r["bad"] == 0, (what, r)
    return r


def _assert_every_element(got, a, b, sa, sb, m, n, k, what):
    """A bound per element, tight enough to see one lost or doubled K block anywhere:

        |C - ref| <= 2^-7 |ref| + 2^-12 S,   S = sum over K blocks of scale * sum |a| |b|

    ref = the oracle's fp32 value before its bf16 cast.  2^-7 |ref| = one bf16 ulp (the output
    rounding, and a neighbouring code when the two fp32 sums straddle a rounding boundary);
    2^-12 S bounds what a different summation order inside the blocks can move, also where the
    terms cancel (the oracle's sequential fp32 sum and the matrix unit's accumulation each stay
    within about 2^-16 S of the exact sum; with 1 % of the entries fifty times larger the measured
    worst case is 2^-13.7 S).  One missing K block of 56 moves a typical element by 2.5e-3 S
    against a bound of about 4e-4 S."""
    _, ref32 = oracle.ref_gemm(a, b, sa, sb, m, n, k, want_f32=True)
    _, s32 = oracle.ref_gemm(a & 0x7F, b & 0x7F, np.abs(sa), np.abs(sb), m, n, k, want_f32=True)
    c = oracle.bf16_decode(got).astype(np.float64).reshape(m, n)
    err = np.abs(c - ref32.astype(np.float64))
    bound = 2.0 ** -7 * np.abs(ref32.astype(np.float64)) + 2.0 ** -12 * s32.astype(np.float64)
    ratio = err / np.maximum(bound, 1e-30)
    worst = np.unravel_index(np.argmax(ratio), ratio.shape)
    _say(f"[gpu case] {what}: per-element bound, worst err/bound = {ratio[worst]:.3f} at {worst}")
    assert np.isfinite(c).all(), what
    assert (err <= bound).all(), (what, worst, float(err[worst]), float(bound[worst]))


# ------------------------------------------------------------------ scalar definition kernel
@pytest.mark.parametrize("m,n,k", [(1, 1, 128), (48, 80, 128), (64, 128, 256), (33, 130, 384),
                                   (128, 128, 256)])
def test_scalar_kernel_is_bit_exact(pkg, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 100 + m)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, scalar=True)
    assert name == "scalar"
    assert np.array_equal(got, ref)


def test_scalar_kernel_golden_fixture(pkg):
    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_case.npz"))
    m, n, k = [int(v) for v in fx["shape"]]
    got, _ = _run(pkg, fx["a"], fx["b"], fx["a_scale"], fx["b_scale"], m, n, k, scalar=True)
    assert np.array_equal(got, fx["c"])
    got2, name = _run(pkg, fx["a"], fx["b"], fx["a_scale"], fx["b_scale"], m, n, k)
    _assert_close(got2, fx["c"], name)


# ------------------------------------------------------------------ MFMA tile kernels
SHAPES = [(256, 256, 128), (256, 256, 256), (512, 768, 512), (272, 576, 384), (128, 128, 256),
          (16, 16, 128), (1024, 192, 640), (304, 1040, 256), (64, 2048, 1024)]


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_tile_kernel(pkg, variant, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, m * 7 + n + variant, 1.0, 50.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=variant)
    assert name.endswith("_k1"), name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)


# persistent form: several tiles per workgroup (more than 256 tiles), ragged edges, K ranges from
# the shortest the ring allows to many blocks, and a launch with fewer tiles than workgroups
@pytest.mark.parametrize("variant,m,n,k", [(0, 4096, 3456, 512), (0, 1040, 1232, 256), (0, 4112, 3472, 128),
                                           (1, 4096, 2176, 384), (1, 4368, 2064, 256),
                                           (2, 4096, 4096, 384), (2, 2304, 2320, 1024),
                                           (3, 2064, 4032, 640), (3, 2048, 6528, 256)])
def test_tile_kernel_persistent(pkg, variant, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, m + 3 * n + k + variant, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=variant, persistent=1)
    assert name.endswith("_k1_persistent"), name
    _assert_close(got, ref, name)
    plain, name0 = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=variant, persistent=0)
    assert name0.endswith("_k1"), name0
    assert np.array_equal(got, plain), "persistent and plain tile kernels fold the same sums in the same order"


# one-wave-per-SIMD form of the 256 x 192 tile (variant 5, persistent only; its K loop is an assembly
# loop): one tile, fewer tiles than workgroups, several tiles per workgroup, one and two K blocks
# (the copy stream changes tile in every call of the loop), ragged edges in both directions, and a
# column count that makes a wave's 96 columns straddle two b_scale blocks in every alignment
W4_SHAPES = [(256, 192, 128), (512, 384, 256), (1040, 1232, 384), (4096, 3456, 512), (4112, 3472, 128),
             (2048, 2304, 1024), (8192, 4608, 896), (4400, 3280, 256)]


@pytest.mark.parametrize("m,n,k", W4_SHAPES)
def test_tile_kernel_one_wave_per_simd(pkg, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 5 * m + n + k, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=5)
    assert name == "tile256x192w4_k1_persistent", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    plain, name0 = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=0, persistent=0)
    assert name0 == "tile256x192_k1", name0
    assert np.array_equal(got, plain), "both forms fold the same block sums in the same order"
    again, _ = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=5)
    assert np.array_equal(got, again), "run-to-run reproducible"


# the last three: more tiles x splits than CUs (several rounds of workgroups meet in the mailbox), a tile
# count that is not a multiple of 8 with ragged edges, many splits of many small tiles
@pytest.mark.parametrize("m,n,k", [(250, 300, 512), (1000, 200, 256), (4000, 3000, 128), (272, 192, 128)])
def test_tile_kernel_one_wave_per_simd_off_the_grid(pkg, m, n, k):
    """the generated K loop on padded copies (leading dimension of A and a_scale above m, C written in
    place), on a last row tile that is partly empty and on a single K block"""
    a, b, sa, sb = oracle.make_inputs(m, n, k, 7 * m + n + k, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_AUTO, variant=5)
    assert name.endswith("tile256x192w4_k1_persistent") and name.startswith("padded_") == (m % 16 != 0 or n % 16 != 0), name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    plain, name0 = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_AUTO, variant=0, ksplit=1, persistent=0)
    assert name0.endswith("tile256x192_k1"), name0
    assert np.array_equal(got, plain), "both forms fold the same block sums in the same order"
    pkg.release()


@pytest.mark.parametrize("m,n,k", W4_SHAPES + [(256, 256, 128), (4096, 4096, 256), (272, 528, 640)])
def test_tile_kernel_256x256(pkg, m, n, k):
    """the 256 x 256 tile (64 x 128 per wave; persistent form only): same block sums, same fold order"""
    a, b, sa, sb = oracle.make_inputs(m, n, k, 6 * m + n + k, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=6)
    assert name == "tile256x256_k1_persistent", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    plain, name0 = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=0, persistent=0)
    assert name0 == "tile256x192_k1", name0
    assert np.array_equal(got, plain), "both tiles fold the same block sums in the same order"


@pytest.mark.parametrize("variant,ksplit,m,n,k", [(2, 2, 256, 256, 512), (2, 4, 512, 512, 1024),
                                                   (1, 3, 272, 576, 896), (0, 8, 256, 576, 2048),
                                                   (2, 7, 128, 640, 7168), (1, 16, 256, 128, 2048), (3, 5, 384, 576, 1280),
                                                   (4, 3, 208, 336, 768), (4, 2, 64, 64, 256),
                                                   (2, 3, 2048, 576, 1536), (4, 4, 1008, 528, 1024), (4, 8, 512, 512, 2048)])
def test_tile_kernel_split_k(pkg, variant, ksplit, m, n, k):
    """the K range split over workgroups: partial tiles added by the reduction kernel (fused=0) and by the
    last workgroup of each tile inside the GEMM kernel (fused=1) -- same sums in the same order"""
    a, b, sa, sb = oracle.make_inputs(m, n, k, m + n + k + ksplit)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SPLITK, variant=variant, ksplit=ksplit, fused=0)
    assert name.endswith(f"_k{ksplit}"), name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)   # a partial tile dropped by one split shows here
    for rep in range(3):
        inside, fname = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SPLITK, variant=variant, ksplit=ksplit,
                             fused=1)
        assert fname == name + "f", fname
        assert np.array_equal(got, inside), f"{fname} run {rep}: differs from the reduction kernel's result"


@pytest.mark.parametrize("m,n,k", [(32, 7168, 2048), (16, 96, 512), (32, 576, 7168), (32, 32, 128),
                                   (16, 1040, 384), (32, 4096, 256)])
def test_skinny_kernel(pkg, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 900 + n)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=0)   # 0 = the narrow strips
    assert name.startswith("skinny")
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)


@pytest.mark.parametrize("m,n,k,ksplit", [(32, 1536, 7168, 4), (16, 1040, 2048, 2), (32, 576, 7168, 7),
                                          (32, 96, 1024, 8), (16, 4608, 1536, 3)])
def test_skinny_kernel_with_the_k_range_split_over_workgroups(pkg, m, n, k, ksplit):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 950 + n + ksplit)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=0, ksplit=ksplit)
    assert name == f"skinny_k{ksplit}", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)


# wide strips (128 columns), the K splits of a strip added inside the kernel by the waves of its last split:
# every K split count the kernel takes, one and two row tiles, a ragged last strip (n % 128 != 0), more
# strips x splits than CUs (several rounds of workgroups), a single K block per split
DECODE_STRIP_CASES = [(32, 7168, 2048, 4), (16, 7168, 2048, 4), (32, 7168, 2048, 1), (32, 576, 1024, 3),
                      (32, 1040, 2048, 16), (16, 96, 512, 2), (32, 128, 128, 1), (32, 4608, 7168, 7),
                      (16, 1536, 1536, 12), (32, 2048, 384, 3), (32, 16384, 1024, 4), (16, 16, 2048, 6),
                      (32, 7168, 7168, 8),
                      # more strips than the device holds workgroups, no K split: the streaming form (a workgroup
                      # walks through several strips, one copy stream); ragged last strip; a single K block
                      (16, 33040, 384, 1), (32, 40960, 256, 1), (48, 33024, 128, 1),
                      # wide enough for 256-column strips on every CU: full strips, a last strip that ends in its
                      # first half, one that ends in its second, one to four row tiles
                      (32, 65536, 256, 1), (16, 65616, 384, 1), (64, 65744, 128, 1), (48, 66000, 256, 1)]


@pytest.mark.parametrize("m,n,k,ksplit", DECODE_STRIP_CASES)
def test_decode_strip_kernel(pkg, m, n, k, ksplit):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1200 + n + k + ksplit, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ksplit)
    assert name == f"decode128_k{ksplit}", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    # the sum runs in split order whatever the timing, and the mailbox is zero again after every launch
    for rep in range(4):
        again, _ = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ksplit)
        assert np.array_equal(got, again), f"run {rep}: not reproducible"


# row counts off the 16-byte grid: the kernel copies A's K blocks as the packed slabs they are and spreads them
# into padded rows in the LDS (no padded copy of A, no extra launch): one to 63 rows, one and two row tiles and
# the four-row-tile form, split and unsplit, a ragged last strip, a single K block, more K blocks than ring slots
DECODE_RAGGED_CASES = [(1, 7168, 2048, 4), (7, 7168, 2048, 4), (8, 7168, 2048, 1), (3, 576, 1024, 3),
                       (13, 1040, 2048, 16), (2, 96, 512, 2), (5, 128, 128, 1), (31, 4608, 7168, 7),
                       (17, 1536, 1536, 12), (15, 2048, 384, 3), (24, 16384, 1024, 4), (9, 16, 2048, 1),
                       (33, 7168, 2048, 4), (47, 1536, 1536, 3), (63, 2064, 7168, 8), (50, 256, 128, 1),
                       (4, 33040, 384, 1), (36, 512, 3584, 1)]


@pytest.mark.parametrize("m,n,k,ksplit", DECODE_RAGGED_CASES)
def test_decode_strip_kernel_with_rows_off_the_grid(pkg, m, n, k, ksplit):
    import torch
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1250 + m + n + k + ksplit, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ksplit)
    assert name == f"decode128_k{ksplit}", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    # bit-identical to the same problem on zero-padded copies with rows on the grid, and nothing written past row m
    m16 = (m + 15) // 16 * 16
    ap = np.zeros((k, m16), np.uint8)
    ap[:, :m] = a.reshape(k, m)
    sap = np.zeros((k // 128, m16), np.float32)
    sap[:, :m] = sa.reshape(k // 128, m)
    padded, pname = _run(pkg, ap.reshape(-1), b, sap.reshape(-1), sb, m16, n, k, kernel=pkg.KERNEL_SKINNY, variant=1,
                         ksplit=ksplit)
    assert pname == name
    assert np.array_equal(got.reshape(m, n), padded.reshape(m16, n)[:m]), "differs from the padded problem"
    da, db, dsa, dsb = _dev(a, b, sa, sb)
    dc = torch.full((m16 + 16, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)
    pkg.select(pkg.KERNEL_SKINNY)
    pkg.force_config(1, ksplit)
    try:
        pkg.gemm(da, db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
    out = dc.cpu().numpy().view(np.uint16)
    assert np.array_equal(out[:m].reshape(-1), got.reshape(-1))
    assert (out[m:] == 0x7FC1).all(), "rows past m were written"


def test_decode_rows_off_the_grid_run_without_a_padded_copy(pkg):
    """automatic dispatch: a decode batch of seven rows takes the decode kernel directly; with A off a 16-byte
    boundary it takes the padded plan as before"""
    import torch
    m, n, k = 7, 7168, 2048
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1288, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k)
    assert name.startswith("decode128_k"), name
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    da, db, dsa, dsb = _dev(a, b, sa, sb)
    shifted = torch.zeros(a.size + 16, dtype=torch.uint8, device="cuda")
    shifted[4:4 + a.size] = da.view(torch.uint8).reshape(-1)
    dc = torch.full((m, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)
    pkg.gemm(shifted[4:4 + a.size], db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert pkg.last_kernel().startswith("padded_decode128_k"), pkg.last_kernel()
    assert np.array_equal(dc.cpu().numpy().view(np.uint16).reshape(-1), got.reshape(-1))


# 256-column strips (tile_variant 2 of the decode family): two 128-column halves per stage, their own b_scale
# each; strips whose last one ends in its first half / in its second; every row-tile count, rows on and off the
# 16-byte grid; split and unsplit; results bit-identical to the 128-column strips with the same K split
# rows on the 16-byte grid with 28 or more K blocks per workgroup run in the instances that spread A's packed slabs
DECODE_LONG_K_CASES = [(16, 2048, 4096, 1), (32, 1536, 7168, 2), (48, 640, 3584, 1), (64, 1024, 7168, 2), (32, 256, 8192, 2)]


@pytest.mark.parametrize("m,n,k,ksplit", DECODE_LONG_K_CASES)
def test_decode_rows_on_the_grid_with_a_long_k_range_per_workgroup(pkg, m, n, k, ksplit):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1370 + m + n + k + ksplit, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ksplit)
    assert name == f"decode128_k{ksplit}", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    # the same K split with fewer K blocks per workgroup is not available; the 256-column strips (plain instances
    # at any K range) give the same bits
    wide, wname = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=2, ksplit=ksplit)
    assert wname == f"decode256_k{ksplit}", wname
    assert np.array_equal(got, wide), "slab-spreading instance and plain 256-column instance differ"


DECODE_WIDE_STRIP_CASES = [(32, 7168, 2048, 4), (16, 7168, 2048, 1), (32, 576, 1024, 3), (32, 1200, 2048, 16),
                           (7, 4608, 7168, 6), (40, 2064, 7168, 8), (63, 256, 128, 1), (1, 18432, 1024, 2),
                           (24, 16384, 1024, 4), (48, 7168, 2048, 2), (64, 112, 512, 2), (33, 18432, 384, 3)]


@pytest.mark.parametrize("m,n,k,ksplit", DECODE_WIDE_STRIP_CASES)
def test_decode_kernel_with_256_column_strips(pkg, m, n, k, ksplit):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1270 + m + n + k + ksplit, 0.5, 30.0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=2, ksplit=ksplit)
    assert name == f"decode256_k{ksplit}", name
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)
    narrow, nname = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ksplit)
    assert nname == f"decode128_k{ksplit}", nname
    assert np.array_equal(got, narrow), "differs from the 128-column strips"
    for rep in range(3):
        again, _ = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=2, ksplit=ksplit)
        assert np.array_equal(got, again), f"run {rep}: not reproducible"


def test_decode_strip_split_that_outgrows_the_mailbox_is_refused(pkg):
    """128 strips x 15 sending splits x 16 KiB of patches do not fit the 16 MiB mailbox: no such plan"""
    m, n, k = 32, 16384, 2048
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1290)
    with pytest.raises(pkg.Fp8GemmError) as info:
        _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=16)
    assert info.value.code == -3


def test_decode_strip_mailbox_survives_a_change_of_shape(pkg):
    """launches of different strip and split counts back to back share the mailbox"""
    import torch
    st = torch.cuda.current_stream().cuda_stream
    cases = [(32, 7168, 2048, 4), (16, 1536, 1024, 8), (32, 7168, 2048, 2), (32, 640, 4096, 16), (32, 7168, 2048, 4)]
    prepared = []
    for (m, n, k, ks) in cases:
        a, b, sa, sb = oracle.make_inputs(m, n, k, 1300 + n + ks)
        prepared.append((oracle.ref_gemm(a, b, sa, sb, m, n, k), _dev(a, b, sa, sb),
                         torch.full((m, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)))
    _say(f"[gpu case] decode strips, shapes back to back without a synchronisation: {cases}")
    pkg.select(pkg.KERNEL_SKINNY)
    try:
        for rep in range(3):
            for (m, n, k, ks), (_, dev, dc) in zip(cases, prepared):
                pkg.force_config(1, ks)
                pkg.gemm(dev[0], dev[1], dev[2], dev[3], dc, m, n, k, st)
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
    torch.cuda.synchronize()
    for (m, n, k, ks), (ref, _, dc) in zip(cases, prepared):
        _assert_close(dc.cpu().numpy().view(np.uint16), ref, f"decode128_k{ks} {m}x{n}x{k}")


def test_decode_strips_in_a_caller_workspace_need_its_zeroed_flag(pkg):
    """fp8_block_gemm_ex: the in-kernel reduction keeps its hand-over state (the
    mailbox) in the header of the workspace, so a per-call workspace gets it only when the caller vouches for
    a zeroed header; without the flag the call takes a plan that needs none"""
    import torch
    m, n, k = 32, 7168, 2048
    a, b, sa, sb = oracle.make_inputs(m, n, k, 1400)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    dev = _dev(a, b, sa, sb)
    st = torch.cuda.current_stream().cuda_stream
    need = pkg.workspace_bytes_ex(m, n, k)
    assert need == pkg.WORKSPACE_HEADER_BYTES
    ws = torch.full((need,), 0xAB, dtype=torch.uint8, device="cuda")          # garbage, also in the header
    dc = torch.full((m, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)
    _say(f"[gpu case] decode in a caller workspace without / with the zeroed flag m={m} n={n} k={k}")
    pkg.gemm_ex(dev[0], dev[1], dev[2], dev[3], dc, m, n, k, None, ws, need, st)
    torch.cuda.synchronize()
    assert not pkg.last_kernel().startswith("decode128_k4"), pkg.last_kernel()
    _assert_close(dc.cpu().numpy().view(np.uint16), ref, pkg.last_kernel())
    ws[:pkg.WORKSPACE_HEADER_BYTES] = 0
    dc.fill_(0x7FC1)
    opt = pkg.Options(flags=pkg.FLAG_WORKSPACE_ZEROED)
    for rep in range(3):
        pkg.gemm_ex(dev[0], dev[1], dev[2], dev[3], dc, m, n, k, opt, ws, need, st)
    torch.cuda.synchronize()
    assert pkg.last_kernel() == "decode128_k4", pkg.last_kernel()
    _assert_close(dc.cpu().numpy().view(np.uint16), ref, "decode128_k4 in a caller workspace")
    assert int(ws[:pkg.WORKSPACE_HEADER_BYTES].to(torch.int32).sum().item()) == 0, "header not back to zero"


@pytest.mark.parametrize("m,n,k", [(32, 7168, 7168), (16, 4608, 7168), (32, 1536, 7168), (32, 7168, 4096),
                                   (48, 1536, 4096), (64, 7168, 2048)])
def test_decode_shapes_under_automatic_dispatch(pkg, m, n, k):
    """what the dispatcher picks for small M (decode kernel, its K split, or 64x64 tiles with a K split)"""
    a, b, sa, sb = oracle.make_inputs(m, n, k, 990 + m + n // 7)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k)
    _assert_close(got, ref, name)
    _assert_every_element(got, a, b, sa, sb, m, n, k, name)


@pytest.mark.parametrize("m,n,k", [(33, 100, 128), (17, 129, 256), (100, 100, 384)])
def test_scalar_kernel_takes_unaligned_shapes(pkg, m, n, k):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 5 + m)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SCALAR)
    assert name == "scalar"
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("m,n,k", [(33, 100, 128), (17, 129, 256), (100, 100, 384), (1, 1, 128), (1, 7, 256),
                                   (5, 1, 128), (250, 300, 512), (1000, 777, 1024), (33, 4100, 1024),
                                   (2049, 2049, 256), (17, 129, 8192), (8, 8200, 2048), (4100, 24, 1280),
                                   (255, 257, 384), (1022, 510, 640), (130, 4607, 256)])
def test_unaligned_shapes_run_on_padded_copies(pkg, m, n, k):
    """m or n not a multiple of 16: the MFMA kernels run on zero-padded copies in the workspace
    and C's m x n corner is copied out"""
    a, b, sa, sb = oracle.make_inputs(m, n, k, 77 + m)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k)
    assert name.startswith("padded_"), name
    _assert_close(got, ref, name)
    assert pkg.plan(m, n, k) == name
    assert pkg.workspace_bytes(m, n, k) >= ((m + 15) // 16 * 16) * ((n + 15) // 16 * 16) * 2
    pkg.release()


def test_misaligned_operand_addresses_run_on_padded_copies(pkg):
    """multiples of 16 everywhere, but a, a_scale and c start 4 or 8 bytes off a 16-byte boundary"""
    import torch
    m, n, k = 512, 384, 1024
    a, b, sa, sb = oracle.make_inputs(m, n, k, 78)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    da = torch.zeros(k * m + 16, dtype=torch.uint8, device="cuda")[8:8 + k * m]
    da.copy_(torch.from_numpy(a).reshape(-1))
    dsa = torch.zeros(sa.size + 4, dtype=torch.float32, device="cuda")[1:1 + sa.size]
    dsa.copy_(torch.from_numpy(sa).reshape(-1))
    dc = torch.full((m * n + 8,), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16)[2:2 + m * n]
    db, dsb = torch.from_numpy(b).cuda(), torch.from_numpy(sb).cuda()
    assert da.data_ptr() % 16 == 8 and dsa.data_ptr() % 16 == 4 and dc.data_ptr() % 16 == 4
    _say(f"[gpu case] misaligned operands m={m} n={n} k={k}")
    pkg.gemm(da, db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    name = pkg.last_kernel()
    assert name.startswith("padded_"), name
    _assert_close(dc.cpu().numpy().view(np.uint16).reshape(m, n), ref, name)
    pkg.release()


# ------------------------------------------------------------------ the five benchmark configurations
@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
def test_benchmark_config_full_size(pkg, name):
    m, n, k, a, b, sa, sb = oracle.make_config_inputs(name)
    _say(f"[gpu case] {name}: oracle on {oracle.max_threads()} threads")
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, kname = _run(pkg, a, b, sa, sb, m, n, k)
    r = _assert_close(got, ref, f"{name} {kname}")
    _say(f"[gpu case] {name} {kname}: max_err={r['max_err']:.4g} bound={r['bound']:.4g}")
    assert kname != "scalar"
    _assert_every_element(got, a, b, sa, sb, m, n, k, f"{name} {kname}")


# the 18 shapes of the reference's results table (/root/reference/README.md:15-25), which the
# dispatcher's cost model and table were fitted on: automatic dispatch against the whole oracle result
CHALLENGE_KN = [(7168, 1536), (1536, 3072), (7168, 576), (256, 7168), (2048, 7168), (7168, 4608),
                (2304, 7168), (7168, 512), (512, 4096)]


@pytest.mark.parametrize("m", [1024, 6144])
@pytest.mark.parametrize("k,n", CHALLENGE_KN)
def test_challenge_shapes_under_automatic_dispatch(pkg, m, k, n):
    a, b, sa, sb = oracle.make_inputs(m, n, k, 9000 + m + n + k)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, kname = _run(pkg, a, b, sa, sb, m, n, k)
    assert kname == pkg.plan(m, n, k) and kname != "scalar", kname
    _assert_close(got, ref, f"{m}x{n}x{k} {kname}")
    _assert_every_element(got, a, b, sa, sb, m, n, k, f"{m}x{n}x{k} {kname}")


# ------------------------------------------------------------------ size-independent properties
def test_results_are_bitwise_reproducible(pkg):
    m, n, k = 512, 576, 2048
    a, b, sa, sb = oracle.make_inputs(m, n, k, 31)
    for kw in (dict(kernel=2, variant=0), dict(kernel=3, variant=2, ksplit=4)):
        x, _ = _run(pkg, a, b, sa, sb, m, n, k, **kw)
        y, _ = _run(pkg, a, b, sa, sb, m, n, k, **kw)
        assert np.array_equal(x, y)
    a, b, sa, sb = oracle.make_inputs(32, 1024, 2048, 32)
    for variant in (0, 1):
        x, _ = _run(pkg, a, b, sa, sb, 32, 1024, 2048, kernel=4, variant=variant)
        y, _ = _run(pkg, a, b, sa, sb, 32, 1024, 2048, kernel=4, variant=variant)
        assert np.array_equal(x, y)


def test_n576_equals_zero_padded_n640_bit_for_bit(pkg):
    m, k = 256, 1024
    a, b, sa, sb = oracle.make_inputs(m, 576, k, 77)
    bp = np.zeros((k, 640), np.uint8)
    bp[:, :576] = b
    x, _ = _run(pkg, a, b, sa, sb, m, 576, k, kernel=2, variant=2)
    y, _ = _run(pkg, a, bp, sa, sb, m, 640, k, kernel=2, variant=2)
    assert np.array_equal(x, y[:, :576])


def test_power_of_two_scale_change_scales_the_result_exactly(pkg):
    m, n, k = 256, 256, 512
    a, b, sa, sb = oracle.make_inputs(m, n, k, 88)
    x, _ = _run(pkg, a, b, sa, sb, m, n, k, kernel=2, variant=0)
    y, _ = _run(pkg, a, b, sa * 4, sb * 0.5, m, n, k, kernel=2, variant=0)
    assert np.array_equal(oracle.bf16_decode(y), oracle.bf16_decode(x) * 2)


def test_one_hot_inputs_pick_single_products(pkg):
    m, n, k = 256, 384, 384
    rng = np.random.RandomState(4)
    sa = rng.uniform(1, 2, (3, m)).astype(np.float32)
    sb = rng.uniform(1, 2, (3, 3)).astype(np.float32)
    a = np.zeros((k, m), np.uint8)
    b = np.zeros((k, n), np.uint8)
    pts = [(0, 0, 0), (255, 383, 383), (17, 129, 130), (200, 256, 127)]
    for (mi, ni, ki) in pts:
        a[ki, mi] = 0x44  # 3.0... (code 0x44 = 1.5 * 2^1)
        b[ki, ni] = 0x38  # 1.0
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    for kw in (dict(kernel=2, variant=0), dict(kernel=2, variant=2), dict(kernel=3, variant=1, ksplit=3)):
        got, _ = _run(pkg, a, b, sa, sb, m, n, k, **kw)
        assert np.array_equal(got, ref)
    assert np.count_nonzero(ref) == len(pts)


def test_nan_and_zero_scale_do_not_leak_into_other_elements(pkg):
    m, n, k = 256, 256, 256
    a, b, sa, sb = oracle.make_inputs(m, n, k, 99)
    a[5, 7] = 0x7F          # NaN in row 7
    sa[1, 9] = 0.0          # K block 1 of row 9 contributes nothing
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=2, variant=0)
    gf, rf = oracle.bf16_decode(got), oracle.bf16_decode(ref)
    assert np.isnan(gf[7]).all() and np.isnan(rf[7]).all()
    assert not np.isnan(np.delete(gf, 7, axis=0)).any()
    _assert_close(np.delete(got, 7, axis=0), np.delete(ref, 7, axis=0), name)


@pytest.mark.parametrize("m,n,k,kw", [(32, 1536, 1024, dict(kernel=4, variant=1, ksplit=4)),
                                      (64, 640, 512, dict(kernel=4, variant=1, ksplit=2)),
                                      (256, 384, 1024, dict(kernel=3, variant=4, ksplit=4, fused=1)),
                                      (256, 384, 768, dict(kernel=3, variant=2, ksplit=3, fused=1))])
def test_special_values_through_the_mailbox_plans(pkg, m, n, k, kw):
    """plans whose K splits meet in the mailbox write +0.0 as -0.0 so that no word is zero: all-zero operands
    still give +0.0 bit for bit, one-hot operands (most partial sums are zero) the exact single products, a NaN
    stays in its row, and the mailbox is zero again afterwards (the next launch is right)"""
    nkb = k // 128
    sn = (n + 127) // 128
    rng = np.random.RandomState(m + n + k)
    sa = rng.uniform(1, 2, (nkb, m)).astype(np.float32)
    sb = rng.uniform(1, 2, (nkb, sn)).astype(np.float32)
    zeros_a, zeros_b = np.zeros((k, m), np.uint8), np.zeros((k, n), np.uint8)
    got, name = _run(pkg, zeros_a, zeros_b, sa, sb, m, n, k, **kw)
    assert (got == 0).all(), f"{name}: all-zero operands must give +0.0 everywhere"
    a, b = zeros_a.copy(), zeros_b.copy()
    pts = [(0, 0, 0), (m - 1, n - 1, k - 1), (m // 2 + 1, n // 3, k // 2), (3, n - 2, 129), (m - 2, 5, k - 130)]
    for (mi, ni, ki) in pts:
        a[ki, mi] = 0x44   # 3.0
        b[ki, ni] = 0xB8   # -1.0
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, **kw)
    assert np.array_equal(got, ref), name
    assert np.count_nonzero(ref) == len(pts)
    a2, b2, sa2, sb2 = oracle.make_inputs(m, n, k, 4100 + m)
    a2[k - 3, 7] = 0x7F     # NaN in row 7, in the last split's K range
    a2[2, 11] = 0xFF        # NaN in row 11, in the first split's
    ref = oracle.ref_gemm(a2, b2, sa2, sb2, m, n, k)
    got, name = _run(pkg, a2, b2, sa2, sb2, m, n, k, **kw)
    gf = oracle.bf16_decode(got)
    assert np.isnan(gf[7]).all() and np.isnan(gf[11]).all()
    keep = np.delete(np.arange(m), [7, 11])
    assert not np.isnan(gf[keep]).any()
    _assert_close(got[keep], ref[keep], name)
    # and the launch after those finds a clean mailbox
    a3, b3, sa3, sb3 = oracle.make_inputs(m, n, k, 4200 + m)
    got, name = _run(pkg, a3, b3, sa3, sb3, m, n, k, **kw)
    _assert_close(got, oracle.ref_gemm(a3, b3, sa3, sb3, m, n, k), name)
    _assert_every_element(got, a3, b3, sa3, sb3, m, n, k, name)


def test_mailbox_plans_back_to_back_in_random_order(pkg):
    """three seconds of launches of the plans that hand their K splits over through the mailbox, shapes in random
    order and without synchronisation in between (every launch finds the zeros the one before left behind):
    every result equals that plan's first one bit for bit"""
    import time
    import torch
    st = torch.cuda.current_stream().cuda_stream
    cases = [(32, 7168, 2048, pkg.KERNEL_SKINNY, 1, 4), (16, 1536, 7168, pkg.KERNEL_SKINNY, 1, 8),
             (1024, 512, 2048, pkg.KERNEL_SPLITK, 4, 2), (2048, 576, 7168, pkg.KERNEL_SPLITK, 2, 3),
             (512, 512, 4096, pkg.KERNEL_SPLITK, 4, 4), (48, 1536, 2048, pkg.KERNEL_SKINNY, 1, 6)]
    prep = []
    pkg.set_fused_reduction(1)
    try:
        for (m, n, k, ker, v, ks) in cases:
            a, b, sa, sb = oracle.make_inputs(m, n, k, 31 + m + n + k)
            dev = _dev(a, b, sa, sb)
            c = torch.zeros((m, n), dtype=torch.int16, device="cuda")
            pkg.select(ker)
            pkg.force_config(v, ks)
            pkg.gemm(*dev, c, m, n, k, st)
            torch.cuda.synchronize()
            name = pkg.last_kernel()
            assert name.startswith("decode128_k") or name.endswith("f"), name
            _assert_close(c.cpu().numpy().view(np.uint16), oracle.ref_gemm(a, b, sa, sb, m, n, k), name)
            prep.append((m, n, k, ker, v, ks, dev, c, c.clone(), name))
        _say(f"[gpu case] mailbox plans back to back: {[p[9] for p in prep]}")
        rs = np.random.RandomState(5)
        t0 = time.time()
        launches = 0
        while time.time() - t0 < 3.0:
            outs = []
            for i in rs.permutation(len(prep)):
                m, n, k, ker, v, ks, dev, c, good, name = prep[i]
                pkg.select(ker)
                pkg.force_config(v, ks)
                for _ in range(int(rs.randint(1, 6))):
                    c.fill_(0x7FC1)
                    pkg.gemm(*dev, c, m, n, k, st)
                    launches += 1
                outs.append((i, c.clone()))
            torch.cuda.synchronize()
            for i, o in outs:
                assert torch.equal(o, prep[i][8]), f"{prep[i][9]} after {launches} launches"
        assert launches > 1000
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
        pkg.set_fused_reduction(-1)


# ------------------------------------------------------------------ converter, host launcher, workspace, drivers
def test_convert_kernel_is_bit_exact(pkg):
    import torch
    rng = np.random.RandomState(1)
    codes = np.array([c for c in range(0x7F)], np.uint8)
    vals = oracle.e4m3fn_decode(codes)
    mids = ((vals[:-1].astype(np.float64) + vals[1:]) / 2).astype(np.float32)
    x = np.concatenate([rng.standard_normal(100003).astype(np.float32) * 100, rng.standard_normal(5000).astype(np.float32) * 0.02,
                        mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                        np.array([0.0, -0.0, 448, -448, 449, 464, 465, 1e30, -1e30, np.inf, -np.inf, 2.0 ** -10, 2.0 ** -11, 1e-30], np.float32)])
    want = oracle.e4m3fn_encode(x)
    dx = torch.from_numpy(x).cuda()
    dq = torch.zeros(x.size, dtype=torch.uint8, device="cuda")
    _say(f"[gpu case] convert {x.size} elements")
    pkg.convert_f32_to_e4m3fn(dx, dq, x.size)
    torch.cuda.synchronize()
    assert np.array_equal(dq.cpu().numpy(), want)
    xn = np.array([np.nan, 1.0, -np.nan], np.float32)
    dxn = torch.from_numpy(xn).cuda()
    dqn = torch.zeros(3, dtype=torch.uint8, device="cuda")
    pkg.convert_f32_to_e4m3fn(dxn, dqn, 3)
    q = dqn.cpu().numpy()
    assert (q[0] & 0x7F) == 0x7F and q[1] == 0x38 and (q[2] & 0x7F) == 0x7F


def test_host_launcher_matches_device_path(pkg):
    """fp8_gemm_host (gemmGPU's counterpart): fp32 host values -> convert on device -> GEMM."""
    m, n, k = 128, 128, 256
    a, b, sa, sb = oracle.make_inputs(m, n, k, 61)
    af, bf = oracle.e4m3fn_decode(a), oracle.e4m3fn_decode(b)   # exactly representable
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    L = pkg.lib()
    for option, exact in ((2, True), (0, False), (1, False), (102, False)):
        c = np.zeros((m, n), np.uint16)
        _say(f"[gpu case] fp8_gemm_host option={option}")
        rc = L.fp8_gemm_host(c.ctypes.data, af.ctypes.data, bf.ctypes.data, sa.ctypes.data, sb.ctypes.data, m, n, k, option)
        assert rc == 0
        if exact:
            assert np.array_equal(c, ref)
        else:
            _assert_close(c, ref, f"host option {option}")
    assert L.fp8_gemm_host(c.ctypes.data, af.ctypes.data, bf.ctypes.data, sa.ctypes.data, sb.ctypes.data, m, n, k, 7) == -3


def test_caller_workspace(pkg):
    import torch
    m, n, k = 256, 256, 1024
    a, b, sa, sb = oracle.make_inputs(m, n, k, 62)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    pkg.select(3)
    pkg.force_config(2, 8)
    try:
        need = pkg.workspace_bytes(m, n, k)
    finally:
        pkg.force_config(-1, 0)
        pkg.select(0)
    assert need == pkg.WORKSPACE_HEADER_BYTES + 8 * m * n * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    pkg.set_workspace(ws, need)
    try:
        got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=3, variant=2, ksplit=8)
        _assert_close(got, ref, name)
        pkg.set_workspace(ws, 1024)  # too small for an 8-way split
        with pytest.raises(pkg.Fp8GemmError) as ei:
            _run(pkg, a, b, sa, sb, m, n, k, kernel=3, variant=2, ksplit=8)
        assert ei.value.code == -4
    finally:
        pkg.set_workspace(None, 0)
    got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=3, variant=2, ksplit=8)
    _assert_close(got, ref, name)
    pkg.release()


def test_check_driver_reproduces_the_reference_procedure(pkg):
    """bin/check: seed-7 uniform(-5,5) inputs and scales, M=N=128, K=256, tolerance 100
    (check.cu:137-177), plus a larger shape."""
    exe = os.path.join(os.path.dirname(pkg.lib_path()), "bin", "check")
    if not os.path.exists(exe):
        pytest.skip("bin/check not built")
    for args in ([], ["512", "384", "512", "100"]):
        _say(f"[gpu case] bin/check {' '.join(args)}")
        out = subprocess.run([exe] + args, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "2 matrices are equal" in out.stdout


def test_custom_kernel_operator_form(pkg):
    """torch tensors in the column-major layouts of the challenge harness; fp8 dtype views"""
    import torch
    m, n, k = 256, 576, 512
    a, b, sa, sb = oracle.make_inputs(m, n, k, 321)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    ta = torch.from_numpy(a).cuda().view(torch.float8_e4m3fn).t()        # [m, k], strides (1, m)
    tb = torch.from_numpy(b).cuda().view(torch.float8_e4m3fn).t()
    tsa = torch.from_numpy(sa).cuda().t()                                # [m, k/128], strides (1, m)
    tsb = torch.from_numpy(sb).cuda().t()                                # [ceil(n/128), k/128]
    c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    _say(f"[gpu case] custom_kernel m={m} n={n} k={k}")
    out = pkg.custom_kernel((ta, tb, tsa, tsb, c))
    torch.cuda.synchronize()
    assert out is c
    _assert_close(c.view(torch.int16).cpu().numpy().view(np.uint16), ref, "custom_kernel")
    with pytest.raises(ValueError):
        pkg.custom_kernel((ta.contiguous(), tb, tsa, tsb, c))            # row-major a is refused
    with pytest.raises(ValueError):
        pkg.custom_kernel((ta, tb, tsa, tsb, c.t()))


# ------------------------------------------------------------------ grouped GEMM
def _grouped_case(pkg, ms, n, k, variant, seed):
    import torch
    st = torch.cuda.current_stream().cuda_stream
    host, dev, outs = [], [], []
    for g, m in enumerate(ms):
        mm = max(m, 16)                       # an empty group still gets valid (unused) buffers
        a, b, sa, sb = oracle.make_inputs(mm, n, k, seed + 17 * g)
        host.append((a, b, sa, sb))
        dev.append(_dev(a, b, sa, sb))
        outs.append(torch.full((mm, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16))
    _say(f"[gpu case] grouped ms={ms} n={n} k={k} variant={variant}")
    pkg.force_config(variant, 0)
    try:
        pkg.gemm_grouped([d[0] for d in dev], [d[1] for d in dev], [d[2] for d in dev], [d[3] for d in dev],
                         outs, ms, n, k, st)
        torch.cuda.synchronize()
        name = pkg.last_kernel()
    finally:
        pkg.force_config(-1, 0)
    return host, dev, outs, name


@pytest.mark.parametrize("variant,ms,n,k", [(2, [256, 16, 1040, 0, 512], 576, 768),
                                            (0, [4096, 272, 2048, 1024, 16], 1536, 512),
                                            (1, [512] * 9 + [48, 2064], 1024, 384),
                                            (3, [144] * 40, 384, 640),
                                            (6, [2048, 272, 16, 1024, 4096], 1280, 512),
                                            (2, [128], 128, 384)])
def test_grouped_gemm_equals_the_problems_one_by_one(pkg, variant, ms, n, k):
    host, dev, outs, name = _grouped_case(pkg, ms, n, k, variant, 7000 + n + k)
    assert "_grouped" in name, name
    for g, m in enumerate(ms):
        if m == 0:
            assert (outs[g].cpu().numpy().view(np.uint16) == 0x7FC1).all()      # untouched
            continue
        a, b, sa, sb = host[g]
        got = outs[g].cpu().numpy().view(np.uint16)
        ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
        _assert_close(got, ref, f"{name} group {g}")
        _assert_every_element(got, a, b, sa, sb, m, n, k, f"{name} group {g}")
        single, _ = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_LARGE, variant=variant, persistent=0)
        assert np.array_equal(got, single), f"group {g}: grouped launch and single launch differ"


@pytest.mark.parametrize("ms,n,k", [([40, 256, 24], 256, 256), ([1, 0, 1000, 333, 16], 520, 384),
                                    ([129] * 20, 100, 512), ([2049, 17], 1544, 1024)])
def test_grouped_gemm_pads_groups_off_the_16_byte_grid(pkg, ms, n, k):
    """ragged m (and n): one grouped launch on padded copies, C rows beyond m untouched"""
    import torch
    st = torch.cuda.current_stream().cuda_stream
    host, dev, outs = [], [], []
    for g, m in enumerate(ms):
        mm = max(m, 1)
        a, b, sa, sb = oracle.make_inputs(mm, n, k, 8100 + 13 * g)
        host.append((a, b, sa, sb))
        dev.append(_dev(a, b, sa, sb))
        outs.append(torch.full((mm + 16, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16))  # 16 guard rows
    _say(f"[gpu case] grouped, padded ms={ms} n={n} k={k}")
    pkg.gemm_grouped([d[0] for d in dev], [d[1] for d in dev], [d[2] for d in dev], [d[3] for d in dev],
                     outs, ms, n, k, st)
    torch.cuda.synchronize()
    name = pkg.last_kernel()
    # groups of at most 64 rows go to the decode kernel, taller ones to the tile kernel: one launch of each
    parts = name.split("+")
    # each launch pads only if its own groups need it: the decode kernel takes any row count, the tile kernel
    # and both kernels' columns need multiples of 16
    assert any(p.startswith("padded_") for p in parts) == (n % 16 != 0 or any(m > 64 and m % 16 for m in ms)), name
    assert sum(int(p.rsplit("_grouped", 1)[1]) for p in parts) == sum(1 for m in ms if m), name
    assert ("decode128" in name) == any(0 < m <= 64 for m in ms) and ("tile" in name) == any(m > 64 for m in ms), name
    for g, m in enumerate(ms):
        got = outs[g].cpu().numpy().view(np.uint16)
        assert (got[m:] == 0x7FC1).all(), f"group {g}: rows beyond m written"
        if m:
            a, b, sa, sb = host[g]
            _assert_close(got[:m], oracle.ref_gemm(a, b, sa, sb, m, n, k), f"{name} group {g}")
            _assert_every_element(got[:m], a, b, sa, sb, m, n, k, f"{name} group {g}")
    pkg.release()


def test_grouped_gemm_with_a_tile_shape_that_has_no_grouped_form(pkg):
    """tile variant 5 pinned (its K loop is written for a single problem): the groups run one by one"""
    ms, n, k = [256, 528, 48], 384, 256
    host, dev, outs, name = _grouped_case(pkg, ms, n, k, 5, 8250)
    assert name == "tile256x192w4_k1_persistent", name
    for g, m in enumerate(ms):
        a, b, sa, sb = host[g]
        _assert_close(outs[g].cpu().numpy().view(np.uint16), oracle.ref_gemm(a, b, sa, sb, m, n, k), f"group {g}")


@pytest.mark.parametrize("ms,n,k,expect", [
    ([16 + (g % 3) for g in range(70)], 64, 128, "decode128_k1_grouped35x2"),
    ([1 + (5 * g) % 64 for g in range(130)], 512, 384, "_grouped42x3"),                       # 44 + 44 + 42
    ([0, 0] + [16] * 64 + [0], 256, 256, "_grouped64"),                                       # 64 live ones: one launch
    ([(8 if g % 2 else 80 + g) for g in range(150)], 256, 256, "_grouped37x2+"),              # 75 small, 75 tall
])
def test_grouped_gemm_takes_more_groups_than_one_launch_holds(pkg, ms, n, k, expect):
    """more groups than a launch holds (64) run as the fewest launches of equal size, every group as in a
    call of its own"""
    host, dev, outs, name = _grouped_case(pkg, ms, n, k, -1, 8300 + len(ms))
    assert expect in name, name
    if "+" in expect:
        assert name.endswith("_grouped37x2"), name
    for g, m in enumerate(ms):
        got = outs[g].cpu().numpy().view(np.uint16)
        assert (got[m:] == 0x7FC1).all(), f"group {g}: rows beyond m written"
        if m == 0:
            continue
        a, b, sa, sb = host[g]
        # buffers made for 16 rows and read with m < 16 per k-row: the first k * m values, as the kernel sees them
        a_seen = np.ascontiguousarray(a.reshape(-1)[:k * m].reshape(k, m))
        sa_seen = np.ascontiguousarray(sa.reshape(-1)[:(k // 128) * m].reshape(k // 128, m))
        _assert_close(got[:m], oracle.ref_gemm(a_seen, b, sa_seen, sb, m, n, k), f"group {g}")
    pkg.release()


@pytest.mark.parametrize("ms,n,k", [([16, 32, 64, 48, 16, 0, 32], 1536, 2048),      # K split inside the kernel
                                    ([64] * 24, 512, 1024),
                                    ([16] * 64, 256, 384),
                                    ([32, 48], 576, 128),                             # one K block: nothing to split
                                    ([16, 64, 32, 16], 7168, 512),
                                    ([16] * 62 + [48, 32], 4096, 768)])              # 2048 work units: two workgroups per CU
def test_grouped_decode_groups_equal_the_problems_one_by_one(pkg, ms, n, k):
    """groups of at most 64 rows (an MoE layer in a decode step): one launch of the decode kernel, every
    group bit-identical to a single launch of that kernel with the same K split"""
    host, dev, outs, name = _grouped_case(pkg, ms, n, k, -1, 9100 + n + k)
    live = sum(1 for m in ms if m)
    assert name.startswith("decode128_k") and name.endswith(f"_grouped{live}"), name
    ks = int(name.split("_k")[1].split("_")[0])
    for g, m in enumerate(ms):
        if m == 0:
            assert (outs[g].cpu().numpy().view(np.uint16) == 0x7FC1).all()      # untouched
            continue
        a, b, sa, sb = host[g]
        got = outs[g].cpu().numpy().view(np.uint16)
        _assert_close(got, oracle.ref_gemm(a, b, sa, sb, m, n, k), f"{name} group {g}")
        _assert_every_element(got, a, b, sa, sb, m, n, k, f"{name} group {g}")
        single, sname = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_SKINNY, variant=1, ksplit=ks)
        assert sname == f"decode128_k{ks}", sname
        assert np.array_equal(got, single), f"group {g}: grouped launch and single launch differ"


def test_grouped_decode_groups_off_the_16_byte_grid_and_mixed_with_tall_groups(pkg):
    """ragged token counts of 1 to 64 rows run in one decode launch (on padded copies only when n is off the
    grid, or the launch is large enough for the streaming form); a
    call that also holds taller groups launches the tile kernel for those; rows beyond m stay untouched"""
    import torch
    st = torch.cuda.current_stream().cuda_stream
    for ms, n, k in [([1, 7, 64, 33, 16, 50, 2], 1536, 1024), ([5, 300, 64, 1000, 17], 640, 512), ([3, 9], 200, 256),
                     # more than one round of workgroups; more K blocks than ring slots
                     ([3, 16, 9, 1] * 6, 2048, 384), ([17, 31, 5, 20] * 5, 2048, 384), ([20, 7], 256, 3328),
                     # enough 256-column strips for the streaming form, which wants rows on the grid: padded copies of A
                     ([1 + (7 * g) % 40 for g in range(64)], 2048, 256)]:
        host, dev, outs = [], [], []
        for g, m in enumerate(ms):
            a, b, sa, sb = oracle.make_inputs(m, n, k, 9300 + 11 * g + n)
            host.append((a, b, sa, sb))
            dev.append(_dev(a, b, sa, sb))
            outs.append(torch.full((m + 16, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16))
        _say(f"[gpu case] grouped decode, ragged ms={ms} n={n} k={k}")
        pkg.gemm_grouped([d[0] for d in dev], [d[1] for d in dev], [d[2] for d in dev], [d[3] for d in dev],
                         outs, ms, n, k, st)
        torch.cuda.synchronize()
        name = pkg.last_kernel()
        wide_units = sum(1 for m in ms if m <= 64) * -(-n // 256)
        streams = wide_units >= 256 and 5 * wide_units >= 4 * -(-wide_units // 256) * 256
        assert "decode128_k" in name and name.startswith("padded_decode128_k") == (n % 16 != 0 or streams), name
        if max(ms) > 64:
            assert "+" in name and "tile" in name, name
        for g, m in enumerate(ms):
            got = outs[g].cpu().numpy().view(np.uint16)
            assert (got[m:] == 0x7FC1).all(), f"group {g}: rows beyond m written"
            a, b, sa, sb = host[g]
            _assert_close(got[:m], oracle.ref_gemm(a, b, sa, sb, m, n, k), f"{name} group {g}")
            _assert_every_element(got[:m], a, b, sa, sb, m, n, k, f"{name} group {g}")
    pkg.release()


@pytest.mark.parametrize("ms,n,k,expect", [
    ([16, 160, 144, 208, 96, 128, 272], 7168, 256, "tile256x256_k1_grouped7"),           # one small group rides along
    ([5, 161, 144, 200, 96, 130, 272, 64], 6400, 384, "padded_tile256x256_k1_grouped8"),  # ragged: all on padded copies
    ([5, 160, 144, 208, 96, 128, 272, 176], 7168, 256, "_grouped1+tile256x256_k1_grouped7"),  # tall ones on the grid
    ([16, 32, 160, 144, 208], 512, 256, "_grouped2+tile"),                               # too many small ones to fold
    ([16, 160, 144, 208, 96, 128, 272], 512, 256, "_k1_grouped7"),                       # few tiles: the cost model's shape
    ([300, 700, 512, 160], 768, 256, "_grouped4"),                                       # taller groups: likewise
])
def test_grouped_tile_launch_of_groups_of_one_tile_and_small_groups_riding_along(pkg, ms, n, k, expect):
    """groups of up to 256 rows take the 256x256 tile (one tile row each, B streamed once); a few groups of at
    most 64 rows beside many taller ones join the tile launch unless that alone would force padded copies"""
    import torch
    st = torch.cuda.current_stream().cuda_stream
    host, dev, outs = [], [], []
    for g, m in enumerate(ms):
        a, b, sa, sb = oracle.make_inputs(m, n, k, 9700 + 13 * g + n)
        host.append((a, b, sa, sb))
        dev.append(_dev(a, b, sa, sb))
        outs.append(torch.full((m + 16, n), 0x7FC1, dtype=torch.int32, device="cuda").to(torch.int16))
    _say(f"[gpu case] grouped, groups of one tile ms={ms} n={n} k={k}")
    pkg.gemm_grouped([d[0] for d in dev], [d[1] for d in dev], [d[2] for d in dev], [d[3] for d in dev],
                     outs, ms, n, k, st)
    torch.cuda.synchronize()
    name = pkg.last_kernel()
    assert expect in name and (expect[0] in "+_" or name == expect), name
    for g, m in enumerate(ms):
        got = outs[g].cpu().numpy().view(np.uint16)
        assert (got[m:] == 0x7FC1).all(), f"group {g}: rows beyond m written"
        a, b, sa, sb = host[g]
        _assert_close(got[:m], oracle.ref_gemm(a, b, sa, sb, m, n, k), f"{name} group {g}")
        _assert_every_element(got[:m], a, b, sa, sb, m, n, k, f"{name} group {g}")
    pkg.release()


def test_seeded_sweep_of_shapes_and_plans(pkg):
    """forty pseudo-random (shape, tile, K split, persistence) combinations against the oracle"""
    rs = np.random.RandomState(20241125)
    for case in range(40):
        m = int(rs.randint(1, 48)) * 16
        n = int(rs.randint(1, 48)) * 16
        k = int(rs.randint(1, 13)) * 128
        variant = int(rs.randint(-1, 5))
        nkb = k // 128
        ksplit = int(rs.choice([0, 1, 1, 2, 3, 5])) if nkb >= 5 else int(rs.choice([0, 1]))
        if ksplit > 1 and (ksplit - 1) * -(-nkb // ksplit) >= nkb:
            ksplit = 0                        # a split without a K block of its own: not a valid pin
        persistent = int(rs.randint(-1, 2))
        a, b, sa, sb = oracle.make_inputs(m, n, k, 9000 + case, 0.5, 20.0)
        ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
        got, name = _run(pkg, a, b, sa, sb, m, n, k, kernel=pkg.KERNEL_AUTO, variant=variant, ksplit=ksplit,
                         persistent=persistent)
        _assert_close(got, ref, f"case {case}: m={m} n={n} k={k} -> {name}")
        _assert_every_element(got, a, b, sa, sb, m, n, k, f"case {case}: {name}")
