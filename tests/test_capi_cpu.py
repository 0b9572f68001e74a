"""Host-side behaviour of the C ABI that needs no GPU: the library loads, exports every
symbol include/fp8_block_gemm.h declares, validates arguments before any device call, and
the dispatcher's shape logic.  No compute call is made here."""
import ctypes as C
import os

import pytest


def test_library_exports_every_declared_symbol(pkg):
    L = pkg.lib()
    names = pkg.abi_symbols()
    assert "fp8_block_gemm" in names and "fp8_gemm_host" in names and "fp8_block_gemm_ex" in names
    assert len(names) >= 22
    for name in names:
        assert hasattr(L, name), f"{name} declared in the header but not exported"
    assert L.fp8_block_gemm_abi_version() == 5


def test_argument_validation_happens_before_any_device_call(pkg):
    L = pkg.lib()
    p = 4096  # never dereferenced
    assert L.fp8_block_gemm(None, p, p, p, p, 16, 16, 128) == -1
    assert L.fp8_block_gemm(p, p, p, p, None, 16, 16, 128) == -1
    assert L.fp8_block_gemm(p, p, p, p, p, 0, 16, 128) == -2
    assert L.fp8_block_gemm(p, p, p, p, p, 16, -3, 128) == -2
    assert L.fp8_block_gemm(p, p, p, p, p, 16, 16, 100) == -2
    assert L.fp8_block_gemm(p, p, p, p, p, 16, 16, 0) == -2
    assert L.fp8_block_gemm_stream(p, p, p, p, p, 70000, 16, 65536, None) == -5
    assert L.fp8_block_gemm_scalar(p, None, p, p, p, 16, 16, 128, None) == -1
    assert L.fp8_gemm_host(None, p, p, p, p, 16, 16, 128, 0) == -1
    assert L.fp8_gemm_host(p, p, p, p, p, 16, 16, 130, 0) == -2
    assert L.fp8_convert_f32_to_e4m3fn(None, p, 10, None) == -1
    assert L.fp8_convert_f32_to_e4m3fn(None, None, 0, None) == 0
    assert L.fp8_convert_f32_to_e4m3fn(p + 4, p, 10, None) == -7     # float4 loads need 16-byte alignment
    assert L.fp8_convert_f32_to_e4m3fn(p, p + 2, 10, None) == -7     # 4-byte stores
    for fn in (L.fp8_quantize_a_1x128, L.fp8_quantize_b_128x128):
        assert fn(None, 0, p, p, 16, 128, None) == -1
        assert fn(p, 0, p, None, 16, 128, None) == -1
        assert fn(p, 0, p, p, 0, 128, None) == -2
        assert fn(p, 0, p, p, 16, 192, None) == -2
        assert fn(p, 0, p, p, 70000, 65536, None) == -5
        assert fn(p, 7, p, p, 16, 128, None) == -6
        assert fn(p + 2, 0, p, p, 16, 128, None) == -7


def test_grouped_entry_point_validates_every_group_first(pkg):
    L = pkg.lib()
    p = 4096
    arr = lambda *v: (C.c_void_p * len(v))(*v)
    ints = lambda *v: (C.c_int * len(v))(*v)
    ok = arr(p, p)
    assert L.fp8_block_gemm_grouped(-1, ok, ok, ok, ok, ok, ints(16, 16), 16, 128, None) == -2
    assert L.fp8_block_gemm_grouped(0, None, None, None, None, None, None, 16, 128, None) == 0
    assert L.fp8_block_gemm_grouped(2, ok, ok, ok, ok, ok, None, 16, 128, None) == -1
    assert L.fp8_block_gemm_grouped(2, ok, ok, ok, ok, ok, ints(0, 0), 16, 128, None) == 0      # nothing to do
    assert L.fp8_block_gemm_grouped(2, ok, arr(p, None), ok, ok, ok, ints(16, 16), 16, 128, None) == -1
    assert L.fp8_block_gemm_grouped(2, ok, arr(p, None), ok, ok, ok, ints(16, 0), 16, 100, None) == -2
    assert L.fp8_block_gemm_grouped(2, ok, ok, ok, ok, ok, ints(16, -4), 16, 128, None) == -2
    with pytest.raises(ValueError):
        pkg.gemm_grouped([p], [p, p], [p], [p], [p], [16], 16, 128)
    # the per-call form validates the same way, and its options as fp8_block_gemm_ex does
    ex = L.fp8_block_gemm_grouped_ex
    assert ex(-1, ok, ok, ok, ok, ok, ints(16, 16), 16, 128, None, None, 0, None) == -2
    assert ex(2, ok, ok, ok, ok, ok, None, 16, 128, None, None, 0, None) == -1
    assert ex(2, ok, ok, ok, ok, ok, ints(0, 0), 16, 128, None, None, 0, None) == 0
    assert ex(2, ok, arr(p, None), ok, ok, ok, ints(16, 16), 16, 128, None, None, 0, None) == -1
    assert ex(2, ok, ok, ok, ok, ok, ints(16, -4), 16, 128, None, None, 0, None) == -2
    bad = pkg.Options(kernel=9)
    assert ex(2, ok, ok, ok, ok, ok, ints(16, 16), 16, 128, C.byref(bad), None, 0, None) == \
        L.fp8_block_gemm_ex(p, p, p, p, p, 16, 16, 128, C.byref(bad), None, 0, None) != 0
    with pytest.raises(ValueError):
        pkg.gemm_grouped_ex([p], [p, p], [p], [p], [p], [16], 16, 128)


def test_error_strings_and_exception(pkg):
    assert "NULL" in pkg.error_string(-1)
    assert "128" in pkg.error_string(-2)
    assert pkg.error_string(0) == "success"
    with pytest.raises(pkg.Fp8GemmError) as ei:
        pkg.gemm(4096, 4096, 4096, 4096, 4096, 16, 16, 64)
    assert ei.value.code == -2


def test_select_and_force_config_validate(pkg):
    L = pkg.lib()
    assert L.fp8_block_gemm_select(99) == -3
    assert L.fp8_block_gemm_select(-1) == -3
    assert L.fp8_block_gemm_force_config(99, 0) == -3
    assert L.fp8_block_gemm_force_config(0, 1000) == -3
    assert L.fp8_block_gemm_force_config(0, 17) == -3                # the dispatcher splits K at most 16 times
    assert L.fp8_block_gemm_force_config(0, 16) == 0
    for kid in (1, 2, 3, 4, 0):
        assert L.fp8_block_gemm_select(kid) == 0
    assert L.fp8_block_gemm_force_config(-1, 0) == 0
    assert L.fp8_block_gemm_set_persistent(2) == -3
    assert L.fp8_block_gemm_set_persistent(1) == 0
    assert pkg.plan(8192, 4608, 7168).endswith("_persistent")
    assert pkg.plan(2048, 2048, 2048).endswith("_persistent")   # forced: whenever the kernel allows
    assert pkg.plan(256, 256, 256) == "tile64x64_k1"             # the 64x64 tile has no persistent form
    assert L.fp8_block_gemm_set_persistent(0) == 0
    assert not pkg.plan(8192, 4608, 7168).endswith("_persistent")
    assert L.fp8_block_gemm_set_persistent(-1) == 0
    assert pkg.plan(8192, 4608, 7168).endswith("_persistent")   # 768 tiles on 256 CUs
    assert not pkg.plan(2048, 2048, 2048).endswith("_persistent")


def test_workspace_contract(pkg):
    L = pkg.lib()
    assert pkg.workspace_bytes(0, 8, 128) == 0
    assert pkg.workspace_bytes(64, 64, 128) == 0                     # one K block: nothing to split
    assert pkg.workspace_bytes(8192, 4608, 7168) == 0                # plan does not split K
    assert pkg.plan(1024, 512, 7168) == "tile64x64_k2f"                # f: the K splits are added inside the kernel
    H = pkg.WORKSPACE_HEADER_BYTES                                   # the mailbox ahead of every plan's data
    assert pkg.workspace_bytes(1024, 512, 7168) == H + 2 * 1024 * 512 * 4
    assert L.fp8_block_gemm_force_config(2, 8) == 0                  # follows a forced configuration
    try:
        assert pkg.workspace_bytes(256, 256, 1024) == H + 8 * 256 * 256 * 4
    finally:
        assert L.fp8_block_gemm_force_config(-1, 0) == 0
    assert L.fp8_block_gemm_set_workspace(4096 + 8, 1 << 20) == -4   # misaligned
    assert L.fp8_block_gemm_set_workspace(None, 0) == 0
    assert L.fp8_block_gemm_release() == 0                           # nothing allocated yet


def test_per_call_entry_point_validates_and_never_allocates(pkg):
    """fp8_block_gemm_ex / _ws: bad options and a missing workspace are host-side errors, reported
    before any device call (the pointers below are never dereferenced)."""
    L = pkg.lib()
    p = 4096
    O = pkg.Options
    assert L.fp8_block_gemm_ex(p, p, p, p, p, 16, 16, 100, None, None, 0, None) == -2
    assert L.fp8_block_gemm_ex(None, p, p, p, p, 16, 16, 128, None, None, 0, None) == -1
    for bad in (O(kernel=9), O(tile_variant=99), O(ksplit=17), O(ksplit=-1), O(persistent=2)):
        assert L.fp8_block_gemm_ex(p, p, p, p, p, 256, 256, 1024, C.byref(bad), None, 0, None) == -3
        assert pkg.workspace_bytes_ex(256, 256, 1024, bad) == 0
    split = O(kernel=pkg.KERNEL_SPLITK, tile_variant=2, ksplit=4)
    need = pkg.workspace_bytes_ex(256, 256, 1024, split)
    assert need == pkg.WORKSPACE_HEADER_BYTES + 4 * 256 * 256 * 4
    assert L.fp8_block_gemm_ex(p, p, p, p, p, 256, 256, 1024, C.byref(O(flags=2)), None, 0, None) == -3   # unknown flag
    # a plan that needs a workspace and is not given one (or too little, or a misaligned one)
    assert L.fp8_block_gemm_ex(p, p, p, p, p, 256, 256, 1024, C.byref(split), None, 0, None) == -4
    assert L.fp8_block_gemm_ex(p, p, p, p, p, 256, 256, 1024, C.byref(split), p, need - 1, None) == -4
    assert L.fp8_block_gemm_ex(p, p, p, p, p, 256, 256, 1024, C.byref(split), p + 16, need, None) == -4
    # operands off a 16-byte boundary run on padded copies: the aligned figure is not enough, and says so
    assert L.fp8_block_gemm_ws(p + 1, p, p, p, p, 256, 256, 1024, p, 1024, None) == -4
    # the per-call options do not leak into, or read, the process-wide switches
    pkg.force_config(1, 4)
    try:
        assert pkg.workspace_bytes_ex(1024, 512, 2048) == pkg.workspace_bytes_ex(1024, 512, 2048, O())
        assert pkg.workspace_bytes(1024, 512, 2048) == pkg.WORKSPACE_HEADER_BYTES + 4 * 1024 * 512 * 4
    finally:
        pkg.force_config(-1, 0)


def test_workspace_queries_cover_every_alignment(pkg):
    for (m, n, k) in [(256, 256, 1024), (1024, 512, 7168), (8192, 4608, 7168), (33, 100, 128), (32, 7168, 2048)]:
        aligned = pkg.workspace_bytes_ex(m, n, k)
        anyal = pkg.workspace_bytes_ex(m, n, k, None, True)
        assert anyal >= aligned
        m16, n16 = (m + 15) // 16 * 16, (n + 15) // 16 * 16
        copies = k * m16 + (k // 128) * m16 * 4 + k * n16 + m16 * n16 * 2
        assert anyal >= copies, (m, n, k)
    # grouped: at least the copies of every group, and at least any single group's need
    ms = [509, 1027, 771]
    tot = pkg.grouped_workspace_bytes(ms, 7168, 2048)
    assert tot >= sum(2048 * ((x + 15) // 16 * 16) for x in ms)
    assert tot >= max(pkg.workspace_bytes_ex(x, 7168, 2048, None, True) for x in ms)
    assert pkg.grouped_workspace_bytes([], 7168, 2048) == 0
    # decode-sized groups: the header (their K splits meet in its mailbox) and every group's padded copies
    small = [16, 64, 33]
    assert pkg.grouped_workspace_bytes(small, 7168, 2048) >= pkg.WORKSPACE_HEADER_BYTES + sum(
        2048 * ((x + 15) // 16 * 16) + 2048 * 7168 for x in small)
    assert pkg.grouped_workspace_bytes([16, 32], 256, 256) >= pkg.WORKSPACE_HEADER_BYTES
    assert pkg.grouped_workspace_bytes(small, 7168, 2048, per_call=True) == pkg.grouped_workspace_bytes(small, 7168, 2048)
    assert pkg.grouped_workspace_bytes(small, 7168, 2048, pkg.Options(kernel=9)) == 0


def test_noalloc_entry_point_validates_before_any_device_call(pkg):
    L = pkg.lib()
    p = 4096
    assert L.fp8_block_gemm_noalloc(None, p, p, p, p, 16, 16, 128, None) == -1
    assert L.fp8_block_gemm_noalloc(p, p, p, p, p, 16, 16, 100, None) == -2
    assert L.fp8_block_gemm_noalloc(p, p, p, p, p, 70000, 16, 65536, None) == -5
    # a plan whose partial sums exceed the fixed array: refused by size, no device touched
    pkg.select(pkg.KERNEL_SPLITK)
    pkg.force_config(2, 4)
    try:
        assert pkg.workspace_bytes(4096, 4096, 1024) > pkg.NOALLOC_MAX_BYTES
        assert L.fp8_block_gemm_noalloc(p, p, p, p, p, 4096, 4096, 1024, None) == -4
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)


def test_one_wave_per_simd_variant_is_opt_in(pkg):
    assert "w4" not in pkg.plan(8192, 4608, 7168)
    pkg.force_config(5, 0)
    try:
        assert pkg.plan(8192, 4608, 7168) == "tile256x192w4_k1_persistent"
        assert pkg.plan(256, 192, 128) == "tile256x192w4_k1_persistent"   # exists in the persistent form only
        pkg.force_config(5, 2)
        with pytest.raises(pkg.Fp8GemmError):
            pkg.plan(1024, 512, 2048)                                     # and without a K split
    finally:
        pkg.force_config(-1, 0)


def test_dispatcher_plans(pkg):
    pkg.select(pkg.KERNEL_AUTO)
    pkg.force_config(-1, 0)
    assert pkg.plan(8192, 4608, 7168).startswith("tile")
    assert "_k1" in pkg.plan(8192, 4608, 7168)
    assert pkg.plan(32, 7168, 2048).startswith("decode128")
    assert pkg.plan(33, 100, 128).startswith("padded_")   # rows not 16-byte aligned: padded copies
    assert pkg.plan(8191, 4607, 7168) == "padded_" + pkg.plan(8192, 4608, 7168)
    assert pkg.plan(16777215, 16, 128) == "scalar"         # padding would pass the operand size limit
    assert pkg.workspace_bytes(33, 100, 128) >= 128 * 48 + 128 * 112 + 48 * 4 + 48 * 112 * 2
    ks = int(pkg.plan(2048, 576, 7168).split("_k")[1].rstrip("f"))
    assert ks > 1                                          # few tiles, long K: split
    # a handful of 64x64 tiles: one launch (unsplit, or the splits added inside the kernel), not a split of
    # every few K blocks with a reduction kernel behind it
    assert pkg.plan(112, 96, 1536) == "tile64x64_k1"
    assert pkg.plan(128, 128, 7168) == "tile64x64_k7f"
    assert pkg.plan(256, 256, 3072) == "tile64x64_k4f"
    assert pkg.plan(1536, 64, 2304) == "tile64x64_k3f"
    # 85 tiles x 3 splits added inside the kernel would be 88 x 3 workgroups (the splits of a tile share an XCD):
    # more than one round
    assert pkg.plan(2144, 608, 3072) == "tile128x128_k2f"
    assert pkg.plan(2048, 576, 3072) == "tile128x128_k3f"  # 80 tiles x 3: one round
    # 128x128 tiles do not split into ranges of fewer than 8 K blocks (64 KB per split to hand over)
    assert pkg.plan(1024, 2048, 1536) == "tile128x128_k1"
    # 129 ... 256 rows over 32 MB of B or more: one row of 256x128 tiles streams B once
    assert pkg.plan(208, 18816, 3072) == "tile256x128_k1"
    assert pkg.plan(192, 14720, 7168) == "tile256x128_k2"   # ... where the model would take 128x128 tiles as well
    assert pkg.plan(256, 7168, 7168) == "tile128x128_k2f"   # no 256x128 plan within reach: stays
    assert pkg.plan(400, 11648, 7168) == "tile128x192_k1"  # more rows: the cost model's tile
    # decode shapes (M <= 32): 128-column strips with the K range split so that one round of workgroups
    # (at most 256) streams B, the splits added inside the kernel
    assert pkg.plan(32, 7168, 2048) == "decode128_k4"      # 56 strips x 4
    assert pkg.plan(16, 1536, 2048) == "decode128_k4"
    assert pkg.plan(32, 16384, 7168) == "decode128_k2"     # 128 strips x 2
    assert pkg.plan(32, 128, 128) == "decode128_k1"        # one K block: nothing to split
    assert pkg.workspace_bytes(32, 7168, 2048) == pkg.WORKSPACE_HEADER_BYTES   # the splits meet in the header's mailbox
    # 33 ... 64 rows: 64x64 tiles with the K range split inside the kernel, tiles x splits within one workgroup
    # per CU and at least 3 K blocks per split; the wide strips where N x K is large or the row count is off
    # the 16-byte grid (the strips take it as it is, the tiles would need padded copies)
    assert pkg.plan(64, 1536, 7168) == "tile64x64_k8f"     # 24 tiles x 8
    assert pkg.plan(48, 1536, 1536) == "tile64x64_k4f"     # 3 K blocks per split
    assert pkg.plan(64, 7168, 2048) == "tile64x64_k2f"     # 112 tiles x 2
    assert pkg.plan(64, 7168, 7168) == "decode128_k4"
    assert pkg.plan(40, 4608, 7168) == "decode128_k6"      # 36 strips over 8 XCDs: 5 x 6 workgroups on an XCD's 32 CUs
    assert pkg.plan(7, 7168, 2048) == "decode128_k4"       # a decode batch of 7 rows: no padded copy
    # 256-column strips where they save a round of workgroups on an XCD (144 strips x 3 splits: 54 on 32 CUs;
    # 72 x 3: 27) and in unsplit launches of several rounds (a projection onto a vocabulary)
    assert pkg.plan(32, 18432, 7168) == "decode256_k3"
    assert pkg.plan(8, 131072, 4096) == "decode256_k1"
    # 129 ... 256 strips of 256 columns unsplit: one round that streams (384 strips of 128 would take two turns)
    assert pkg.plan(16, 49152, 4096) == "decode256_k1"
    assert pkg.plan(16, 57344, 8192) == "decode256_k1"
    assert pkg.plan(8, 81920, 2048) == "decode256_k1"      # rows off the grid, several rounds: the wider strips
    assert pkg.plan(16, 28672, 4096) == "decode128_k1"     # 224 strips of 128: one round
    assert pkg.plan(32, 7168, 7168) == "decode128_k4"
    pkg.select(pkg.KERNEL_SKINNY)
    pkg.force_config(-1, 3)
    assert pkg.plan(32, 7168, 2048) == "decode128_k3"      # a pinned K split reaches the decode kernels too
    pkg.force_config(0, 0)                                 # tile_variant 0 / 1 under this family: narrow / wide strips
    assert pkg.plan(32, 7168, 2048) == "skinny_k1"
    assert pkg.plan(32, 1536, 7168) == "skinny_k4"
    pkg.force_config(1, 2)
    assert pkg.plan(32, 7168, 2048) == "decode128_k2"
    pkg.force_config(-1, 0)
    pkg.select(pkg.KERNEL_AUTO)
    pkg.set_fused_reduction(0)                             # reduction kernel instead of the in-kernel reduction
    try:
        assert pkg.plan(64, 1536, 7168) == "tile64x64_k7" and pkg.plan(32, 7168, 2048) == "skinny_k1"
        assert pkg.plan(2048, 576, 7168) == "tile128x128_k3"
        pkg.set_fused_reduction(1)
        pkg.select(pkg.KERNEL_SPLITK)
        pkg.force_config(1, 3)
        assert pkg.plan(2048, 576, 7168) == "tile256x128_k3f"   # whenever the other splits' tiles fit the mailbox
        pkg.force_config(1, 6)
        assert pkg.plan(2048, 576, 7168) == "tile256x128_k6"    # 40 tiles x 5 x 128 KiB do not
        pkg.force_config(-1, 0)
        pkg.select(pkg.KERNEL_AUTO)
    finally:
        pkg.set_fused_reduction(-1)
        pkg.force_config(-1, 0)
        pkg.select(pkg.KERNEL_AUTO)
    assert pkg.plan(2048, 576, 7168) == "tile128x128_k3f"   # two or three splits of 128x128 tiles: inside the kernel
    assert pkg.plan(512, 512, 4096).startswith("tile64x64_k") and pkg.plan(512, 512, 4096).endswith("f")
    pkg.select(pkg.KERNEL_SCALAR)
    assert pkg.plan(8192, 4608, 7168) == "scalar"
    pkg.select(pkg.KERNEL_SKINNY)
    with pytest.raises(pkg.Fp8GemmError):
        pkg.plan(8192, 4608, 7168)                         # skinny cannot run M = 8192
    pkg.select(pkg.KERNEL_AUTO)
    pkg.force_config(1, 4)
    assert pkg.plan(1024, 512, 2048) == "tile256x128_k4"
    pkg.force_config(-1, 0)


def test_library_owned_workspace_growth_policy(pkg):
    """the library-owned workspace at least doubles when it grows: the buffers it retires on the way
    never add up to more than the live one"""
    grow = pkg.lib().fp8_block_gemm_workspace_growth
    assert grow(0, 1000) == 1000 and grow(4096, 100) == 4096 and grow(4096, 4096) == 4096
    assert grow(4096, 4097) == 8192 and grow(4096, 100000) == 100000
    have, retired = 0, 0
    for need in [1 << 10, 3 << 10, 5 << 10, 6 << 10, 7 << 10, 100 << 10, 101 << 10, 1 << 20, (1 << 20) + 1]:
        new = grow(have, need)
        assert new >= need
        if new != have:
            retired += have
            have = new
        assert retired <= have
    assert grow(2 ** 63 + 5, 2 ** 63 + 6) == 2 ** 64 - 1        # saturates instead of wrapping


def test_header_cites_reference_for_every_entry_point(pkg):
    hdr = open(os.path.join(os.path.dirname(pkg.lib_path()), "..", "include", "fp8_block_gemm.h")).read()
    assert hdr.count("/root/reference/") >= 8


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_generated_k_loop_is_what_its_generator_writes():
    """csrc/w4_loop.inc (the assembly K loop of tile variant 5) is committed generated text: it has to be
    exactly what csrc/gen_w4_loop.py prints, or the library was built from something nobody can regenerate"""
    import os
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fp8-quant-matmul_amd", "csrc")
    out = subprocess.run([sys.executable, os.path.join(csrc, "gen_w4_loop.py")], capture_output=True, text=True,
                         check=True).stdout
    with open(os.path.join(csrc, "w4_loop.inc")) as f:
        assert f.read() == out
