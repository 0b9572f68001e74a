"""fp8_block_gemm_noalloc: the entry point whose workspace is a fixed array in the library's device
image.  Called through the C ABI on plans that use that workspace (a K split, padded copies), twice in
a row with the second problem smaller, against fp8_block_gemm_stream on the same inputs: bit for bit."""
import sys

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _both(pkg, m, n, k, seed, expect):
    import torch
    a, b, sa, sb = oracle.make_inputs(m, n, k, seed)
    dev = [torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in (a, b, sa, sb)]
    c0 = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
    c1 = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _say(f"[gpu case] noalloc m={m} n={n} k={k} plan={pkg.plan(m, n, k)}")
    pkg.gemm(*dev, c0, m, n, k, st)
    torch.cuda.synchronize()
    name0 = pkg.last_kernel()
    pkg.gemm_noalloc(*dev, c1, m, n, k, st)
    torch.cuda.synchronize()
    name1 = pkg.last_kernel()
    assert name0 == name1 and expect in name1, (name0, name1)
    assert np.array_equal(c0.cpu().numpy(), c1.cpu().numpy()), name1
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    assert oracle.compare_bf16(c1.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0, name1


def test_noalloc_entry_point_matches_the_stream_entry_point(pkg):
    pkg.select(0)
    pkg.force_config(-1, 0)
    _both(pkg, 2048, 576, 7168, 8501, "_k3")       # K split: 14 MB of fp32 partials in the fixed array
    _both(pkg, 1024, 512, 7168, 8502, "_k2")       # a smaller problem right after, same array
    _both(pkg, 250, 300, 512, 8503, "padded_")     # padded copies
    _both(pkg, 8192, 4608, 256, 8504, "_k1")       # needs no workspace at all


def test_noalloc_entry_point_refuses_what_does_not_fit(pkg):
    import torch
    L = pkg.lib()
    m, n, k = 4096, 4096, 1024
    pkg.select(pkg.KERNEL_SPLITK)
    pkg.force_config(2, 4)
    try:
        assert pkg.workspace_bytes(m, n, k) > pkg.NOALLOC_MAX_BYTES
        t = torch.zeros(16, dtype=torch.uint8, device="cuda")   # never dereferenced: the size check comes first
        p = t.data_ptr()
        assert L.fp8_block_gemm_noalloc(p, p, p, p, p, m, n, k, None) == -4
        assert L.fp8_block_gemm_noalloc(None, p, p, p, p, m, n, k, None) == -1
        assert L.fp8_block_gemm_noalloc(p, p, p, p, p, m, n, 100, None) == -2
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
