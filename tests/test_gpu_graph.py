"""The launches of the library can be recorded into a HIP graph and replayed.

Every entry point that takes a stream only enqueues kernels on it (no allocation, no
synchronisation, no memset) as long as a K-splitting plan finds its workspace in place, so a
caller may capture a quantise -> GEMM chain once and replay it.  Each case below records the
calls on a capturing stream, then replays the graph several times with new contents in the
same input buffers and eager work in between, and requires every replay to equal the eager
result on the same contents bit for bit.
"""
import sys

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _fill(dst, src):
    import torch
    dst.copy_(torch.from_numpy(np.ascontiguousarray(src)).view(dst.dtype).reshape(dst.shape))


CASES = [
    # m, n, k, kernel family, tile variant, ksplit, persistent mode
    (32, 1024, 512, 0, -1, 0, -1),      # decode shape under automatic dispatch
    (32, 1024, 512, 4, 0, 0, -1),       # narrow-strip decode kernel
    (32, 2048, 2048, 4, 1, 4, -1),      # wide-strip decode kernel, K splits added inside the kernel (mailbox in the workspace header)
    (5, 2048, 2048, 0, -1, 0, -1),      # a decode batch off the 16-row grid: rows taken as they are, no copy launch in the graph
    (40, 1536, 1024, 0, -1, 0, -1),     # the same with three row tiles
    (256, 384, 512, 0, -1, 0, -1),      # small tile kernel picked by the dispatcher
    (512, 512, 384, 0, 2, 0, 1),        # persistent form
    (256, 256, 1024, 3, 2, 4, -1),      # K split over workgroups + reduction, caller's workspace
]


@pytest.mark.parametrize("m,n,k,kernel,variant,ksplit,persistent", CASES)
def test_gemm_graph_replays_equal_eager(pkg, m, n, k, kernel, variant, ksplit, persistent):
    import torch
    sets = [oracle.make_inputs(m, n, k, 7100 + i) for i in range(3)]
    da = torch.empty((k, m), dtype=torch.uint8, device="cuda")
    db = torch.empty((k, n), dtype=torch.uint8, device="cuda")
    dsa = torch.empty((k // 128, m), dtype=torch.float32, device="cuda")
    dsb = torch.empty((k // 128, (n + 127) // 128), dtype=torch.float32, device="cuda")
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    pkg.select(kernel)
    pkg.force_config(variant, ksplit)
    pkg.set_persistent(persistent)
    ws = None
    try:
        need = pkg.workspace_bytes(m, n, k)
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            pkg.set_workspace(ws, need)

        def call():
            pkg.gemm(da, db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)

        eager = []
        for a, b, sa, sb in sets:
            for dst, src in ((da, a), (db, b), (dsa, sa), (dsb, sb)):
                _fill(dst, src)
            dc.fill_(-1)
            call()
            torch.cuda.synchronize()
            eager.append(dc.cpu().numpy().copy())
        name = pkg.last_kernel()
        _say(f"[gpu case] graph capture m={m} n={n} k={k} kernel={name}")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call()
        torch.cuda.synchronize()
        for rnd in range(2):
            for i, (a, b, sa, sb) in enumerate(sets):
                for dst, src in ((da, a), (db, b), (dsa, sa), (dsb, sb)):
                    _fill(dst, src)
                dc.fill_(-1)
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                got = dc.cpu().numpy()
                assert np.array_equal(got, eager[i]), (name, "replay", rnd, i)
        ref = oracle.ref_gemm(*sets[2], m, n, k)
        r = oracle.compare_bf16(eager[2].view(np.uint16), ref, 1e-2, 1e-3)
        assert r["bad"] == 0, (name, r)
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
        pkg.set_persistent(-1)
        if ws is not None:
            pkg.set_workspace(None, 0)


def test_quantise_then_gemm_graph_replays_equal_eager(pkg):
    """bf16 activations and weights -> both quantisers -> GEMM, one graph"""
    import torch
    m, n, k = 256, 384, 512
    xs = [(oracle.gen_normal_bf16(m, k, 7200 + i), oracle.gen_normal_bf16(n, k, 7300 + i)) for i in range(3)]

    def bits(x):
        return (np.ascontiguousarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16).view(np.int16)

    dxa = torch.empty((m, k), dtype=torch.int16, device="cuda")
    dxb = torch.empty((n, k), dtype=torch.int16, device="cuda")
    da = torch.empty((k, m), dtype=torch.uint8, device="cuda")
    db = torch.empty((k, n), dtype=torch.uint8, device="cuda")
    dsa = torch.empty((k // 128, m), dtype=torch.float32, device="cuda")
    dsb = torch.empty((k // 128, (n + 127) // 128), dtype=torch.float32, device="cuda")
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")

    def call():
        st = torch.cuda.current_stream().cuda_stream
        pkg.quantize_a_1x128(dxa, da, dsa, m, k, pkg.DTYPE_BF16, st)
        pkg.quantize_b_128x128(dxb, db, dsb, n, k, pkg.DTYPE_BF16, st)
        pkg.gemm(da, db, dsa, dsb, dc, m, n, k, st)

    eager = []
    for xa, xb in xs:
        _fill(dxa, bits(xa))
        _fill(dxb, bits(xb))
        dc.fill_(-1)
        call()
        torch.cuda.synchronize()
        eager.append(dc.cpu().numpy().copy())
    _say(f"[gpu case] graph capture quantise + gemm m={m} n={n} k={k}")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    torch.cuda.synchronize()
    for rnd in range(2):
        for i, (xa, xb) in enumerate(xs):
            _fill(dxa, bits(xa))
            _fill(dxb, bits(xb))
            dc.fill_(-1)
            da.fill_(0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(dc.cpu().numpy(), eager[i]), ("replay", rnd, i)
    a, sa = oracle.quantize_a_1x128(xs[2][0], bf16_arith=True)
    b, sb = oracle.quantize_b_128x128(xs[2][1], bf16_arith=True)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    r = oracle.compare_bf16(eager[2].view(np.uint16), ref, 1e-2, 1e-3)
    assert r["bad"] == 0, r
