"""The per-call entry points (fp8_block_gemm_ex / fp8_block_gemm_ws) on the GPU: own workspace, own
options, no process-wide state -- concurrent use from two host threads on two streams, stream capture
with and without a workspace, operands off the 16-byte grid with a caller's workspace."""
import sys
import threading

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _dev(*arrs):
    import torch
    return [torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in arrs]


def test_two_threads_two_streams_with_their_own_workspaces(pkg):
    """Two different plans that split K run at the same time, each on its own stream with its own
    workspace and options: every result equals the one the same call gives alone."""
    import torch
    jobs = []
    for (m, n, k, opt, seed) in [(256, 256, 2048, pkg.Options(pkg.KERNEL_SPLITK, 2, 4), 8101),
                                 (512, 384, 1024, pkg.Options(pkg.KERNEL_SPLITK, 4, 2), 8102)]:
        a, b, sa, sb = oracle.make_inputs(m, n, k, seed)
        need = pkg.workspace_bytes_ex(m, n, k, opt)
        assert need > 0
        jobs.append(dict(shape=(m, n, k), opt=opt, host=(a, b, sa, sb), dev=_dev(a, b, sa, sb),
                         ws=torch.empty(need, dtype=torch.uint8, device="cuda"), need=need,
                         c=torch.zeros((m, n), dtype=torch.int16, device="cuda"),
                         stream=torch.cuda.Stream()))
    torch.cuda.synchronize()

    def call(j):
        m, n, k = j["shape"]
        pkg.gemm_ex(*j["dev"], j["c"], m, n, k, j["opt"], j["ws"], j["need"], j["stream"].cuda_stream)

    for j in jobs:   # alone
        _say(f"[gpu case] per-call entry point alone {j['shape']}")
        call(j)
        torch.cuda.synchronize()
        j["alone"] = j["c"].cpu().numpy().copy()
        ref = oracle.ref_gemm(*j["host"], *j["shape"])
        assert oracle.compare_bf16(j["alone"].view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    errors = []

    def worker(j, rounds):
        try:
            for _ in range(rounds):
                call(j)
        except Exception as exc:   # reported by the main thread
            errors.append(exc)

    _say("[gpu case] per-call entry point from two threads on two streams")
    for j in jobs:
        j["c"].fill_(-1)
    torch.cuda.synchronize()
    threads = [threading.Thread(target=worker, args=(j, 200)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for j in jobs:
        assert np.array_equal(j["c"].cpu().numpy(), j["alone"]), j["shape"]


def test_capture_without_workspace_is_refused_and_leaves_the_capture_valid(pkg):
    """A plan that needs the process-wide workspace, called while its stream is being captured and
    before that workspace exists: FP8GEMM_E_WORKSPACE, nothing allocated, and the capture goes on."""
    import torch
    m, n, k = 256, 256, 1024
    a, b, sa, sb = oracle.make_inputs(m, n, k, 8201)
    da, db, dsa, dsb = _dev(a, b, sa, sb)
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    dc2 = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    pkg.set_workspace(None, 0)
    pkg.release()                      # no library-owned buffer left
    pkg.select(pkg.KERNEL_LARGE)
    pkg.force_config(2, 0)
    try:
        pkg.gemm(da, db, dsa, dsb, dc, m, n, k, torch.cuda.current_stream().cuda_stream)   # eager, no K split
        torch.cuda.synchronize()
        eager = dc.cpu().numpy().copy()
        _say("[gpu case] capture: K-splitting plan without a workspace")
        refused = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            st = torch.cuda.current_stream().cuda_stream
            try:
                pkg.gemm_ex(da, db, dsa, dsb, dc2, m, n, k, pkg.Options(pkg.KERNEL_SPLITK, 2, 4), None, 0, st)
            except pkg.Fp8GemmError as exc:
                refused = exc.code
            pkg.select(pkg.KERNEL_SPLITK)
            pkg.force_config(2, 4)
            try:
                pkg.gemm(da, db, dsa, dsb, dc2, m, n, k, st)    # process-wide workspace would have to be allocated
            except pkg.Fp8GemmError as exc:
                refused = (refused, exc.code)
            pkg.select(pkg.KERNEL_LARGE)
            pkg.force_config(2, 0)
            pkg.gemm(da, db, dsa, dsb, dc2, m, n, k, st)        # needs no workspace: recorded
        assert refused == (-4, -4), refused
        torch.cuda.synchronize()
        dc2.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dc2.cpu().numpy(), eager)
        # outside a capture the same call allocates and runs
        pkg.select(pkg.KERNEL_SPLITK)
        pkg.force_config(2, 4)
        pkg.gemm(da, db, dsa, dsb, dc2, m, n, k, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert pkg.last_kernel() == "tile128x128_k4"
        ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
        assert oracle.compare_bf16(dc2.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
        pkg.release()


@pytest.mark.parametrize("m,n,k,shift", [(250, 300, 512, 0), (256, 384, 512, 1), (1000, 200, 256, 3)])
def test_padded_plan_with_callers_workspace_eager_and_in_a_graph(pkg, m, n, k, shift):
    """Shapes off the 16 grid, or operands `shift` bytes off a 16-byte boundary, run on padded copies in
    the caller's workspace (sized by the any-alignment query); the launches replay from a graph."""
    import torch
    a, b, sa, sb = oracle.make_inputs(m, n, k, 8300 + m)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)

    def shifted(x):   # the same bytes at an address `shift` elements past an aligned one
        t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
        if shift == 0:
            return t, t
        flat = torch.empty(t.numel() + 64, dtype=t.dtype, device="cuda")
        view = flat[shift:shift + t.numel()].view(t.shape)
        view.copy_(t)
        return view, flat

    (da, _ka), (db, _kb) = shifted(a), shifted(b)
    dsa, dsb = _dev(sa, sb)
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    need = pkg.workspace_bytes_ex(m, n, k, None, True)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _say(f"[gpu case] padded plan with caller workspace m={m} n={n} k={k} shift={shift}")
    if shift or m % 16 or n % 16:   # the figure for aligned operands on the grid would not do
        with pytest.raises(pkg.Fp8GemmError) as ei:
            pkg.gemm_ex(da, db, dsa, dsb, dc, m, n, k, None, ws, 1024, st)
        assert ei.value.code == -4
    pkg.gemm_ex(da, db, dsa, dsb, dc, m, n, k, None, ws, need, st)
    torch.cuda.synchronize()
    name = pkg.last_kernel()
    assert name.startswith("padded_"), name
    eager = dc.cpu().numpy().copy()
    assert oracle.compare_bf16(eager.view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0, name
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pkg.gemm_ex(da, db, dsa, dsb, dc, m, n, k, None, ws, need, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for rnd in range(3):
        dc.fill_(-1)
        ws.fill_(rnd)            # eager work between the replays; the plan rewrites all it reads
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dc.cpu().numpy(), eager), (name, "replay", rnd)


def test_host_launcher_does_not_touch_process_wide_switches(pkg):
    """fp8_gemm_host with a forced family (option 100 + id) leaves the selection alone"""
    m, n, k = 64, 128, 256
    a, b, sa, sb = oracle.make_inputs(m, n, k, 8401)
    af, bf = oracle.e4m3fn_decode(a), oracle.e4m3fn_decode(b)
    ch = np.zeros((m, n), np.uint16)
    pkg.select(pkg.KERNEL_SCALAR)
    try:
        rc = pkg.lib().fp8_gemm_host(ch.ctypes.data, af.ctypes.data, bf.ctypes.data, sa.ctypes.data,
                                     sb.ctypes.data, m, n, k, 100 + pkg.KERNEL_LARGE)
        assert rc == 0
        assert pkg.plan(m, n, k) == "scalar"          # still what this test selected
    finally:
        pkg.select(0)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    assert oracle.compare_bf16(ch, ref, 1e-2, 1e-3)["bad"] == 0


def test_library_owned_workspace_growth_keeps_device_memory_bounded(pkg):
    """K-splitting plans whose need creeps up call by call (a growing batch): the library-owned workspace
    at least doubles when it grows and frees the buffers it has outgrown once their work is done, so the
    memory it holds stays within a small multiple of the largest need instead of the sum of all needs"""
    import torch
    pkg.set_workspace(None, 0)
    pkg.release()
    st = torch.cuda.current_stream().cuda_stream
    m, k = 1024, 512
    shapes = [(m, 1024 + 64 * i, k) for i in range(25)]
    n_max = shapes[-1][1]
    a, b, sa, sb = oracle.make_inputs(m, n_max, k, 8401)
    da, dsa = _dev(a, sa)
    dc = torch.zeros((m, n_max), dtype=torch.int16, device="cuda")
    pkg.select(pkg.KERNEL_SPLITK)
    pkg.force_config(2, 4)
    try:
        needs = [pkg.workspace_bytes(*s) for s in shapes]
        assert needs[0] > 16 << 20 and all(x < y for x, y in zip(needs, needs[1:]))
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _say(f"[gpu case] workspace growth over {len(shapes)} calls, needs {needs[0] >> 20} .. {needs[-1] >> 20} MiB")
        for (mm, n, kk) in shapes:
            bn = np.ascontiguousarray(b[:, :n])
            sbn = np.ascontiguousarray(sb[:, :(n + 127) // 128])
            db, dsb = _dev(bn, sbn)
            pkg.gemm(da, db, dsa, dsb, dc[:, :n].contiguous(), mm, n, kk, st)
            torch.cuda.synchronize()
            del db, dsb
        torch.cuda.empty_cache()
        held = free_before - torch.cuda.mem_get_info()[0]
        _say(f"[gpu case] held after growth: {held >> 20} MiB; sum of needs {sum(needs) >> 20} MiB")
        assert held <= 4 * needs[-1] + (64 << 20), (held, needs[-1])
    finally:
        pkg.select(0)
        pkg.force_config(-1, 0)
    pkg.release()


def test_grouped_per_call_form_from_two_threads_on_two_streams(pkg):
    """fp8_block_gemm_grouped_ex: two grouped calls (decode-sized groups with the K range split inside the
    kernel; ragged taller groups on padded copies) run at the same time, each on its own stream with its own
    zeroed workspace; results equal the ones each call gives alone and the oracle's."""
    import torch
    jobs = []
    for (ms, n, k, seed) in [([16, 64, 32, 48, 16, 16, 64, 32], 1536, 2048, 8601), ([250, 40, 1000], 392, 512, 8602)]:
        host, dev = [], []
        for g, m in enumerate(ms):
            a, b, sa, sb = oracle.make_inputs(m, n, k, seed + 31 * g)
            host.append((a, b, sa, sb))
            dev.append(_dev(a, b, sa, sb))
        opt = pkg.Options(flags=pkg.FLAG_WORKSPACE_ZEROED)
        need = pkg.grouped_workspace_bytes(ms, n, k, opt)
        assert need > pkg.WORKSPACE_HEADER_BYTES
        jobs.append(dict(ms=ms, n=n, k=k, host=host, dev=dev, opt=opt, need=need,
                         ws=torch.zeros(need, dtype=torch.uint8, device="cuda"),
                         outs=[torch.zeros((m, n), dtype=torch.int16, device="cuda") for m in ms],
                         stream=torch.cuda.Stream()))
    torch.cuda.synchronize()

    def call(j):
        d = j["dev"]
        pkg.gemm_grouped_ex([x[0] for x in d], [x[1] for x in d], [x[2] for x in d], [x[3] for x in d], j["outs"],
                            j["ms"], j["n"], j["k"], j["opt"], j["ws"], j["need"], j["stream"].cuda_stream)

    for j in jobs:
        _say(f"[gpu case] grouped per-call entry point alone ms={j['ms']}")
        call(j)
        torch.cuda.synchronize()
        j["name"] = pkg.last_kernel()
        j["alone"] = [c.cpu().numpy().copy() for c in j["outs"]]
        for g, m in enumerate(j["ms"]):
            ref = oracle.ref_gemm(*j["host"][g], m, j["n"], j["k"])
            assert oracle.compare_bf16(j["alone"][g].view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0, (j["name"], g)
    assert jobs[0]["name"].startswith("decode128_k") and not jobs[0]["name"].startswith("decode128_k1_"), jobs[0]["name"]
    assert "padded_" in jobs[1]["name"] and "+" in jobs[1]["name"], jobs[1]["name"]
    errors = []

    def worker(j, rounds):
        try:
            for _ in range(rounds):
                call(j)
        except Exception as exc:
            errors.append(exc)

    _say("[gpu case] grouped per-call entry point from two threads on two streams")
    for j in jobs:
        for c in j["outs"]:
            c.fill_(-1)
    torch.cuda.synchronize()
    threads = [threading.Thread(target=worker, args=(j, 100)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for j in jobs:
        for g in range(len(j["ms"])):
            assert np.array_equal(j["outs"][g].cpu().numpy(), j["alone"][g]), (j["ms"], g)
    # without a workspace the decode-sized groups still run as one launch, unsplit; ragged groups cannot
    j = jobs[0]
    d = j["dev"]
    pkg.gemm_grouped_ex([x[0] for x in d], [x[1] for x in d], [x[2] for x in d], [x[3] for x in d], j["outs"],
                        j["ms"], j["n"], j["k"], None, None, 0, j["stream"].cuda_stream)
    torch.cuda.synchronize()
    assert pkg.last_kernel() == f"decode128_k1_grouped{len(j['ms'])}", pkg.last_kernel()
    for g, m in enumerate(j["ms"]):
        ref = oracle.ref_gemm(*j["host"][g], m, j["n"], j["k"])
        assert oracle.compare_bf16(j["outs"][g].cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    j = jobs[1]
    d = j["dev"]
    with pytest.raises(pkg.Fp8GemmError) as info:
        pkg.gemm_grouped_ex([x[0] for x in d], [x[1] for x in d], [x[2] for x in d], [x[3] for x in d], j["outs"],
                            j["ms"], j["n"], j["k"], None, None, 0, j["stream"].cuda_stream)
    assert info.value.code == -4
    torch.cuda.synchronize()


def test_plan_without_the_header_runs_when_no_workspace_can_be_had(pkg):
    """a shape whose preferred plan adds its K splits inside the kernel (and so needs the workspace header)
    still runs when no workspace is at hand -- a per-call entry without a buffer, the process-wide entry while
    its stream is being captured and nothing is allocated yet -- on the plan that needs none"""
    import torch
    m, n, k = 1024, 512, 2048
    assert pkg.plan(m, n, k) == "tile64x64_k2f"
    a, b, sa, sb = oracle.make_inputs(m, n, k, 8701)
    ref = oracle.ref_gemm(a, b, sa, sb, m, n, k)
    dev = _dev(a, b, sa, sb)
    dc = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _say(f"[gpu case] per-call entry without a workspace m={m} n={n} k={k}")
    pkg.gemm_ex(*dev, dc, m, n, k, pkg.Options(flags=pkg.FLAG_WORKSPACE_ZEROED), None, 0, st)
    torch.cuda.synchronize()
    assert pkg.last_kernel() == "tile64x64_k1", pkg.last_kernel()
    assert oracle.compare_bf16(dc.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    pkg.set_workspace(None, 0)
    pkg.release()
    dc.fill_(-1)
    torch.cuda.synchronize()
    _say("[gpu case] process-wide entry under capture, nothing allocated")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pkg.gemm(*dev, dc, m, n, k, torch.cuda.current_stream().cuda_stream)
        name = pkg.last_kernel()
    assert name == "tile64x64_k1", name
    graph.replay()
    torch.cuda.synchronize()
    assert oracle.compare_bf16(dc.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    del graph
    # with the library's workspace in place the preferred plan runs
    pkg.gemm(*dev, dc, m, n, k, st)
    torch.cuda.synchronize()
    assert pkg.last_kernel() == "tile64x64_k2f", pkg.last_kernel()
    assert oracle.compare_bf16(dc.cpu().numpy().view(np.uint16), ref, 1e-2, 1e-3)["bad"] == 0
    pkg.release()
