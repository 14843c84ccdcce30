"""GPU: behaviour of the C ABI at its edges - set-up, stream capture, more than one stream."""
import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_first_call_inside_a_capture_is_a_defined_error_then_init_and_capture_work():
    """A process whose very first library call is a launcher on a capturing stream: the launcher
    records nothing and returns QTIP_E_NOT_INIT; after qtip_init() the same capture records, and
    its replays equal the eager result.  (Own process: set-up happens once per process.)"""
    code = textwrap.dedent("""
        import ctypes, sys
        import torch
        sys.path.insert(0, %r)
        from qtip_amd._lib import LIB_PATH
        lb = ctypes.CDLL(LIB_PATH)
        lb.qtip_decompress_matvec.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        m, k, K = 512, 2048, 2
        g = torch.Generator().manual_seed(0)
        pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
        tl = torch.randn(512, 2, generator=g).half().cuda()
        x = torch.randn(k, generator=g).half().cuda()
        out = torch.zeros(m, device="cuda")
        def launch():
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            return lb.qtip_decompress_matvec(out.data_ptr(), pk.data_ptr(), x.data_ptr(), tl.data_ptr(), m, k, K, None, 0, st)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rc_first = launch()
            y = x * 2  # the refused call recorded nothing; keep the capture non-empty
        assert rc_first == -7, rc_first
        assert lb.qtip_init() == 0
        assert launch() == 0
        torch.cuda.synchronize()
        eager = out.clone()
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2):
            assert launch() == 0
        for _ in range(3):
            out.zero_()
            graph2.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
        assert float(eager.abs().max()) > 0
        print("ok")
    """) % ROOT
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "ok" in res.stdout, res.stdout + res.stderr


def test_size_queries_as_first_call_inside_a_capture_run_no_set_up():
    """The size queries may be a process's first library call and may come during a capture: they
    answer from the CU count alone (no hipFuncSetAttribute inside the capture), the capture stays
    valid, and the device still counts as not set up for a launcher in the same capture."""
    code = textwrap.dedent("""
        import ctypes, sys
        import torch
        sys.path.insert(0, %r)
        from qtip_amd._lib import LIB_PATH
        lb = ctypes.CDLL(LIB_PATH)
        lb.qtip_matvec_workspace_bytes.restype = ctypes.c_size_t
        lb.qtip_gemm_workspace_bytes.restype = ctypes.c_size_t
        lb.qtip_decompress_matvec.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        m, k, K = 128, 28672, 2
        g = torch.Generator().manual_seed(0)
        pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
        tl = torch.randn(512, 2, generator=g).half().cuda()
        x = torch.randn(k, generator=g).half().cuda()
        out = torch.zeros(m, device="cuda")
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            split = lb.qtip_matvec_split(m, k, K)
            need = lb.qtip_matvec_workspace_bytes(m, k, K)
            gneed = lb.qtip_gemm_workspace_bytes(m, k, K, 8)
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = lb.qtip_decompress_matvec(out.data_ptr(), pk.data_ptr(), x.data_ptr(), tl.data_ptr(), m, k, K, None, 0, st)
            y = x * 2
        assert split > 1 and need > 0 and need %% (m * 4) == 0 and gneed > 0, (split, need, gneed)
        assert rc == -7, rc
        graph.replay(); torch.cuda.synchronize()
        assert torch.equal(y, x * 2)
        assert lb.qtip_init() == 0
        assert lb.qtip_matvec_split(m, k, K) == split and lb.qtip_matvec_workspace_bytes(m, k, K) == need
        print("ok")
    """) % ROOT
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "ok" in res.stdout, res.stdout + res.stderr


def test_workspace_growth_keeps_the_buffer_a_recorded_graph_writes_to():
    """A graph recorded with the split-k workspace of the moment keeps working after a later,
    larger request replaced that workspace: the old buffer stays allocated."""
    import numpy as np
    import torch
    from oracle import c_oracle
    from qtip_amd import ops
    from synth import make_layer
    m, k, K = 128, 28672, 2
    L = make_layer(m, k, K, seed=3)
    pk, x, tl = (torch.from_numpy(np.ascontiguousarray(L[n])).cuda() for n in ("packed", "x", "tlut"))
    x = x.reshape(-1)
    out = torch.zeros(m, device="cuda")
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        ops.decompress_matvec(pk, x, tl, m, k, K, out=out)  # eager first: allocations happen here
        torch.cuda.synchronize()
        eager = out.clone()
        held = ops._WORKSPACE[(pk.device.index, s.cuda_stream)]
        n_before, old = len(held), held[-1]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            ops.decompress_matvec(pk, x, tl, m, k, K, out=out)
        bigger = ops._workspace(pk.device, old.numel() + 1)
        assert bigger.numel() > old.numel() and len(held) == n_before + 1 and held[-2] is old
        filler = [torch.full((old.numel(),), 0x7F, dtype=torch.uint8, device="cuda") for _ in range(4)]
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
        del filler
    ref = c_oracle.matvec(L["packed"], L["x"].reshape(-1), L["tlut"], m, k, K)
    assert np.abs(eager.double().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()


def test_launchers_on_two_streams_do_not_disturb_each_other():
    """The launchers are re-entrant: matvecs with k-split workspaces, layer transforms and the
    batched product issued alternately on two streams (each stream its own outputs and its own
    workspaces, as the wrappers hand them out) give the results of the same calls issued alone."""
    import torch
    from qtip_amd import ops
    g = torch.Generator().manual_seed(11)
    tl = torch.randn(512, 2, generator=g).half().cuda()
    cases = []
    for m, k, K in ((4096, 4096, 2), (2048, 11008, 3), (10240, 8192, 2), (1024, 28672, 4)):
        pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
        x = torch.randn(k, generator=g).half().cuda()
        X = torch.randn(8, k, generator=g).half().cuda()
        cases.append((pk, x, X, m, k, K))

    def work(c):
        pk, x, X, m, k, K = c
        return (ops.decompress_matvec(pk, x, tl, m, k, K, split_k=True),
                ops.decompress_matvec_parts(pk, x, tl, m, k, K).sum(0),
                ops.decompress_gemm(pk, X, tl, m, k, K))

    alone = [work(c) for c in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [None] * len(cases)
    for rep in range(6):
        for i, c in enumerate(cases):
            with torch.cuda.stream(streams[(i + rep) % 2]):
                got[i] = work(c)
        torch.cuda.synchronize()
        for a, b in zip(alone, got):
            for ta, tb in zip(a, b):
                assert torch.equal(ta, tb)
