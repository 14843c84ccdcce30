"""GPU: the allocation-free matvec entry point (split-k partial sums in the library's static
device array) against qtip_decompress_matvec with a caller workspace, through the C ABI.
The two share their kernels, so the bar is bit-identity; the oracle bounds both."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import c_oracle
from synth import make_layer

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _call_pair(L, m, k, K, nparts=0):
    """(no-alloc result, workspace result) for one seeded matrix, both through the C ABI."""
    from qtip_amd._lib import check, lib, stream_ptr
    lb = lib()
    pk, x, tl = dev(L["packed"]), dev(L["x"].reshape(-1)), dev(L["tlut"])
    st = stream_ptr(pk.device)
    got = torch.full((m,), float("nan"), device="cuda")
    check(lb.qtip_decompress_matvec_noalloc(_p(got), _p(pk), _p(x), _p(tl), m, k, K, nparts, st), "noalloc")
    want = torch.full((m,), float("nan"), device="cuda")
    if nparts == 0:
        ws = torch.empty(16 * m * 4, dtype=torch.uint8, device="cuda")
        check(lb.qtip_decompress_matvec(_p(want), _p(pk), _p(x), _p(tl), m, k, K, _p(ws), ws.numel(), st), "matvec")
    else:
        parts = torch.empty((nparts, m), dtype=torch.float32, device="cuda")
        check(lb.qtip_decompress_matvec_parts(_p(parts), _p(pk), _p(x), _p(tl), m, k, K, nparts, st), "parts")
        want = parts[0].clone()
        for s in range(1, nparts):  # the order in which the library's summing launch adds them
            want += parts[s]
    torch.cuda.synchronize()
    return got, want


def test_noalloc_matches_workspace_entry_point_twice_in_a_row():
    from qtip_amd._lib import lib
    # the larger call first, then a smaller one: the scratch keeps the first call's partial sums
    for (m, k, K) in [(128, 28672, 2), (64, 20480, 3)]:
        assert lib().qtip_matvec_workspace_bytes(m, k, K) > 0, "shape should split k"
        L = make_layer(m, k, K, seed=m + k)
        got, want = _call_pair(L, m, k, K)
        assert torch.equal(got, want)
        ref = c_oracle.matvec(L["packed"], L["x"].reshape(-1), L["tlut"], m, k, K)
        d = np.abs(got.double().cpu().numpy() - ref)
        assert d.max() <= 1e-2 * np.abs(ref).max() and d.mean() <= 1e-3 * np.abs(ref).mean()


@pytest.mark.parametrize("m,k,K,nparts", [(4096, 4096, 2, 2), (2048, 8192, 4, 8), (512, 11008, 3, 5), (4096, 4096, 2, 1)])
def test_noalloc_with_a_given_split(m, k, K, nparts):
    L = make_layer(m, k, K, seed=nparts)
    got, want = _call_pair(L, m, k, K, nparts)
    assert torch.equal(got, want)


def test_noalloc_rejects_what_does_not_fit_and_leaves_out_alone():
    from qtip_amd._lib import lib
    lb = lib()
    m, k, K = 8192, 4096, 2
    L = make_layer(m, k, K, seed=1)
    pk, x, tl = dev(L["packed"]), dev(L["x"].reshape(-1)), dev(L["tlut"])
    out = torch.full((m,), 7.0, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lb.qtip_decompress_matvec_noalloc(_p(out), _p(pk), _p(x), _p(tl), m, k, K, 16, st) == -6  # 16 * 8192 floats
    assert b"scratch" in lb.qtip_error_string(-6)
    assert lb.qtip_decompress_matvec_noalloc(_p(out), _p(pk), _p(x), _p(tl), m, k, K, 17, st) == -1
    assert lb.qtip_decompress_matvec_noalloc(_p(out), _p(pk), _p(x), _p(tl), m, k, K, -1, st) == -1
    torch.cuda.synchronize()
    assert torch.all(out == 7.0)
    assert lb.qtip_decompress_matvec_noalloc(_p(out), _p(pk), _p(x), _p(tl), m, k, K, 8, st) == 0  # 8 * 8192 just fits
    ref = c_oracle.matvec(L["packed"], L["x"].reshape(-1), L["tlut"], m, k, K)
    d = np.abs(out.double().cpu().numpy() - ref)
    assert d.max() <= 1e-2 * np.abs(ref).max()
