"""GPU parity of the packing tools (all through the C ABI) against the numpy oracle: bit-exact."""
import numpy as np
import pytest
import torch

from oracle import qtip_oracle as O

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("m,k", [(32, 32), (64, 96), (256, 512), (2048, 1024)])
def test_repack_both_ways(m, k, K):
    from qtip_amd import ops
    rng = np.random.default_rng(m + k + K)
    nat = rng.integers(0, 65536, size=(m // 16 * k // 16, 16 * K), dtype=np.uint16)
    want = O.repack_for_kernel(nat, m, k, K)
    got = ops.repack(torch.from_numpy(nat.view(np.int16)).to(_dev()), m, k, K, to_kernel=True)
    assert got.shape == (m // 16 * k // 16, 16 * K) and got.dtype == torch.int16
    assert np.array_equal(got.cpu().numpy(), want)
    back = ops.repack(got, m, k, K, to_kernel=False)
    assert np.array_equal(back.cpu().numpy().view(np.uint16), nat)
    assert np.array_equal(back.cpu().numpy().view(np.uint16), O.kernel_to_natural(want, m, k, K))


@pytest.mark.parametrize("K", [2, 3, 4])
def test_repacked_stream_decodes_like_the_natural_one(K):
    """natural -> kernel packing -> fused decode kernel equals the natural decode with the
    quantiser's within-tile order (three statements of the layout agree on the GPU too)."""
    from qtip_amd import ops
    m, k = 128, 256
    rng = np.random.default_rng(K)
    nat = rng.integers(0, 65536, size=(m // 16 * k // 16, 16 * K), dtype=np.uint16)
    tl = rng.standard_normal((512, 2)).astype(np.float16)
    ker = ops.repack(torch.from_numpy(nat.view(np.int16)).to(_dev()), m, k, K)
    W = ops.decode(ker.reshape(-1), torch.from_numpy(tl).to(_dev()), m, k, K).cpu().numpy()
    want = O.decode_natural(nat, O.quantlut_sym(tl), m, k, K, kernel_order=True)
    assert np.array_equal(W.view(np.uint16), want.view(np.uint16))


CASES = [(256, 2, 2), (256, 3, 2), (256, 4, 2), (256, 2, 1), (256, 5, 1), (64, 4, 1), (64, 1, 2), (256, 8, 2)]


@pytest.mark.parametrize("T,K,V", CASES)
def test_unpack_and_pack_states(T, K, V):
    from qtip_amd import ops
    rng = np.random.default_rng(T + 7 * K + V)
    words = rng.integers(0, 65536, size=(37, T * K // 16), dtype=np.uint16)
    dw = torch.from_numpy(words.view(np.int16)).to(_dev())
    st = ops.unpack_trellis(dw, T, K, V)
    assert st.dtype == torch.int32 and st.shape == (37, T // V)
    assert np.array_equal(st.cpu().numpy(), O.unpack_trellis_generic(words, T, K, V))
    pk = ops.pack_trellis(st, K, V)
    assert pk.dtype == torch.uint16
    assert np.array_equal(pk.cpu().numpy(), words)
    assert np.array_equal(pk.cpu().numpy(), O.pack_trellis_generic(st.cpu().numpy(), K, V))


def test_pack_rejects_non_walk_and_bad_shapes():
    from qtip_amd import ops
    st = torch.zeros(3, 128, dtype=torch.int32, device=_dev())
    st[1, 7] = 1 << 15
    with pytest.raises(ValueError, match="trellis walk"):
        ops.pack_trellis(st, 2, 2)
    with pytest.raises(ValueError):
        ops.unpack_trellis(torch.zeros(10, dtype=torch.int16, device=_dev()), 256, 2, 2)   # not whole tiles
    with pytest.raises(ValueError):
        ops.unpack_trellis(torch.zeros(32, dtype=torch.int16, device=_dev()), 250, 2, 2)   # T*K % 16
    with pytest.raises(ValueError):
        ops.unpack_trellis(torch.zeros(32, dtype=torch.int16), 256, 2, 2)                  # host tensor


@pytest.mark.parametrize("mode,V,K,tdx,tdy,dtype", [
    ("quantlut_sym", 2, 2, 16, 16, torch.float16),
    ("quantlut_sym", 2, 3, 16, 16, torch.float32),
    ("quantlut", 2, 4, 16, 16, torch.float16),
    ("quantlut", 1, 2, 16, 16, torch.float32),
    ("lut", 2, 2, 8, 8, torch.float32),
    ("1mad", 1, 2, 16, 16, torch.float32),
    ("2mad", 1, 4, 8, 16, torch.float32),
    ("3inst", 1, 2, 16, 8, torch.float32),
])
def test_decode_natural_all_modes(mode, V, K, tdx, tdy, dtype):
    from qtip_amd import ops
    from qtip_amd.codebook.bitshift import BitshiftLinear
    m, n = 4 * tdx, 6 * tdy
    T = tdx * tdy
    rng = np.random.default_rng(K + tdx)
    words = rng.integers(0, 65536, size=(24, T * K // 16), dtype=np.uint16)
    bits = 16 if mode == "lut" else 9
    mod = BitshiftLinear(tdx, tdy, 16, K, V, bits, mode, has_kernel=False)
    lut = mod.cb.lut.to(dtype).contiguous()
    got = ops.decode_natural(torch.from_numpy(words.view(np.int16)).to(_dev()), lut.to(_dev()), m, n, tdx, tdy, K, V)
    want = O.decode_natural_generic(words, lut.numpy(), m, n, tdx, tdy, K, V)
    assert got.dtype == dtype
    g = got.cpu().numpy()
    assert np.array_equal(g.view(np.uint16 if dtype == torch.float16 else np.uint32),
                          want.view(np.uint16 if dtype == torch.float16 else np.uint32))
    # the module's own accessor gives the same matrix as the reference's two-step route
    mod.cb.lut = lut
    W2 = mod.get_hatW_natural(torch.from_numpy(words.view(np.int16)).to(_dev()), m, n)
    st = mod.cb.unpack_trellis(torch.from_numpy(words.view(np.int16)).to(_dev()), T)
    W3 = mod.get_hatW(st, m, n)
    assert torch.equal(W2, got) and torch.equal(W3.to(dtype), got)


@pytest.mark.parametrize("mode,V", [("quantlut_sym", 2), ("3inst", 1)])
def test_forward_without_fused_kernel(mode, V):
    """has_kernel=False forward (natural packing, any decode mode) against the dense formula."""
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    m, k, K = 128, 256, 2
    rng = np.random.default_rng(5)
    words = rng.integers(0, 65536, size=(m // 16 * k // 16, 256 * K // 16), dtype=np.uint16)
    g = torch.Generator().manual_seed(3)
    tl = torch.randn(512, 2, generator=g).half() if mode == "quantlut_sym" else None
    mod = BitshiftLinear(16, 16, 16, K, V, 9, mode, tlut=tl, has_kernel=False)
    SU = torch.sign(torch.randn(k, generator=g) + 1e-5).half().to(_dev())
    SV = (torch.sign(torch.randn(m, generator=g) + 1e-5) / k**0.5).float().to(_dev())
    x = torch.randn(3, k, generator=g).half().to(_dev())
    hl, Kl = mh.get_hadK(k)
    hr, Kr = mh.get_hadK(m)
    tr = torch.from_numpy(words.view(np.int16)).to(_dev())
    y = mod(x, tr, SU, SV, hl, hr, Kl, Kr, 0, 8).float().cpu().numpy()
    W = O.decode_natural_generic(words, mod.cb.lut.float().numpy(), m, k, 16, 16, K, V).astype(np.float64)
    xt = O.hadamard_transform(x.cpu().numpy().astype(np.float64) * SU.cpu().numpy().astype(np.float64), transpose=True) / 32
    xt = xt.astype(np.float16).astype(np.float64)
    ref = O.hadamard_transform(xt @ W.T) * (SV.cpu().numpy().astype(np.float64) * 32)
    err = np.abs(y - ref)
    assert err.max() <= 1e-2 * np.abs(ref).max() and err.mean() <= 2e-3 * np.abs(ref).mean()
