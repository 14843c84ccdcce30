"""CPU tests of the packing-tool and decode-mode restatements in the oracle (no GPU needed)."""
import struct

import numpy as np
import pytest
import torch

from oracle import qtip_oracle as O
from qtip_amd.codebook import bitshift as B


def _bitstring_states(words_row, T, K, V):
    """Definition by string slicing: the tile's words as a big-endian bit string, made circular."""
    bits = "".join(format(int(w), "016b") for w in words_row)
    assert len(bits) == T * K
    ext = bits + bits[:16]
    kv = K * V
    return [int(ext[i * kv:i * kv + 16], 2) for i in range(T // V)]


@pytest.mark.parametrize("T,K,V", [(256, 2, 2), (256, 3, 2), (256, 4, 2), (256, 2, 1), (64, 4, 1), (64, 1, 2),
                                   (256, 8, 2)])
def test_generic_unpack_is_the_window_definition(T, K, V):
    rng = np.random.default_rng(T + 10 * K + V)
    words = rng.integers(0, 65536, size=(5, T * K // 16), dtype=np.uint16)
    st = O.unpack_trellis_generic(words, T, K, V)
    for t in range(5):
        assert st[t].tolist() == _bitstring_states(words[t], T, K, V)
    # any circular stream is a valid walk: packing the states gives the stream back
    assert np.array_equal(O.pack_trellis_generic(st, K, V), words)


@pytest.mark.parametrize("K", [2, 3, 4])
def test_generic_equals_16x16_v2_statements(K):
    rng = np.random.default_rng(K)
    words = rng.integers(0, 65536, size=(8, 16 * K), dtype=np.uint16)
    assert np.array_equal(O.unpack_trellis_generic(words, 256, K, 2), O.unpack_trellis_natural(words, K))
    st = O.unpack_trellis_natural(words, K)
    assert np.array_equal(O.pack_trellis_generic(st, K, 2), O.pack_trellis_natural(st, K))
    lut = O.quantlut_sym(rng.standard_normal((512, 2)).astype(np.float16))  # (65536, 2)
    a = O.decode_natural_generic(words, lut.T, 32, 64, 16, 16, K, 2)
    b = O.decode_natural(words, lut, 32, 64, K, kernel_order=False)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_pack_rejects_non_walk():
    st = np.zeros((1, 128), dtype=np.int64)
    st[0, 5] = 1 << 15  # top bit cannot come from the previous state
    with pytest.raises(ValueError):
        O.pack_trellis_generic(st, 2, 2)


def test_decode_natural_generic_places_elements_row_major():
    # one 8x4 tile grid of 2x8 tiles, V=1, lut = identity on the state value
    td_x, td_y, K, V = 2, 8, 2, 1
    m, n = 4, 16
    rng = np.random.default_rng(3)
    words = rng.integers(0, 65536, size=((m // td_x) * (n // td_y), td_x * td_y * K // 16), dtype=np.uint16)
    lut = np.arange(65536, dtype=np.float32)[None]
    W = O.decode_natural_generic(words, lut, m, n, td_x, td_y, K, V)
    st = O.unpack_trellis_generic(words, td_x * td_y, K, V)
    for t in range(words.shape[0]):
        ti, tj = divmod(t, n // td_y)
        for p in range(td_x * td_y):
            assert W[ti * td_x + p // td_y, tj * td_y + p % td_y] == st[t, p]


def _mad_scalar(x, mul, add):
    return (x * mul + add) & 0xFFFFFFFF


def _bytesum_scalar(x):
    return (sum((x >> s) & 255 for s in (0, 8, 16, 24)) - 510) / 147.800537109375


@pytest.mark.parametrize("s", [0, 1, 2, 255, 256, 4660, 32768, 65535])
def test_computed_codes_scalar_known_answers(s):
    assert O.code_1mad(np.array([s]))[0] == np.float32(_bytesum_scalar(_mad_scalar(s, 34038481, 76625530)))
    x = _mad_scalar(s, 264435761, 1013904223)
    x = (((x * 1664525) >> 32) + x) & 0xFFFFFFFF
    assert O.code_2mad(np.array([s]))[0] == np.float32(_bytesum_scalar(x))
    r = (_mad_scalar(s, 89226354, 64248484) & 0x8FFF8FFF) ^ 996162400
    top = struct.unpack("<e", struct.pack("<H", r >> 16))[0]
    bot = struct.unpack("<e", struct.pack("<H", r & 0xFFFF))[0]
    assert O.code_3inst(np.array([s]))[0] == np.float32(np.float16(top) + np.float16(bot))


def test_computed_codes_structure():
    s = np.arange(65536)
    for f in (O.code_1mad, O.code_2mad):
        v = f(s).astype(np.float64) * 147.800537109375
        assert np.allclose(v, np.round(v), atol=1e-3)            # integer byte sums
        assert v.min() >= -510 and v.max() <= 510
        assert abs(f(s).mean()) < 0.02 and abs(f(s).std() - 1) < 0.02
    # byte-sum normalisation: variance of 4 independent uniform bytes
    assert abs(147.800537109375**2 - 4 * (256**2 - 1) / 12) < 1e-2
    v3 = O.code_3inst(s)
    assert np.isfinite(v3).all() and abs(v3.mean()) < 0.02 and np.abs(v3).max() < 8


def test_quantlut_known_answers():
    # index = bits 7..15 of s*(s+1) for a 9-bit table (quantlut_sym uses bits 6..14 and bit 15 as sign)
    tl = np.arange(1024, dtype=np.float32).reshape(512, 2)
    lut = O.quantlut(tl)
    for s, idx in ((0, 0), (1, 0), (11, 1), (0xFF, 510), (0x100, 2), (0x1234, 217), (0xFFFF, 0)):
        assert ((s * (s + 1)) >> 7) & 511 == idx
        assert lut[s, 0] == 2 * idx and lut[s, 1] == 2 * idx + 1


@pytest.mark.parametrize("mode,V,fn", [("1mad", 1, O.code_1mad), ("2mad", 1, O.code_2mad), ("3inst", 1, O.code_3inst)])
def test_codebook_modes_match_oracle(mode, V, fn):
    cb = B.bitshift_codebook(16, 2, V, 0, mode)
    assert cb.lut.shape == (1, 65536)
    assert np.array_equal(cb.lut[0].numpy(), fn(np.arange(65536)))


def test_codebook_quantlut_and_lut_modes():
    g = torch.Generator().manual_seed(1)
    tl = torch.randn(512, 2, generator=g).half()
    cb = B.bitshift_codebook(16, 2, 2, 9, 'quantlut', tlut=tl)
    assert np.array_equal(cb.lut.T.numpy(), O.quantlut(tl.numpy()))
    full = torch.randn(65536, 2, generator=g)
    cb = B.bitshift_codebook(16, 2, 2, 16, 'lut', tlut=full)
    assert torch.equal(cb.lut, full.T)
    for mode, V, bits in (("lut", 2, 16), ("quantlut", 1, 8), ("quantlut", 2, 9), ("quantlut_sym", 2, 9)):
        cb = B.bitshift_codebook(16, 2, V, bits, mode)
        assert cb.lut.shape == (V, 65536) and torch.isfinite(cb.lut).all()
    with pytest.raises(ValueError):
        B.bitshift_codebook(16, 2, 2, 9, '1mad')
    with pytest.raises(ValueError):
        B.bitshift_codebook(16, 2, 2, 9, 'nope')
