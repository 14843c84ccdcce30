"""CPU: pins the oracle (oracle/qtip_oracle.py, oracle/qtip_oracle.c) against the
known-answer tests the reference holds, against what the mathematics fixes,
and its independent statements of the packed layout against each other."""
import numpy as np
import pytest
import scipy.linalg

from oracle import c_oracle
from oracle import qtip_oracle as O

RNG = np.random.default_rng(1234)
TLUT = RNG.standard_normal((512, 2)).astype(np.float16)


# ---- a1: HYB hash and table expansion -------------------------------------
def test_hash_known_answers():
    # hand-computed (state -> index, sign): p = s*(s+1), index bits 6..14, sign bit 15
    kat = {0: (0, 0), 1: (0, 0), 7: (0, 0), 8: (1, 0), 0xB5: (2, 1), 0xFF: (508, 1),
           0x100: (4, 0), 0x1234: (435, 0), 0x8000: (0, 1), 0xFFFF: (0, 0)}
    for s, (q, sg) in kat.items():
        qq, ss = O.hyb_hash(np.array([s]))
        assert (int(qq[0]), int(ss[0])) == (q, sg), hex(s)


def test_quantlut_sym_matches_device_form_for_all_states():
    # device statement (inference.cu:349-359): 16-bit product, mask 0x7FC0 for
    # the index, xor of bit 15 into the sign of the low half
    lut = O.quantlut_sym(TLUT)
    tl = TLUT.view(np.uint16)
    s = np.arange(65536, dtype=np.uint32)
    p = (s * (s + 1)) & 0xFFFF
    q = (p & 0x7FC0) >> 6
    lo = tl[q, 0] ^ (p & 0x8000).astype(np.uint16)
    hi = tl[q, 1]
    assert np.array_equal(lut.view(np.uint16)[:, 0], lo)
    assert np.array_equal(lut.view(np.uint16)[:, 1], hi)


def test_quantlut_sym_sign_only_on_element0():
    lut = O.quantlut_sym(np.ones((512, 2), np.float16))
    assert set(np.unique(lut[:, 0])) == {-1.0, 1.0}
    assert np.all(lut[:, 1] == 1.0)


# ---- a2/a4: natural packing ------------------------------------------------
@pytest.mark.parametrize("K", [2, 3, 4])
def test_pack_unpack_roundtrip_and_overlap(K):
    words = RNG.integers(0, 65536, (5, 16 * K), dtype=np.uint16)
    st = O.unpack_trellis_natural(words, K)
    assert st.shape == (5, 128)
    low = (1 << (16 - 2 * K)) - 1
    assert np.all((st[:, :-1] & low) == (st[:, 1:] >> (2 * K)))
    # tail biting: last state's low bits are the first state's high bits
    assert np.all((st[:, -1] & low) == (st[:, 0] >> (2 * K)))
    assert np.array_equal(O.pack_trellis_natural(st, K), words)


def test_pack_rejects_non_trellis():
    st = RNG.integers(0, 65536, (1, 128))
    with pytest.raises(ValueError):
        O.pack_trellis_natural(st, 2)


def test_unpack_hand_example():
    # K=2: stream = 0x1234 0x5678 ...; state0 = 0x1234, state1 = window at bit 4 = 0x2345
    words = np.zeros((1, 32), dtype=np.uint16)
    words[0, 0], words[0, 1] = 0x1234, 0x5678
    st = O.unpack_trellis_natural(words, 2)
    assert st[0, 0] == 0x1234 and st[0, 1] == 0x2345 and st[0, 4] == 0x5678
    assert st[0, 127] == 0x0123  # wraps around to the head


@pytest.mark.parametrize("K", [2, 3, 4])
def test_permute_is_the_mma_fragment_order(K):
    # lib/algo/ldlq.py:10-13 against the explicit formula: sequence position
    # p = 2*s+e, s = 4*lane + j  ->  row lane/4 + 8*(j%2), col 2*(lane%4) + 8*(j/2) + e
    for p in range(256):
        s, e = divmod(p, 2)
        lane, j = divmod(s, 4)
        r = lane // 4 + 8 * (j % 2)
        c = 2 * (lane % 4) + 8 * (j // 2) + e
        assert O.PERMUTE[p] == 16 * r + c


# ---- a3: three descriptions of the kernel packing agree -------------------
@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("shape", [(32, 32), (64, 96), (96, 64)])
def test_decode_cross_consistency(K, shape):
    m, n = shape
    lut = O.quantlut_sym(TLUT)
    nat = RNG.integers(0, 65536, (m // 16 * n // 16, 16 * K), dtype=np.uint16)
    pk = O.repack_for_kernel(nat, m, n, K)
    assert np.array_equal(O.kernel_to_natural(pk, m, n, K), nat)
    a = O.decode_natural(nat, lut, m, n, K, kernel_order=True).view(np.uint16)
    b = O.decode_kernel_tensor(pk, lut, m, n, K).view(np.uint16)
    c = O.decode_kernel_lanes(pk, lut, m, n, K).view(np.uint16)
    d = c_oracle.decode(pk, TLUT, m, n, K).view(np.uint16)
    assert np.array_equal(a, b)
    assert np.array_equal(a, c)
    assert np.array_equal(a, d)


@pytest.mark.parametrize("K", [2, 3, 4])
def test_zero_stream_known_answer(K):
    # qtip-kernels/src/test.cu:23-58: zero bitstream, table of ones, x of ones -> out[i] == k
    m, k = 64, 256
    pk = np.zeros((m // 16 * k // 16, 16 * K), dtype=np.int16)
    ones = np.ones((512, 2), dtype=np.float16)
    w = O.decode_kernel(pk, ones, m, k, K)
    assert np.all(w == 1.0)
    out = O.decompress_matvec(pk, np.ones(k, np.float16), ones, m, k, K)
    assert np.all(out == k)
    assert np.all(c_oracle.matvec(pk, np.ones(k, np.float16), ones, m, k, K) == k)


@pytest.mark.parametrize("K", [2, 3, 4])
def test_single_bit_flip_locality(K):
    # flipping one stream bit changes only the states whose 16-bit circular
    # window covers it: at most ceil(16 / 2K) states = that many weight pairs,
    # all inside one 16x16 tile
    m, n = 32, 32
    lut = O.quantlut_sym(TLUT)
    nat = RNG.integers(0, 65536, (4, 16 * K), dtype=np.uint16)
    base = O.decode_natural(nat, lut, m, n, K, True).view(np.uint16)
    pk0 = O.repack_for_kernel(nat, m, n, K)
    for _ in range(24):
        tile = int(RNG.integers(0, 4))
        bit = int(RNG.integers(0, 256 * K))
        mod = nat.copy()
        mod[tile, bit // 16] ^= np.uint16(1 << (15 - bit % 16))
        pk = O.repack_for_kernel(mod, m, n, K)
        # exactly one bit of the kernel stream differs too
        diff = np.bitwise_xor(pk.view(np.uint16), pk0.view(np.uint16))
        assert sum(bin(int(v)).count("1") for v in diff.reshape(-1)) == 1
        out = O.decode_kernel_lanes(pk, lut, m, n, K).view(np.uint16)
        changed = np.argwhere(out != base)
        assert len(changed) <= 2 * -(-16 // (2 * K))
        if len(changed):
            tm, tn = divmod(tile, 2)
            assert np.all(changed[:, 0] // 16 == tm) and np.all(changed[:, 1] // 16 == tn)
        st0 = O.unpack_trellis_natural(nat, K)
        st1 = O.unpack_trellis_natural(mod, K)
        nchg = int((st0 != st1).sum())
        assert nchg in (16 // (2 * K), -(-16 // (2 * K)))


def test_matvec_equals_dense_product():
    m, k, K = 64, 128, 3
    pk = RNG.integers(-32768, 32768, (m // 16 * k // 16, 16 * K), dtype=np.int16)
    x = RNG.standard_normal(k).astype(np.float16)
    w = O.decode_kernel(pk, TLUT, m, k, K)
    ref = w.astype(np.float64) @ x.astype(np.float64)
    assert np.array_equal(O.decompress_matvec(pk, x, TLUT, m, k, K), ref)
    np.testing.assert_allclose(c_oracle.matvec(pk, x, TLUT, m, k, K), ref, rtol=1e-12, atol=1e-12)


# ---- a7: Hadamard ----------------------------------------------------------
@pytest.mark.parametrize("n", [64, 256, 4096])
def test_fwht_is_sylvester(n):
    x = RNG.standard_normal((2, n))
    np.testing.assert_allclose(O.hadamard_transform(x), x @ scipy.linalg.hadamard(n) / np.sqrt(n), atol=1e-10)


@pytest.mark.parametrize("order", [12, 20, 28, 36, 52, 60, 108, 116, 124, 140, 156, 172])
def test_tables_are_hadamard(order):
    had, K = O.get_hadK(order * 4)
    # 156 and 140 etc. are only reached when no larger order divides n
    h = O._load_tables()[order]
    assert set(np.unique(h)) == {-1.0, 1.0}
    assert np.array_equal(h @ h.T, order * np.eye(order))


def test_known_table_rows():
    # first two rows of the order-12 table as printed in lib/utils/matmul_had.py:131-132
    h = O._load_tables()[12]
    assert h[0].tolist() == [1] + [-1] * 11
    assert h[1].tolist() == [1, 1, -1, 1, -1, -1, -1, 1, 1, 1, -1, 1]
    sym = {o: bool(np.array_equal(O._load_tables()[o], O._load_tables()[o].T)) for o in (12, 20, 28, 172)}
    assert sym == {12: False, 20: False, 28: True, 172: False}


def test_tables_match_the_reference_literals():
    """Every order-K table against tests/golden/had_digests.json: sha256 of the table as the
    reference writes it (lib/utils/matmul_had.py:129-95715), taken by an `ast` parse of that file
    (tests/golden/make_had_digests.py) independent of the reader that produced the .npz.  A row
    permutation, a transposition or a flipped sign changes the digest."""
    import hashlib
    import json
    import os
    import torch
    from qtip_amd.utils import matmul_had as mh
    gold = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "had_digests.json")))
    assert sorted(v["order"] for v in gold.values()) == [12, 20, 28, 36, 52, 60, 108, 116, 124, 140, 156, 172]
    for name, g in gold.items():
        o = g["order"]
        h = O._load_tables()[o]
        assert hashlib.sha256(h.astype(np.int8).tobytes()).hexdigest() == g["sha256"], name
        assert h[0].astype(int).tolist() == g["row0"] and int(h[:, 0].sum()) == g["col0_sum"]
        assert bool(np.array_equal(h, h.T)) == g["symmetric"]
        # the product's own reader of the same file
        hp = 1.0 - 2.0 * mh._table_signs(o).astype(np.float64)
        assert hashlib.sha256(hp.astype(np.int8).tobytes()).hexdigest() == g["sha256"], name
        had, K = mh.get_hadK(o * 8)
        if K == o:  # orders that a larger order does not shadow at this size
            assert hashlib.sha256(had.numpy().astype(np.int8).tobytes()).hexdigest() == g["sha256"]
        hadT, _ = mh.get_hadK(o * 8, transpose=True)
        if K == o:
            assert torch.equal(hadT, had.T)


def test_layer_rounds_the_matmul_result_to_fp16_only_for_more_than_one_row():
    """Hand-built case (synth.rounding_case): output element 0 is 6.0 from the fp32 matvec of a
    single row and 8.0 once the matmul result passes through fp16, as the reference's batched path
    does (lib/codebook/bitshift.py:443-448 against :476-489)."""
    from synth import rounding_case
    L = rounding_case()
    idx, sign = O.hyb_hash(np.array([0x0000, 0x1111]))
    assert idx.tolist() == [0, 336] and sign.tolist() == [0, 0]
    w = O.decode_kernel(L["packed"], L["tlut"], 64, 64, 2).astype(np.float64)
    for r in range(64):
        want = (64.0, 3.0 / 64.0) if r % 32 < 16 else (-64.0, 0.0)
        assert np.all(w[r, 0::2] == want[0]) and np.all(w[r, 1::2] == want[1])
    one, parts = O.bitshift_linear_forward(L["x"], L["packed"], L["SU"], L["SV"], L["tlut"], 2, return_parts=True)
    assert np.all(parts["x4"] == 1.0)
    assert set(np.unique(parts["y0"]).tolist()) == {2049.5, -2048.0}
    assert float(one[0, 0]) == 6.0 and float(one[0, 16]) == 16384.0
    assert np.count_nonzero(one) == 2
    two = O.bitshift_linear_forward(np.repeat(L["x"], 2, axis=0), L["packed"], L["SU"], L["SV"], L["tlut"], 2)
    assert two.shape == (2, 64) and float(two[0, 0]) == 8.0 and float(two[1, 0]) == 8.0
    assert float(two[0, 16]) == 16384.0 and np.count_nonzero(two) == 4


@pytest.mark.parametrize("n,order", [(11008, 172), (12288, 12), (10240, 20), (28672, 28), (22016, 172),
                                     (57344, 28), (4096, 1), (8192, 1)])
def test_get_hadK_factorisation(n, order):
    assert O.get_hadK(n)[1] == order


def test_get_hadK_prefers_first_match_and_rejects():
    assert O.get_hadK(172 * 12 * 0 + 172 * 4)[1] == 172
    assert O.get_hadK(60 * 8)[1] == 60  # 480 is also divisible by 20 and 12
    with pytest.raises(AssertionError):
        O.get_hadK(172 * 3)
    with pytest.raises(AssertionError):
        O.get_hadK(100)


@pytest.mark.parametrize("n", [12 * 8, 20 * 16, 28 * 4, 172 * 2])
def test_general_transform_is_kronecker(n):
    had, K = O.get_hadK(n)
    x = RNG.standard_normal((3, n))
    M = np.kron(had, scipy.linalg.hadamard(n // K)) / np.sqrt(n)
    Mt = np.kron(had.T, scipy.linalg.hadamard(n // K)) / np.sqrt(n)
    np.testing.assert_allclose(O.hadamard_transform(x), x @ M.T, atol=1e-10)
    np.testing.assert_allclose(O.hadamard_transform(x, transpose=True), x @ Mt.T, atol=1e-10)
    # orthogonality: U(Ut(x)) == x and norms are preserved
    np.testing.assert_allclose(O.hadamard_transform(O.hadamard_transform(x, True)), x, atol=1e-10)
    np.testing.assert_allclose(np.linalg.norm(O.hadamard_transform(x), axis=1), np.linalg.norm(x, axis=1))


# ---- a8: layer --------------------------------------------------------------
@pytest.mark.parametrize("m,n,K", [(96, 64, 2), (128, 12 * 32, 3), (20 * 32, 128, 4)])
def test_layer_matches_dense_equivalent(m, n, K):
    from synth import make_layer
    L = make_layer(m, n, K, seed=5, scale=0.05)
    y = O.bitshift_linear_forward(L["x"], L["packed"], L["SU"], L["SV"], L["tlut"], K)
    W = O.dense_equivalent(L["packed"], L["SU"], L["SV"], L["tlut"], K)
    yd = L["x"].astype(np.float64) @ W.T
    # differences: one fp16 rounding of the transformed activation and of the output
    err = np.abs(y.astype(np.float64) - yd).max() / np.abs(yd).max()
    assert err < 5e-3


def test_layer_linearity_in_SV():
    from synth import make_layer
    L = make_layer(64, 64, 2, seed=7, scale=0.05)
    _, p1 = O.bitshift_linear_forward(L["x"], L["packed"], L["SU"], L["SV"], L["tlut"], 2, return_parts=True)
    _, p2 = O.bitshift_linear_forward(L["x"], L["packed"], L["SU"], 2 * L["SV"], L["tlut"], 2, return_parts=True)
    np.testing.assert_allclose(p2["y2"], 2 * p1["y2"], rtol=1e-12)


def test_cpu_baseline_path_decodes_like_the_c_oracle():
    """oracle/torch_cpu_path.py (the code bench.py times as cpu_baseline) against the C
    restatement of the decode, bit for bit, and its matvec against the C matvec."""
    import torch
    from oracle import c_oracle, torch_cpu_path
    from synth import make_layer
    for (m, k, K) in [(64, 96, 2), (32, 256, 3), (128, 64, 4), (256, 1024 + 32, 2)]:
        L = make_layer(m, k, K, seed=m + k + K)
        lut = torch_cpu_path.expand_lut(torch.from_numpy(L["tlut"]))
        w = torch_cpu_path.decode_dense(torch.from_numpy(L["packed"]), lut, m, k, K).numpy()
        ref = c_oracle.decode(L["packed"], L["tlut"], m, k, K)
        assert np.array_equal(w.view(np.uint16), ref.view(np.uint16)), (m, k, K)
        r = torch_cpu_path.time_layer(torch.from_numpy(L["packed"]), torch.from_numpy(L["x"]), torch.from_numpy(L["tlut"]),
                                      m, k, K)
        want = c_oracle.matvec(L["packed"], L["x"].reshape(-1), L["tlut"], m, k, K)
        assert np.abs(r["out"].numpy() - want).max() <= 1e-4 * np.abs(want).max()
