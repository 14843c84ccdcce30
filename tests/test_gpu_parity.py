"""GPU: parity of the HIP kernels (called through the C ABI via ctypes) with the
CPU oracle.  Decoded weights must be bit-exact; matvec / GEMM / layer outputs
must meet max-rel <= 1e-2 and mean-rel <= 1e-3 (relative to the largest /
mean magnitude of the oracle's output), the tolerance stated for the path."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import qtip_oracle as O
from synth import make_layer

pytestmark = pytest.mark.gpu

MAX_REL = 1e-2
MEAN_REL = 1e-3


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_errors(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    return d.max() / np.abs(ref).max(), d.mean() / np.abs(ref).mean()


def assert_close(got, ref, max_rel=MAX_REL, mean_rel=MEAN_REL):
    mx, mn = rel_errors(got, ref)
    assert mx <= max_rel and mn <= mean_rel, (mx, mn)


SMALL = [(32, 32), (64, 96), (256, 256), (96, 416), (1024, 4096 + 32)]


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("shape", SMALL)
def test_decode_bit_exact(K, shape):
    from qtip_amd import ops
    m, k = shape
    L = make_layer(m, k, K, seed=m + k + K)
    got = ops.decode(dev(L["packed"]), dev(L["tlut"]), m, k, K).cpu().numpy()
    ref = c_oracle.decode(L["packed"], L["tlut"], m, k, K)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("K", [2, 3, 4])
def test_decode_bit_exact_4096(K):
    from qtip_amd import ops
    m = k = 4096
    L = make_layer(m, k, K, seed=K)
    got = ops.decode(dev(L["packed"]), dev(L["tlut"]), m, k, K).cpu().numpy()
    ref = c_oracle.decode(L["packed"], L["tlut"], m, k, K)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("K", [2, 3, 4])
def test_zero_stream_known_answer(K):
    # qtip-kernels/src/test.cu:23-58 at a reduced size plus the original 8192^2 for K=2
    from qtip_amd import ops
    for m, k in [(64, 256)] + ([(8192, 8192)] if K == 2 else []):
        pk = torch.zeros(m * k * K // 16, dtype=torch.int16, device="cuda")
        ones = torch.ones(512, 2, dtype=torch.float16, device="cuda")
        x = torch.ones(k, dtype=torch.float16, device="cuda")
        out = ops.decompress_matvec(pk, x, ones, m, k, K)
        assert torch.all(out == float(k))
        assert torch.all(ops.decode(pk, ones, m, k, K) == 1.0)


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("shape", SMALL + [(4096, 4096), (4096, 11008), (128, 28672), (64, 20480), (32, 14368),
                                           (96, 28672 - 32)])
@pytest.mark.parametrize("split", [True, False])
def test_matvec_vs_oracle(K, shape, split):
    from qtip_amd import ops
    m, k = shape
    L = make_layer(m, k, K, seed=3 * m + k + K)
    x = L["x"].reshape(-1)
    got = ops.decompress_matvec(dev(L["packed"]), dev(x), dev(L["tlut"]), m, k, K, split_k=split).cpu().numpy()
    ref = c_oracle.matvec(L["packed"], x, L["tlut"], m, k, K)
    assert_close(got, ref)
    # the reference's own check (test_decompress_matvec.py:286-294): fp16, atol 1e-5, rtol 1e-2,
    # on its input scale (codebook and x ~ N(0,1)/16)
    xs = (L["x"].reshape(-1) / 16).astype(np.float16)
    ts = (L["tlut"] / 16).astype(np.float16)
    got2 = ops.decompress_matvec(dev(L["packed"]), dev(xs), dev(ts), m, k, K, split_k=split).cpu().numpy()
    ref2 = c_oracle.matvec(L["packed"], xs, ts, m, k, K)
    np.testing.assert_allclose(got2.astype(np.float16).astype(np.float64), ref2.astype(np.float16).astype(np.float64),
                               atol=1e-5 + 2e-3 * np.abs(ref2).max(), rtol=1e-2)


def test_matvec_deterministic_and_workspace_clean():
    from qtip_amd import ops
    m, k, K = 4096, 4096, 2
    L = make_layer(m, k, K, seed=11)
    pk, x, tl = dev(L["packed"]), dev(L["x"].reshape(-1)), dev(L["tlut"])
    a = ops.decompress_matvec(pk, x, tl, m, k, K)
    for _ in range(5):
        b = ops.decompress_matvec(pk, x, tl, m, k, K)
        assert torch.equal(a, b)


def test_matvec_full_size_properties():
    # 70B-shaped matrix: linearity in x and agreement with a dense product of
    # the HIP-decoded weights (decode itself is bit-exact-tested above)
    from qtip_amd import ops
    m, k, K = 8192, 28672, 2
    g = torch.Generator().manual_seed(0)
    pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
    tl = torch.randn(512, 2, generator=g).half().cuda()
    x1 = torch.randn(k, generator=g).half().cuda()
    w = ops.decode(pk, tl, m, k, K)
    y1 = ops.decompress_matvec(pk, x1, tl, m, k, K)
    ref = (w.double() @ x1.double()).cpu().numpy()
    assert_close(y1.cpu().numpy(), ref)
    y2 = ops.decompress_matvec(pk, (x1 * 2).half(), tl, m, k, K)
    assert torch.allclose(y2, 2 * y1, rtol=1e-5, atol=1e-3)
    # checksum of checksums: column sums of the decoded matrix dotted with x
    np.testing.assert_allclose(float(y1.double().sum()), float((w.double().sum(0) @ x1.double())), rtol=1e-4)


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("shape", [(64, 96), (256, 256), (512, 1024 + 32)])
@pytest.mark.parametrize("batch", [1, 2, 8, 16, 17, 32, 33, 64, 70])
def test_gemm_vs_oracle(K, shape, batch):
    from qtip_amd import ops
    m, k = shape
    L = make_layer(m, k, K, seed=m + k + K + batch)
    rng = np.random.default_rng(batch)
    X = rng.standard_normal((batch, k)).astype(np.float16)
    got = ops.decompress_gemm(dev(L["packed"]), dev(X), dev(L["tlut"]), m, k, K, round_f16=False).cpu().numpy()
    w = c_oracle.decode(L["packed"], L["tlut"], m, k, K).astype(np.float64)
    ref = X.astype(np.float64) @ w.T
    assert_close(got, ref)
    got16 = ops.decompress_gemm(dev(L["packed"]), dev(X), dev(L["tlut"]), m, k, K, round_f16=True).cpu().numpy()
    assert np.array_equal(got16, got.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("K", [2, 4])
@pytest.mark.parametrize("shape", [(128, 4096), (96, 8192 + 64), (160, 2048 + 32), (4096 + 32, 512)])
@pytest.mark.parametrize("batch", [5, 32, 40])
def test_gemm_split_k_and_ragged_groups(K, shape, batch):
    """Few row blocks: k is cut (partials through the workspace, extra summing launch); row-block
    counts that are not a multiple of 4 leave waves of the last group without work."""
    from qtip_amd import ops
    from qtip_amd._lib import lib
    m, k = shape
    if m <= 160 and k >= 4096:
        assert lib().qtip_gemm_workspace_bytes(m, k, K, batch) > 0
    L = make_layer(m, k, K, seed=m + k + K + batch)
    rng = np.random.default_rng(batch)
    X = rng.standard_normal((batch, k)).astype(np.float16)
    pk, xd, tl = dev(L["packed"]), dev(X), dev(L["tlut"])
    ops._workspace(pk.device, 1).fill_(0xFF)  # NaN patterns: a partial result that is never written shows
    got = ops.decompress_gemm(pk, xd, tl, m, k, K, round_f16=False).cpu().numpy()
    w = c_oracle.decode(L["packed"], L["tlut"], m, k, K).astype(np.float64)
    assert_close(got, X.astype(np.float64) @ w.T)
    again = ops.decompress_gemm(pk, xd, tl, m, k, K, round_f16=False).cpu().numpy()
    assert np.array_equal(got, again)  # deterministic
    got16 = ops.decompress_gemm(pk, xd, tl, m, k, K, round_f16=True).cpu().numpy()
    assert np.array_equal(got16, got.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("n", [2, 16, 64, 128, 256, 1024, 4096, 8192, 32768, 131072])
@pytest.mark.parametrize("rows", [1, 3])
def test_rht_pow2(n, rows):
    import qtip_amd.utils.matmul_had  # registers hadamard::hadamard
    from qtip_amd import ops
    rng = np.random.default_rng(n + rows)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    got = ops.rht(dev(x)).cpu().numpy()
    ref = O.hadamard_transform(x)
    assert_close(got, ref, 1e-5, 1e-5)
    got_op = torch.ops.hadamard.hadamard(dev(x), 0.25).cpu().numpy()
    assert_close(got_op, ref * np.sqrt(n) * 0.25, 1e-5, 1e-5)


@pytest.mark.parametrize("n", [12 * 64, 11008, 22016, 12288, 10240, 28672, 57344, 52 * 256])
@pytest.mark.parametrize("transpose", [False, True])
def test_rht_tables(n, transpose):
    from qtip_amd.utils import matmul_had as mh
    rng = np.random.default_rng(n)
    x = rng.standard_normal((2, n)).astype(np.float32)
    hadK, K = mh.get_hadK(n)
    fn = mh.matmul_hadUt_cuda if transpose else mh.matmul_hadU_cuda
    got = fn(dev(x), hadK, K).cpu().numpy()
    assert_close(got, O.hadamard_transform(x, transpose=transpose), 1e-5, 1e-5)
    # caller-supplied table tensor (as QuantizedLinear passes it) gives the same
    got2 = fn(dev(x), hadK.clone().cuda(), K).cpu().numpy()
    assert np.array_equal(got, got2)


def test_rht_fused_sign_scale_and_parts():
    from qtip_amd import ops
    from qtip_amd.utils import matmul_had as mh
    n = 11008
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, n)).astype(np.float32)  # 2 parts, 3 rows
    pre = np.sign(rng.standard_normal(n)).astype(np.float16)
    post = rng.standard_normal(n).astype(np.float32)
    bits = mh.had_bits(None, 172, True, "cuda")
    got = ops.rht(dev(x), order=172, had_bits=bits, pre=dev(pre), post=dev(post), scale=0.5, out_dtype=torch.float16,
                  in_parts=2).cpu().numpy()
    ref = O.hadamard_transform((x[0] + x[1]) * pre.astype(np.float32), transpose=True) * np.sqrt(n) * 0.5 * post
    assert_close(got, ref, 2e-3, 5e-4)  # fp16 output rounding


LAYERS = [(4096, 4096, 2), (4096, 11008, 3), (12288, 4096, 4), (1280, 8192, 2), (256, 28672, 2), (3584, 1024, 2)]


@pytest.mark.parametrize("m,n,K", LAYERS)
@pytest.mark.parametrize("bs", [1, 5])
def test_bitshift_linear_forward(m, n, K, bs):
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    L = make_layer(m, n, K, seed=m + n + K)
    rng = np.random.default_rng(bs)
    inp = rng.standard_normal((bs, n)).astype(np.float16)
    layer = BitshiftLinear(16, 16, 16, K, 2, 9, 'quantlut_sym', tlut=dev(L["tlut"]), has_kernel=True)
    had_l, K_l = mh.get_hadK(n)
    had_r, K_r = mh.get_hadK(m)
    out = layer(dev(inp), dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), had_l, had_r, K_l, K_r, 0, 8)
    assert out.dtype == torch.float16 and out.shape == (bs, m)
    ref = O.bitshift_linear_forward(inp, L["packed"], L["SU"], L["SV"], L["tlut"], K)
    assert_close(out.cpu().numpy(), ref)


def test_layer_rounds_the_matmul_result_to_fp16_only_for_more_than_one_row():
    """The hand-built case of synth.rounding_case on the device: 6.0 for one row (fp32 matvec), 8.0
    for two (the batched product's result passes through fp16, lib/codebook/bitshift.py:476-489)."""
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from synth import rounding_case
    L = rounding_case()
    layer = BitshiftLinear(16, 16, 16, 2, 2, 9, 'quantlut_sym', tlut=dev(L["tlut"]), has_kernel=True)
    args = (dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), None, None, 1, 1, 0, 8)
    one = layer(dev(L["x"]), *args).cpu().numpy()
    assert float(one[0, 0]) == 6.0 and float(one[0, 16]) == 16384.0 and np.count_nonzero(one) == 2
    two = layer(dev(np.repeat(L["x"], 2, axis=0)), *args).cpu().numpy()
    assert float(two[0, 0]) == 8.0 and float(two[1, 0]) == 8.0 and np.count_nonzero(two) == 4
    for bs, want in ((1, 6.0), (2, 8.0), (40, 8.0)):
        ref = O.bitshift_linear_forward(np.repeat(L["x"], bs, axis=0), L["packed"], L["SU"], L["SV"], L["tlut"], 2)
        got = layer(dev(np.repeat(L["x"], bs, axis=0)), *args).cpu().numpy()
        assert float(got[0, 0]) == want and np.array_equal(got, ref)


def test_bitshift_linear_matches_dense_equivalent():
    # the reference's own dense form of the layer (bitshift.py:389-413)
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    m, n, K = 12 * 32, 512, 2
    L = make_layer(m, n, K, seed=2)
    layer = BitshiftLinear(16, 16, 16, K, 2, 9, 'quantlut_sym', tlut=dev(L["tlut"]), has_kernel=True)
    had_l, K_l = mh.get_hadK(n)
    had_r, K_r = mh.get_hadK(m)
    out = layer(dev(L["x"]), dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), had_l, had_r, K_l, K_r, 0, 8)
    W = O.dense_equivalent(L["packed"], L["SU"], L["SV"], L["tlut"], K)
    assert_close(out.cpu().numpy(), L["x"].astype(np.float64) @ W.T)


def test_op_names_and_glue():
    import qtip_amd.codebook as cbk
    m, k, K = 4096, 4096, 2
    L = make_layer(m, k, K, seed=9)
    op = getattr(torch.ops.quip_lib, f"decompress_matvec_qtip_{m}_1_{k}_{K}")
    out = op(dev(L["packed"]), dev(L["x"]).float(), dev(L["tlut"]))  # fp32 x as the reference passes it
    assert out.shape == (1, m) and out.dtype == torch.float32
    ref = c_oracle.matvec(L["packed"], L["x"].reshape(-1), L["tlut"], m, k, K)
    assert_close(out.cpu().numpy().reshape(-1), ref)
    assert len(cbk.kernels) >= 61


def test_matvec_random_shapes_against_the_decoded_matrix():
    """A seeded sweep over 40 random (m, k, bits, split) combinations - ragged k (k / 32 not a
    multiple of 4), k ranges on both sides of the LDS staging limits, splits up to 8 - against
    decoded weights (bit-exact against the oracle elsewhere) times x in fp64."""
    from qtip_amd import ops
    rng = np.random.default_rng(2024)
    for case in range(40):
        K = int(rng.choice([2, 3, 4]))
        m = 32 * int(rng.integers(1, 24))
        k = 32 * int(rng.choice([rng.integers(1, 64), rng.integers(64, 256), rng.integers(448, 900)]))
        nwl = (k // 32 + 3) // 4
        S = int(rng.choice([s for s in (1, 2, 4, 8) if s == 1 or nwl // s >= 16] or [1]))
        g = torch.Generator().manual_seed(case)
        pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
        tl = torch.randn(512, 2, generator=g).half().cuda().reshape(-1)
        x = torch.randn(k, generator=g).half().cuda()
        ref = ops.decode(pk, tl, m, k, K).double() @ x.double()
        parts = ops.decompress_matvec_parts(pk, x, tl, m, k, K, nparts=S)
        got = parts.double().sum(0).reshape(-1)
        err = float((got - ref).abs().max() / ref.abs().max())
        assert err <= 2e-5, (case, m, k, K, S, err)
        full = ops.decompress_matvec(pk, x, tl, m, k, K).double().reshape(-1)
        assert float((full - ref).abs().max() / ref.abs().max()) <= 2e-5, (case, m, k, K)


def test_gemm_random_shapes_against_the_decoded_matrix():
    """Seeded sweep of the batched kernel: 30 random (m, k, bits, batch) combinations, batches on both
    sides of the 16- and 32-row tile limits, against decoded weights times X in fp64 (fp32 results
    and, rounded, the fp16 results the layer uses)."""
    from qtip_amd import ops
    rng = np.random.default_rng(77)
    for case in range(30):
        K = int(rng.choice([2, 3, 4]))
        m = 32 * int(rng.integers(1, 40))
        k = 32 * int(rng.choice([rng.integers(1, 64), rng.integers(64, 300), rng.integers(448, 900)]))
        B = int(rng.choice([2, 7, 8, 15, 16, 17, 31, 32, 33, 50, 64, 70]))
        g = torch.Generator().manual_seed(1000 + case)
        pk = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g).cuda()
        tl = torch.randn(512, 2, generator=g).half().cuda().reshape(-1)
        X = torch.randn(B, k, generator=g).half().cuda()
        ref = X.double() @ ops.decode(pk, tl, m, k, K).double().T
        got = ops.decompress_gemm(pk, X, tl, m, k, K, round_f16=False).double()
        scale = float(ref.abs().max())
        assert got.shape == (B, m) and float((got - ref).abs().max()) <= 2e-5 * scale, (case, m, k, K, B)
        got16 = ops.decompress_gemm(pk, X, tl, m, k, K, round_f16=True).double()
        assert float((got16 - ref).abs().max()) <= 1e-3 * scale, (case, m, k, K, B)


@pytest.mark.parametrize("n", [2048, 4096, 8192, 11008, 12288, 5120])
def test_hadamard_matmul_at_every_row_count_regime(n):
    """matmul_hadU_cuda / matmul_hadUt_cuda pick their route by the number of rows (one vector,
    a few rows, one workgroup per row, library GEMMs for the large table orders): every regime and
    its neighbours against the fp64 Kronecker product of the table and the Sylvester matrix."""
    import scipy.linalg
    from qtip_amd.utils.matmul_had import get_hadK, matmul_hadU_cuda, matmul_hadUt_cuda
    hadK, K = get_hadK(n)
    p = n // K
    Hp = torch.from_numpy(scipy.linalg.hadamard(p).astype(np.float64)).cuda()
    Hk = hadK.double().cuda() if K > 1 else torch.ones(1, 1, dtype=torch.float64).cuda()
    g = torch.Generator().manual_seed(n)
    for rows in (1, 7, 8, 9, 40, 95, 96, 130):
        x = torch.randn(rows, n, generator=g).cuda()
        x3 = x.double().view(rows, K, p)
        for fn, M in ((matmul_hadU_cuda, Hk), (matmul_hadUt_cuda, Hk.T)):
            ref = (torch.einsum("ij,rjp->rip", M, x3) @ Hp).reshape(rows, n) * n**-0.5
            got = fn(x, hadK.cuda() if K > 1 else None, K)
            assert got.shape == x.shape and got.dtype == x.dtype
            assert float((got.double() - ref).abs().max()) <= 1e-5 * float(ref.abs().max()), (n, rows, fn.__name__)


def test_errors_raise_not_exit():
    from qtip_amd import ops
    L = make_layer(64, 64, 2)
    pk, tl, x = dev(L["packed"]), dev(L["tlut"]), dev(L["x"].reshape(-1))
    with pytest.raises(ValueError):
        ops.decompress_matvec(pk, x, tl, 64, 96, 2)  # size mismatch
    with pytest.raises(ValueError):
        ops.decompress_matvec(pk, x, tl, 64, 64, 5)
    with pytest.raises(TypeError):
        ops.decompress_matvec(pk, x.float(), tl, 64, 64, 2)
    with pytest.raises(ValueError):
        ops.decompress_matvec(pk.cpu(), x, tl, 64, 64, 2)
    with pytest.raises(ValueError):
        ops.decode(pk, tl[:100], 64, 64, 2)
    with pytest.raises(ValueError):
        ops.rht(torch.zeros(3, 100, device="cuda"))
    # the launches with a transform in their prologue take a closed set of sizes
    su = torch.ones(64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.decompress_matvec_parts_rht(pk, x, su, 0.1, tl, 64, 64, 2)  # k not in {2048, 4096, 8192}
    kc = torch.zeros(1, 2, 16, 256, dtype=torch.float16, device="cuda")
    inv = torch.ones(128, device="cuda")
    from qtip_amd._lib import QtipLibraryError
    with pytest.raises(QtipLibraryError):  # head size 256 has no transform prologue (refused by the library)
        ops.decode_attention_rht(torch.zeros(1, 8 * 256, device="cuda"), None, 1.0, None, 1, kc, kc.clone(),
                                 torch.tensor([0], device="cuda"), inv, 4, 2, 256)
    with pytest.raises(ValueError):  # a grouped launch takes one to three matrices
        ops.decompress_matvec_group_chain([], [], [], 2048, 2, torch.zeros(1, 2048, device="cuda"),
                                          torch.ones(2048, device="cuda"), 1.0,
                                          torch.zeros(1, 2048, dtype=torch.float16, device="cuda"),
                                          torch.ones(2048, dtype=torch.float16, device="cuda"), 1e-5, [], 1.0)
    with pytest.raises(ValueError):  # one `post` vector per row
        ops.rht_post_rows(torch.zeros(1, 2, 256, device="cuda"), torch.ones(256, device="cuda"))
    kc = torch.zeros(1, 2, 16, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):  # table order without its sign bits
        ops.decode_attention_rht(torch.zeros(1, 12 * 128, device="cuda"), None, 1.0, None, 12, kc, kc.clone(),
                                 torch.tensor([0], device="cuda"), inv[:64], 8, 2, 128)


def test_graph_capture_replays():
    # the forward path must be capturable (no allocation-free requirement on
    # torch's side: outputs come from the graph's private pool)
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    m, n, K = 4096, 4096, 2
    L = make_layer(m, n, K, seed=4)
    layer = BitshiftLinear(16, 16, 16, K, 2, 9, 'quantlut_sym', tlut=dev(L["tlut"]), has_kernel=True)
    had_l, K_l = mh.get_hadK(n)
    had_r, K_r = mh.get_hadK(m)
    args = (dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), had_l, had_r, K_l, K_r, 0, 8)
    static_in = dev(L["x"]).clone()
    eager = layer(static_in, *args).clone()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            layer(static_in, *args)
    torch.cuda.current_stream().wait_stream(s)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        static_out = layer(static_in, *args)
    for it in range(4):
        xin = dev(L["x"]) * (it + 1)
        static_in.copy_(xin)
        g.replay()
        torch.cuda.synchronize()
        ref = layer(xin, *args)
        torch.cuda.synchronize()
        assert torch.equal(static_out, ref), it
    assert torch.equal(layer(dev(L["x"]), *args), eager)


# ---- fused transform prologues / epilogue and the decode attention kernel ----
def _f16(a):
    return np.asarray(a, dtype=np.float16)


@pytest.mark.parametrize("n", [4096, 8192, 1024])
def test_rht_fused_rmsnorm(n):
    # fp16(w * fp16(x * rsqrt(mean(x^2) + eps))) (model/llama.py:129-135), then the input transform
    from qtip_amd import ops
    rng = np.random.default_rng(n)
    x = _f16(rng.standard_normal((1, n)))
    w = _f16(1 + 0.1 * rng.standard_normal(n))
    su = _f16(np.sign(rng.standard_normal(n)))
    eps = 1e-5
    got = ops.rht(dev(x), pre=dev(su), scale=(n**-0.5) / 32, out_dtype=torch.float16, pre_mode=ops.PRE_RMSNORM,
                  norm_weight=dev(w), eps=eps).cpu().numpy()
    xf = x.astype(np.float32)
    h = _f16(xf * (1.0 / np.sqrt((xf.astype(np.float64)**2).mean() + eps)).astype(np.float32))
    normed = _f16(w.astype(np.float32) * h.astype(np.float32))
    ref = O.hadamard_transform(normed.astype(np.float32) * su.astype(np.float32), transpose=True) / 32
    assert_close(got, ref, 3e-3, 1e-3)


def test_rht_fused_silu_mul_and_residual():
    from qtip_amd import ops
    from qtip_amd.utils import matmul_had as mh
    n = 11008
    rng = np.random.default_rng(1)
    ug = _f16(rng.standard_normal((1, 2 * n)))
    su = _f16(np.sign(rng.standard_normal(n)))
    bits = mh.had_bits(None, 172, True, "cuda")
    got = ops.rht(dev(ug), order=172, had_bits=bits, pre=dev(su), scale=(n**-0.5) / 32, out_dtype=torch.float16,
                  pre_mode=ops.PRE_SILU_MUL).cpu().numpy()
    g, u = ug[0, :n].astype(np.float32), ug[0, n:].astype(np.float32)
    act = _f16(_f16(g / (1 + np.exp(-g))).astype(np.float32) * u)
    ref = O.hadamard_transform(act.astype(np.float32)[None] * su.astype(np.float32), transpose=True) / 32
    assert_close(got, ref, 3e-3, 1e-3)
    # output transform with the residual addition folded in, from two split-k partial vectors
    m = 4096
    parts = rng.standard_normal((2, 1, m)).astype(np.float32)
    sv = (rng.standard_normal(m) * 0.05).astype(np.float32)
    res = _f16(rng.standard_normal((1, m)))
    got = ops.rht(dev(parts), post=dev(sv), scale=(m**-0.5) * 32, out_dtype=torch.float16, in_parts=2,
                  residual=dev(res)).cpu().numpy()
    y = _f16(O.hadamard_transform(parts[0] + parts[1]) * 32 * sv)
    ref = _f16(res.astype(np.float32) + y.astype(np.float32))
    assert_close(got, ref, 3e-3, 1e-3)


@pytest.mark.parametrize("heads,kv_heads,pos", [(32, 32, 0), (32, 32, 130), (32, 8, 77), (8, 8, 511)])
def test_decode_attention(heads, kv_heads, pos):
    # RoPE (model/llama.py:264-295) + cache write + attention over slots 0..pos, against torch in fp32
    from qtip_amd import ops
    D, max_len = 128, 512
    g = torch.Generator().manual_seed(pos + heads)
    qkv = torch.randn((heads + 2 * kv_heads) * D, generator=g).half().cuda()
    kc = (torch.randn(1, kv_heads, max_len, D, generator=g) * 0.5).half().cuda()
    vc = torch.randn(1, kv_heads, max_len, D, generator=g).half().cuda()
    kc0, vc0 = kc.clone(), vc.clone()
    inv_freq = (1.0 / (10000.0**(torch.arange(0, D, 2).float() / D))).cuda()
    p = torch.tensor([pos], device="cuda")
    out = ops.decode_attention(qkv, kc, vc, p, inv_freq, heads, kv_heads, D)
    # reference
    q = qkv[:heads * D].view(heads, D).float()
    k = qkv[heads * D:(heads + kv_heads) * D].view(kv_heads, D).float()
    v = qkv[(heads + kv_heads) * D:].view(kv_heads, D)
    ang = pos * inv_freq
    cos = torch.cat([ang.cos(), ang.cos()]).half().float()
    sin = torch.cat([ang.sin(), ang.sin()]).half().float()

    def rope(t):
        rot = torch.cat([-t[:, D // 2:], t[:, :D // 2]], dim=1)
        return ((t * cos).half().float() + (rot * sin).half().float()).half()

    qe, ke = rope(q), rope(k)
    kc0[0, :, pos] = ke
    vc0[0, :, pos] = v
    # cache rows written as the reference would (cos/sin come from the device's cosf/sinf, so a
    # rotated key may differ from torch's by an fp16 ulp); everything else untouched
    assert torch.equal(vc, vc0)
    assert torch.allclose(kc.float(), kc0.float(), atol=4e-3, rtol=2e-3)
    untouched = torch.ones(max_len, dtype=torch.bool)
    untouched[pos] = False
    assert torch.equal(kc[0][:, untouched], kc0[0][:, untouched])
    rep = heads // kv_heads
    kk = kc0[0, :, :pos + 1].float().repeat_interleave(rep, dim=0)
    vv = vc0[0, :, :pos + 1].float().repeat_interleave(rep, dim=0)
    sc = torch.einsum("hd,htd->ht", qe.float(), kk) / D**0.5
    ref = torch.einsum("ht,htd->hd", sc.softmax(-1), vv).reshape(-1)
    assert_close(out.float().cpu().numpy(), ref.cpu().numpy(), 5e-3, 2e-3)


@pytest.mark.parametrize("heads,kv_heads,D,pos,splits", [(32, 32, 128, 1000, 8), (32, 32, 128, 4000, 8),
                                                          (32, 32, 128, 4095, 16), (64, 8, 128, 4000, 4),
                                                          (8, 8, 64, 3000, 8), (32, 32, 128, 5, 8),
                                                          (32, 32, 128, 511, 8), (32, 32, 128, 512, 8),
                                                          (16, 4, 128, 2047, 2)])
def test_decode_attention_over_key_ranges(heads, kv_heads, D, pos, splits):
    """Long contexts: the keys of a head cut into ranges (one workgroup each) and combined by a
    second launch, against a float32 attention over the same cache (model/llama.py:866-880) and
    against the one-workgroup form; ranges past the last key are empty (short context, many ranges)."""
    from qtip_amd import ops
    max_len = 4096
    g = torch.Generator().manual_seed(pos + heads + splits)
    qkv = torch.randn((heads + 2 * kv_heads) * D, generator=g).half().cuda()
    kc = (torch.randn(1, kv_heads, max_len, D, generator=g) * 0.5).half().cuda()
    vc = torch.randn(1, kv_heads, max_len, D, generator=g).half().cuda()
    kc1, vc1 = kc.clone(), vc.clone()
    inv_freq = (1.0 / (10000.0**(torch.arange(0, D, 2).float() / D))).cuda()
    p = torch.tensor([pos], device="cuda")
    one = ops.decode_attention(qkv, kc1, vc1, p, inv_freq, heads, kv_heads, D)
    out = ops.decode_attention(qkv, kc, vc, p, inv_freq, heads, kv_heads, D, key_splits=splits)
    assert torch.equal(kc, kc1) and torch.equal(vc, vc1)  # the same cache rows written once
    # float32 reference on the cache as the kernel left it (row `pos` holds the rotated new key)
    q = qkv[:heads * D].view(heads, D).float()
    ang = pos * inv_freq
    cos = torch.cat([ang.cos(), ang.cos()]).half().float()
    sin = torch.cat([ang.sin(), ang.sin()]).half().float()
    rot = torch.cat([-q[:, D // 2:], q[:, :D // 2]], dim=1)
    qe = ((q * cos).half().float() + (rot * sin).half().float()).half().float()
    rep = heads // kv_heads
    kk = kc[0, :, :pos + 1].float().repeat_interleave(rep, dim=0)
    vv = vc[0, :, :pos + 1].float().repeat_interleave(rep, dim=0)
    sc = torch.einsum("hd,htd->ht", qe, kk) / D**0.5
    ref = torch.einsum("ht,htd->hd", sc.softmax(-1), vv).reshape(-1)
    assert_close(out.float().cpu().numpy(), ref.cpu().numpy(), 5e-3, 2e-3)
    assert_close(out.float().cpu().numpy(), one.float().cpu().numpy(), 5e-3, 2e-3)
    with pytest.raises(ValueError):
        ops.decode_attention(qkv, kc, vc, p, inv_freq, heads, kv_heads, D, key_splits=17)


def test_generate_switches_to_key_ranges_inside_a_run():
    """A run that crosses ops.ATTN_SPLIT_FROM records its step again with the key-range attention
    and keeps decoding the tokens of the eager loop; a short run stays on the one-workgroup form."""
    from qtip_amd import ops
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=1024, heads=8, kv_heads=8, layers=2, ffn=172 * 16, vocab=512)
    T = ops.ATTN_SPLIT_FROM
    assert ops.attention_key_splits(T - 1) == 1 and ops.attention_key_splits(T) == 8
    ids = torch.randint(0, cfg.vocab, (1, T - 4), generator=torch.Generator().manual_seed(4)).cuda()
    model = LlamaDecoder(cfg, max_cache_len=T + 64)
    a, _, _ = generate(model, ids, 10, use_graph=True)
    assert model.cfg.attn_key_splits == 8  # crossed inside the run
    b, _, _ = generate(LlamaDecoder(cfg, max_cache_len=T + 64), ids, 10, use_graph=False)
    assert a.shape == (1, 10) and torch.equal(a, b)
    short, _, _ = generate(model, ids[:, :20], 4)
    assert model.cfg.attn_key_splits == 1 and short.shape == (1, 4)


@pytest.mark.parametrize("heads,kv_heads,D,S", [(32, 32, 128, 1), (64, 8, 128, 2), (8, 8, 128, 3), (16, 16, 64, 1),
                                                 (4, 2, 128, 2), (4, 2, 64, 5), (56, 8, 128, 1)])
def test_decode_attention_with_output_transform_in_prologue(heads, kv_heads, D, S):
    """Attention on the qkv projection's raw partial sums == output transform (a launch of its
    own, checked against the oracle elsewhere) followed by attention: the same fp16 q/k/v up to the
    summation order of the transform, so caches and outputs agree to fp16 rounding."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits
    n = (heads + 2 * kv_heads) * D
    max_len, pos = 256, 77
    g = torch.Generator().manual_seed(n + S)
    parts = (torch.randn(S, n, generator=g) * 0.3).cuda()
    post = (torch.sign(torch.randn(n, generator=g) + 1e-5) * (1.0 + 0.1 * torch.rand(n, generator=g))).cuda()
    hadK, order = get_hadK(n)
    bits = had_bits(hadK, order, False, "cuda") if order > 1 else None
    scale = n**-0.5
    kc = (torch.randn(1, kv_heads, max_len, D, generator=g) * 0.5).half().cuda()
    vc = torch.randn(1, kv_heads, max_len, D, generator=g).half().cuda()
    kc1, vc1 = kc.clone(), vc.clone()
    inv_freq = (1.0 / (10000.0**(torch.arange(0, D, 2).float() / D))).cuda()
    p = torch.tensor([pos], device="cuda")
    qkv = ops.rht(parts if S > 1 else parts.reshape(1, n), order=order, had_bits=bits, post=post, scale=scale,
                  out_dtype=torch.float16, in_parts=S)
    ref = ops.decode_attention(qkv.reshape(-1), kc, vc, p, inv_freq, heads, kv_heads, D)
    got = ops.decode_attention_rht(parts, post, scale, bits, order, kc1, vc1, p, inv_freq, heads, kv_heads, D)
    assert torch.allclose(kc1.float(), kc.float(), atol=2e-3, rtol=2e-3)
    assert torch.allclose(vc1.float(), vc.float(), atol=2e-3, rtol=2e-3)
    assert_close(got.float().cpu().numpy(), ref.float().cpu().numpy(), 5e-3, 1e-3)


@pytest.mark.parametrize("heads,kv_heads,D,S", [(32, 32, 128, 1), (64, 8, 128, 2), (24, 24, 128, 3), (16, 4, 64, 1),
                                                 (40, 40, 128, 2)])
def test_decode_attention_with_three_output_transforms_in_prologue(heads, kv_heads, D, S):
    """Separate q / k / v projections: attention on the three raw partial-sum vectors (column
    ranges of one buffer) == the three output transforms as launches of their own, then attention."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits
    ns = [heads * D, kv_heads * D, kv_heads * D]
    max_len, pos = 128, 33
    g = torch.Generator().manual_seed(sum(ns) + S)
    buf = (torch.randn(S, sum(ns), generator=g) * 0.3).cuda()
    offs = [0, ns[0], ns[0] + ns[1]]
    parts = [buf[:, o:o + n] for o, n in zip(offs, ns)]
    posts = [(torch.sign(torch.randn(n, generator=g) + 1e-5) * (1.0 + 0.1 * torch.rand(n, generator=g))).cuda()
             for n in ns]
    orders, bits, scales, vecs = [], [], [], []
    for p, post, n in zip(parts, posts, ns):
        hadK, order = get_hadK(n)
        b = had_bits(hadK, order, False, "cuda") if order > 1 else None
        orders.append(order)
        bits.append(b)
        scales.append(n**-0.5)
        pc = p.contiguous()
        vecs.append(ops.rht(pc if S > 1 else pc.reshape(1, n), order=order, had_bits=b, post=post, scale=n**-0.5,
                            out_dtype=torch.float16, in_parts=S).reshape(-1))
    kc = (torch.randn(1, kv_heads, max_len, D, generator=g) * 0.5).half().cuda()
    vc = torch.randn(1, kv_heads, max_len, D, generator=g).half().cuda()
    kc1, vc1 = kc.clone(), vc.clone()
    inv_freq = (1.0 / (10000.0**(torch.arange(0, D, 2).float() / D))).cuda()
    p = torch.tensor([pos], device="cuda")
    ref = ops.decode_attention(torch.cat(vecs), kc, vc, p, inv_freq, heads, kv_heads, D)
    got = ops.decode_attention_rht3(parts, posts, scales, bits, orders, kc1, vc1, p, inv_freq, heads, kv_heads, D)
    assert torch.allclose(kc1.float(), kc.float(), atol=2e-3, rtol=2e-3)
    assert torch.allclose(vc1.float(), vc.float(), atol=2e-3, rtol=2e-3)
    assert_close(got.float().cpu().numpy(), ref.float().cpu().numpy(), 5e-3, 1e-3)


def test_fused_decode_with_layer_boundaries_in_the_matvec():
    """Hidden size 2048: the o -> up/gate and down -> next qkv boundaries run inside the following
    matvec launch (8 launches per layer); same logits and caches as the module-by-module forward."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder
    cfg = LlamaConfig(hidden=2048, heads=16, kv_heads=16, layers=3, ffn=172 * 16, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64)
    ids = torch.randint(0, cfg.vocab, (1, 5), generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(5, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([5], device="cuda")
        a = model(tok, pos)
        kc = [c.clone() for c in model.k_cache]
        b = model.decode_fused(tok, pos)
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    for c0, c1 in zip(kc, model.k_cache):
        assert torch.allclose(c0.float(), c1.float(), atol=2e-2)


@pytest.mark.parametrize("n,rows", [(11008, 40), (22016, 33), (28672, 32), (14336, 64), (57344, 32)])
@pytest.mark.parametrize("transpose", [False, True])
def test_transform_of_many_rows_through_gemms(n, rows, transpose):
    """Large table order, many rows: the transform as library GEMMs (the reference's own
    formulation) against the transform kernel, fp32, <= 1e-5 of the largest value."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits, rht_many_rows
    g = torch.Generator().manual_seed(n + rows)
    x = torch.randn(rows, n, generator=g).cuda()
    pre = torch.sign(torch.randn(n, generator=g) + 1e-5).half().cuda()
    post = (torch.sign(torch.randn(n, generator=g) + 1e-5) * (0.5 + torch.rand(n, generator=g))).cuda()
    hadK, K = get_hadK(n)
    ref = ops.rht(x, order=K, had_bits=had_bits(hadK, K, transpose, "cuda"), pre=pre, post=post, scale=n**-0.5 * 2)
    got = rht_many_rows(x, hadK.cuda(), K, transpose, pre=pre, post=post, scale=n**-0.5 * 2)
    assert got.shape == ref.shape and got.dtype == ref.dtype
    assert float((got - ref).abs().max()) <= 1e-5 * float(ref.abs().max())


@pytest.mark.parametrize("n", [2048, 4096, 8192])
@pytest.mark.parametrize("rows,S", [(8, 1), (33, 1), (9, 3), (300, 1)])
@pytest.mark.parametrize("dt_in,dt_out", [(torch.float16, torch.float16), (torch.float32, torch.float16),
                                          (torch.float32, torch.float32), (torch.float16, torch.float32)])
def test_transform_of_many_power_of_two_rows(n, rows, S, dt_in, dt_out):
    """From 8 rows on a power-of-two transform runs one workgroup per row; against the fp64
    Sylvester matrix (what the oracle's transform is pinned to) and the single-row forms."""
    from qtip_amd import ops
    import scipy.linalg
    if S > 1 and dt_in != torch.float32:
        pytest.skip("partial sums are fp32")
    g = torch.Generator().manual_seed(n + rows + S)
    x = torch.randn(S, rows, n, generator=g).to(dt_in).cuda() if S > 1 else torch.randn(rows, n, generator=g).to(dt_in).cuda()
    pre = torch.sign(torch.randn(n, generator=g) + 1e-5).half().cuda()
    post = (torch.sign(torch.randn(n, generator=g) + 1e-5) * (0.5 + torch.rand(n, generator=g))).cuda()
    got = ops.rht(x, pre=pre, post=post, scale=n**-0.5, out_dtype=dt_out, in_parts=S)
    assert got.shape == (rows, n) and got.dtype == dt_out
    xs = x.double().sum(0) if S > 1 else x.double()
    H = torch.from_numpy(scipy.linalg.hadamard(n).astype(np.float64)).cuda()
    ref = ((xs * pre.double()) @ H) * n**-0.5 * post.double()
    tol = 2e-3 if dt_out == torch.float16 else 1e-5
    assert float((got.double() - ref).abs().max()) <= tol * float(ref.abs().max())
    one = ops.rht(x[:, :1].contiguous() if S > 1 else x[:1], pre=pre, post=post, scale=n**-0.5, out_dtype=dt_out, in_parts=S)
    assert float((got[:1].double() - one.double()).abs().max()) <= tol * float(ref.abs().max())


def test_output_transforms_of_several_layers_in_one_launch():
    """rht_post_rows == one qtip_rht per row with that row's post vector, bit for bit."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits
    for n, rows, S in ((11008, 2, 1), (4096, 3, 2), (28672, 2, 2), (1024, 5, 1)):
        g = torch.Generator().manual_seed(n + rows)
        parts = torch.randn(S, rows, n, generator=g).cuda()
        post = (torch.sign(torch.randn(rows, n, generator=g) + 1e-5) * (0.5 + torch.rand(rows, n, generator=g))).cuda()
        hadK, order = get_hadK(n)
        bits = had_bits(hadK, order, False, "cuda") if order > 1 else None
        got = ops.rht_post_rows(parts, post, order=order, had_bits=bits, scale=n**-0.5 * 32)
        for r in range(rows):
            one = ops.rht(parts[:, r].contiguous() if S > 1 else parts[0, r:r + 1].contiguous(), order=order,
                          had_bits=bits, post=post[r].contiguous(), scale=n**-0.5 * 32, out_dtype=torch.float16,
                          in_parts=S)
            assert torch.equal(got[r], one.reshape(-1)), (n, r)


def test_gate_up_output_transforms_with_silu_in_one_launch():
    """rht_silu_pair == the output transform(s) of gate and up followed by the SiLU * up prologue
    of the next input transform: the transformed vector that the down projection reads is
    bit-identical either way, and the paired values match fp16(silu(g)) * u computed in fp64."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits
    for two, n, S in ((False, 22016, 1), (False, 57344, 2), (False, 27648, 3), (False, 106496, 1),
                      (True, 11008, 2), (True, 28672, 1), (True, 13824, 1), (True, 8192, 2), (True, 53248, 2)):
        g = torch.Generator().manual_seed(n + S)
        shape = (S, 2, n) if two else (S, n)
        parts = (torch.randn(shape, generator=g) * 0.7).cuda()
        post = (torch.sign(torch.randn(shape[1:], generator=g) + 1e-5) * (0.5 + torch.rand(shape[1:], generator=g))).cuda()
        hadK, order = get_hadK(n)
        bits = had_bits(hadK, order, False, "cuda") if order > 1 else None
        assert ops.rht_silu_pair_ok(n, order, two), (n, order, two)
        scale = n**-0.5 * 8
        h = ops.rht_silu_pair(parts, post, order=order, had_bits=bits, scale=scale)
        if two:
            gu = ops.rht_post_rows(parts, post, order=order, had_bits=bits, scale=scale).reshape(1, -1)
        else:
            gu = ops.rht(parts if S > 1 else parts.reshape(1, n), order=order, had_bits=bits, post=post, scale=scale,
                         out_dtype=torch.float16, in_parts=S)
        nh = h.numel()
        assert gu.numel() == 2 * nh
        gate, up = gu.reshape(-1)[:nh].double(), gu.reshape(-1)[nh:].double()
        ref = (gate / (1 + torch.exp(-gate))).half().double() * up
        err = (h.double() - ref).abs()
        assert float((err / (ref.abs() + 1e-3)).max()) <= 3e-3, (two, n, S)   # 1-2 fp16 roundings
        # what the down projection reads
        hadL, orderL = get_hadK(nh)
        bitsL = had_bits(hadL, orderL, True, "cuda") if orderL > 1 else None
        su = torch.sign(torch.randn(nh, generator=g) + 1e-5).half().cuda()
        a = ops.rht(h.reshape(1, -1), order=orderL, had_bits=bitsL, pre=su, scale=nh**-0.5, out_dtype=torch.float16)
        b = ops.rht(gu, order=orderL, had_bits=bitsL, pre=su, scale=nh**-0.5, out_dtype=torch.float16,
                    pre_mode=ops.PRE_SILU_MUL)
        assert torch.equal(a.reshape(-1), b.reshape(-1)), (two, n, S)


def test_silu_pair_rejects_what_it_does_not_cover():
    from qtip_amd import ops
    from qtip_amd._lib import QtipLibraryError
    # short vectors; halves that are not whole rows of the table mix (odd order, plain power of two)
    assert not ops.rht_silu_pair_ok(2048, 1, True)
    assert not ops.rht_silu_pair_ok(4096 * 3, 3, False) and not ops.rht_silu_pair_ok(16384, 1, False)
    with pytest.raises(ValueError):
        ops.rht_silu_pair(torch.zeros(1, 3, 8192, device="cuda"), torch.ones(3, 8192, device="cuda"))
    with pytest.raises(QtipLibraryError):
        ops.rht_silu_pair(torch.zeros(1, 16384, device="cuda"), torch.ones(16384, device="cuda"))
    with pytest.raises(QtipLibraryError):
        ops.rht_silu_pair(torch.zeros(1, 3 * 4096, device="cuda"), torch.ones(3 * 4096, device="cuda"), order=3,
                          had_bits=torch.zeros(1, dtype=torch.int32, device="cuda"))


def test_token_head_kernels():
    """Final RMSNorm against the module's formula (model/llama.py:129-135) and the greedy pick
    against torch.argmax: first index among equal maxima, history slot, advanced position."""
    from qtip_amd import ops
    from qtip_amd.llama_decode import RMSNorm
    g = torch.Generator().manual_seed(11)
    for n in (256, 4096, 5120, 8192):
        x = torch.randn(1, n, generator=g).half().cuda()
        mod = RMSNorm(n, 1e-5).cuda()
        mod.weight.data = (1.0 + 0.1 * torch.randn(n, generator=g)).half().cuda()
        ref = mod(x)
        got = ops.rmsnorm(x, mod.weight, 1e-5)
        assert got.shape == ref.shape
        assert torch.allclose(got.float(), ref.float(), atol=0, rtol=2e-3)  # an fp16 ulp (hardware rsqrt)
    for vocab in (512, 32000, 32003):
        lg = torch.randn(vocab, generator=g).half().cuda()
        top = lg.max()
        first, second = vocab // 3, vocab // 3 + 9
        lg[second] = top + 1
        lg[first] = top + 1  # two equal maxima: the lower index wins
        tok = torch.tensor([[0]], device="cuda")
        pos = torch.tensor([40], device="cuda")
        hist = torch.full((8,), -1, dtype=torch.int64, device="cuda")
        ops.greedy_pick(lg, tok, pos, hist, 37)
        assert int(tok) == first == int(torch.argmax(lg.float()))
        assert int(pos) == 41
        assert hist.tolist() == [-1, -1, -1, first, -1, -1, -1, -1]
        ops.greedy_pick(lg, tok, pos, hist, 0)  # slot 41 lies outside the history: token and position only
        assert int(pos) == 42 and hist.tolist() == [-1, -1, -1, first, -1, -1, -1, -1]
        lg[vocab - 1] = top + 2  # the last element (the tail of an odd-sized vocabulary)
        ops.greedy_pick(lg, tok, pos)
        assert int(tok) == vocab - 1 and int(pos) == 43


@pytest.mark.parametrize("heads,kv_heads", [(16, 16), (16, 4)])
def test_decode_of_separate_projections_in_grouped_launches(heads, kv_heads):
    """The layout of the published checkpoints (seven projections per layer): the decode step on
    grouped launches (8 per layer) gives the logits and caches of the module-by-module forward."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=2048, heads=heads, kv_heads=kv_heads, layers=3, ffn=172 * 16, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64, fused=False)
    assert all(layer.grouped_ok() for layer in model.layers)
    ids = torch.randint(0, cfg.vocab, (1, 5), generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(5, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([5], device="cuda")
        a = model(tok, pos)
        kc = [c.clone() for c in model.k_cache]
        vc = [c.clone() for c in model.v_cache]
        b = model.decode_fused(tok, pos)
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    for c0, c1 in zip(kc + vc, list(model.k_cache) + list(model.v_cache)):
        assert torch.allclose(c0.float(), c1.float(), atol=2e-2)
    out, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64, fused=False), ids, 6, use_graph=True)
    ref, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64, fused=False), ids, 6, use_graph=False)
    assert torch.equal(out, ref)


def test_decode_of_separate_projections_with_a_table_order_hidden_size():
    """Hidden size 40 x 64 (the 13B kind: a table order times a power of two): the projections
    that share an input share their launches (12 per layer); logits and caches of the
    module-by-module forward."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder
    cfg = LlamaConfig(hidden=2560, heads=20, kv_heads=20, layers=2, ffn=108 * 32, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64, fused=False)
    assert all(layer.grouped_plain_ok() and not layer.grouped_ok() for layer in model.layers)
    ids = torch.randint(0, cfg.vocab, (1, 5), generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(5, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([5], device="cuda")
        a = model(tok, pos)
        kc = [c.clone() for c in model.k_cache]
        b = model.decode_fused(tok, pos)
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    for c0, c1 in zip(kc, model.k_cache):
        assert torch.allclose(c0.float(), c1.float(), atol=2e-2)


@pytest.mark.parametrize("hidden,heads,ffn", [(2048, 16, 172 * 32), (2560, 20, 108 * 64)])
def test_decode_of_separate_projections_with_paired_gate_up_transform(hidden, heads, ffn):
    """Intermediate sizes above 4096, where the gate / up output transforms and SiLU * up are one
    launch: the decode step (grouped launches; power-of-two and table-order hidden size) against
    the module-by-module forward, and the same tokens with and without a HIP graph."""
    from qtip_amd import ops
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    from qtip_amd.utils.matmul_had import get_hadK
    assert ops.rht_silu_pair_ok(ffn, get_hadK(ffn)[1], True)
    cfg = LlamaConfig(hidden=hidden, heads=heads, kv_heads=heads, layers=2, ffn=ffn, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64, fused=False)
    assert all(layer.grouped_ok() or layer.grouped_plain_ok() for layer in model.layers)
    ids = torch.randint(0, cfg.vocab, (1, 5), generator=torch.Generator().manual_seed(2)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(5, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([5], device="cuda")
        a = model(tok, pos)
        b = model.decode_fused(tok, pos)
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    out, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64, fused=False), ids, 6, use_graph=True)
    ref, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64, fused=False), ids, 6, use_graph=False)
    assert torch.equal(out, ref)


def test_synthetic_model_tables_leave_no_rank_one_part():
    """Seeded random tables have a centred second column (only the first value of an entry gets
    the hash's sign, lib/codebook/bitshift.py:72-80): without that every matrix carries mu * 1 1^T
    and element 0 of each layer's output grows by hundreds of sigma.  The widest output of a
    random layer stays within a few sigma and a deep random model decodes finite logits."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder
    cfg = LlamaConfig(hidden=2048, heads=16, kv_heads=4, layers=40, ffn=172 * 32, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=32)
    for layer in model.layers:
        for lin in layer._fused_linears().values():
            assert abs(float(lin.lin.tlut[:, 1].float().mean())) < 2e-3
    x = torch.randn(4, cfg.ffn, generator=torch.Generator().manual_seed(0)).half().cuda()
    y = model.layers[0].down(x).float()
    assert float(y.abs().max()) < 8 * float(y.std())
    ids = torch.randint(0, cfg.vocab, (1, 12), generator=torch.Generator().manual_seed(3)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(12, device="cuda"))
        st = model.decode_fused(lg[:, -1].argmax(-1, keepdim=True), torch.tensor([12], device="cuda"))
    assert bool(torch.isfinite(lg).all()) and bool(torch.isfinite(st).all())
    assert float(lg.float().abs().max()) < 100


@pytest.mark.parametrize("fused", [True, False])
def test_fused_decode_with_per_shard_transforms(fused):
    """Layers quantised with per-shard transforms (rcp 1: input side, rcp 2: output side, tp_rank
    slices; lib/codebook/bitshift.py:437-441,465-469) run inside the fused decode step: their sharded
    side keeps its transform as a launch of tp_rank rows, everything else stays folded.  Checked
    against the module-by-module forward (whose layer forward is held to the oracle for rcp 1 / 2),
    on both projection layouts, eagerly and through generate()'s recorded graph."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=1024, heads=8, kv_heads=8, layers=3, ffn=172 * 16, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64, fused=fused)

    def shard(lin, rcp, tp):
        if isinstance(lin.rcp, torch.Tensor):  # plain ints after the module's first forward
            lin.rcp.fill_(rcp)
            lin.tp_rank.fill_(tp)
        else:
            lin.rcp, lin.tp_rank = rcp, tp

    l0, l1, l2 = model.layers
    shard(l0.o, 1, 8)
    shard(l0.down, 2, 4)
    if fused:
        shard(l1.qkv, 2, 8)       # 3072 outputs: 8 slices of 384 = 12 x 32
        shard(l1.up_gate, 1, 4)
        shard(l2.up_gate, 2, 8)   # 5504 outputs: 8 slices of 688 = 172 x 4
        shard(l2.qkv, 1, 2)
    else:
        shard(l1.k_proj, 2, 8)
        shard(l1.gate_proj, 1, 4)
        shard(l2.up_proj, 2, 8)   # 2752 outputs: 8 slices of 344 = 172 x 2
        shard(l2.q_proj, 1, 2)
    shard(l2.down, 1, 4)          # 2752 inputs: 4 slices of 688
    assert model.supports_fused_decode()
    ids = torch.randint(0, cfg.vocab, (1, 9), generator=torch.Generator().manual_seed(0)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(9, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([9], device="cuda")
        a = model(tok, pos)
        kc = [c.clone() for c in model.k_cache]
        b = model.decode_fused(tok, pos)
    assert bool(torch.isfinite(b).all())
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    for c0, c1 in zip(kc, model.k_cache):
        assert torch.allclose(c0.float(), c1.float(), atol=2e-2)
    # a sharded side really changes the result: the same weights read as rcp 0 decode differently
    shard(l0.o, 0, 8)
    for name in ("_fused", "_grouped", "_grouped_plain"):
        l0.__dict__.pop(name, None)
    with torch.no_grad():
        c = model.decode_fused(tok, pos)
    assert float((c - b).abs().max()) > 1e-2
    shard(l0.o, 1, 8)
    for name in ("_fused", "_grouped", "_grouped_plain"):
        l0.__dict__.pop(name, None)
    out_g, _, _ = generate(model, ids, 6, use_graph=True, fused=True)
    out_e, _, _ = generate(model, ids, 6, use_graph=False, fused=True)
    assert torch.equal(out_g, out_e) and out_g.shape == (1, 6)
    # the steps after the first, teacher-forced: the tokens the fused loop decoded go through the
    # module path and through the fused step position by position (greedy picks of two paths may
    # part on a near-tie, logits and caches may not differ by more than the rounding allows)
    with torch.no_grad():
        model(ids, torch.arange(9, device="cuda"))
        for t in range(5):
            tok, pos = out_g[:, t:t + 1].contiguous(), torch.tensor([9 + t], device="cuda")
            a = model(tok, pos)
            kc = [c.clone() for c in model.k_cache + model.v_cache]
            for c in model.k_cache + model.v_cache:
                c[:, :, 9 + t].zero_()
            b = model.decode_fused(tok, pos)
            assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
            for c0, c1 in zip(kc, model.k_cache + model.v_cache):
                assert torch.allclose(c0[:, :, :10 + t].float(), c1[:, :, :10 + t].float(), atol=2e-2)


def test_sample_pick_draws_from_the_reference_distribution():
    """Sampled pick (eval/interactive_gen.py:15-40): top_k = 1 is the argmax; draws stay inside the
    top-k set (ties with the k-th value included); empirical frequencies over 4000 draws follow
    softmax(logits / T) on that set; the counter advances so replays differ."""
    from qtip_amd import ops
    g = torch.Generator().manual_seed(5)
    vocab = 32003
    lg = (torch.randn(vocab, generator=g) * 0.5).half()
    top = [17, 4000, 31999, 12345, 9]
    vals = [4.0, 3.5, 3.5, 3.0, 2.0]
    for i, v in zip(top, vals):
        lg[i] = v
    lg = lg.cuda()
    tok = torch.tensor([[0]], device="cuda")
    pos = torch.tensor([10], device="cuda")
    ctr = torch.zeros(1, dtype=torch.int64, device="cuda")
    hist = torch.full((4,), -1, dtype=torch.int64, device="cuda")
    ops.sample_pick(lg, 0.6, 1, 123, ctr, tok, pos, hist, 9)
    assert int(tok) == 17 and int(pos) == 11 and int(ctr) == 1 and hist.tolist() == [-1, 17, -1, -1]
    T, k, n = 0.8, 4, 4000
    counts = {}
    for _ in range(n):
        ops.sample_pick(lg, T, k, 123, ctr, tok, pos)
        t = int(tok)
        counts[t] = counts.get(t, 0) + 1
    assert int(ctr) == n + 1
    assert set(counts) <= set(top[:4])  # the 4th largest value is 3.0; 2.0 is out
    p = torch.softmax(torch.tensor(vals[:4]) / T, 0)
    for i, pi in zip(top[:4], p.tolist()):
        assert abs(counts.get(i, 0) / n - pi) < 0.03, (i, counts.get(i, 0) / n, pi)
    # ties with the k-th value stay in: top_k = 2 keeps both 3.5 entries
    counts = {}
    for _ in range(600):
        ops.sample_pick(lg, T, 2, 7, ctr, tok, pos)
        counts[int(tok)] = counts.get(int(tok), 0) + 1
    assert set(counts) == {17, 4000, 31999}
    # the whole vocabulary (top_k None) at a low temperature: mostly the largest entries, never an error
    for _ in range(50):
        ops.sample_pick(lg, 0.05, None, 7, ctr, tok, pos)
        assert int(tok) in (17, 4000, 31999)


def test_generate_greedy_keeps_its_bookkeeping_on_the_device():
    """Greedy decoding through the captured step (pick kernel inside the graph) returns the tokens
    of the eager loop, and the streaming callback sees them in order."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=1024, heads=8, kv_heads=8, layers=2, ffn=172 * 16, vocab=512)
    ids = torch.randint(0, cfg.vocab, (1, 7), generator=torch.Generator().manual_seed(4)).cuda()
    seen = []
    a, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 9, use_graph=True, callback=lambda t: seen.append(t.clone()))
    b, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 9, use_graph=False)
    c, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 9, use_graph=True, fused=False)
    assert a.shape == (1, 9) and torch.equal(a, b)
    assert len(seen) == 9 and torch.equal(torch.cat(seen, dim=1), a)
    # the module-by-module path rounds differently; its first tokens agree on this model
    assert torch.equal(a[:, :2], c[:, :2])


def test_generate_sampling_and_streaming():
    """Sampled decoding through the captured step: top_k = 1 reproduces the greedy tokens, a
    wider draw stays inside the vocabulary, and the streaming callback sees every token in order."""
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=1024, heads=8, kv_heads=8, layers=2, ffn=172 * 16, vocab=512)
    ids = torch.randint(0, cfg.vocab, (1, 7), generator=torch.Generator().manual_seed(3)).cuda()
    greedy, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 8)
    seen = []
    top1, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 8, temperature=0.6, top_k=1,
                          callback=lambda t: seen.append(t))
    assert torch.equal(top1, greedy)
    assert len(seen) == 8 and torch.equal(torch.cat(seen, dim=1), top1)
    torch.manual_seed(5)
    drawn, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 8, temperature=0.6, top_k=5)
    assert drawn.shape == (1, 8) and int(drawn.min()) >= 0 and int(drawn.max()) < cfg.vocab
    # the draw follows torch.manual_seed, with or without the captured graph
    torch.manual_seed(5)
    again, _, _ = generate(LlamaDecoder(cfg, max_cache_len=64), ids, 8, temperature=0.6, top_k=5, use_graph=False)
    assert torch.equal(drawn, again)


def test_fused_decode_step_matches_generic():
    # the 13-launch fused decode step against the module-by-module forward of the same model
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder
    cfg = LlamaConfig(hidden=1024, heads=8, kv_heads=8, layers=2, ffn=172 * 16, vocab=512)
    model = LlamaDecoder(cfg, max_cache_len=64)
    ids = torch.randint(0, cfg.vocab, (1, 9), generator=torch.Generator().manual_seed(0)).cuda()
    with torch.no_grad():
        lg = model(ids, torch.arange(9, device="cuda"))
        tok = lg[:, -1].argmax(-1, keepdim=True)
        pos = torch.tensor([9], device="cuda")
        a = model(tok, pos)
        kc = [c.clone() for c in model.k_cache]
        b = model.decode_fused(tok, pos)
    assert_close(b.cpu().numpy(), a.cpu().numpy(), 2e-2, 5e-3)
    for c0, c1 in zip(kc, model.k_cache):
        assert torch.allclose(c0.float(), c1.float(), atol=2e-2)


@pytest.mark.parametrize("n", [2048, 4096, 8192])
@pytest.mark.parametrize("S,rows", [(1, 1), (2, 1), (4, 3)])
def test_rht_chain_matches_two_launches(n, S, rows):
    """[transform-out + residual] + [RMSNorm + transform-in] in one workgroup against the two fused
    launches it replaces, and against a float64 statement of the same rounding sequence."""
    from qtip_amd import ops
    g = torch.Generator().manual_seed(n + S + rows)
    parts = torch.randn(S, rows, n, generator=g).cuda()
    SV = (torch.sign(torch.randn(n, generator=g)) * (0.5 + torch.rand(n, generator=g))).cuda()
    SU = torch.sign(torch.randn(n, generator=g)).half().cuda()
    res = torch.randn(rows, n, generator=g).half().cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).half().cuda()
    so, si, eps = 32.0 * n**-0.5, n**-0.5 / 32.0, 1e-5
    x_new, xt = ops.rht_chain(parts, SV, so, res, w, eps, SU, si)
    x_ref = ops.rht(parts, post=SV, scale=so, out_dtype=torch.float16, in_parts=S, residual=res)
    xt_ref = ops.rht(x_ref, pre=SU, scale=si, out_dtype=torch.float16, pre_mode=ops.PRE_RMSNORM, norm_weight=w, eps=eps)
    # fp32 sums in another order: results agree to an fp16 ulp here and there
    assert (x_new.float() - x_ref.float()).abs().max() <= 2e-3 * x_ref.float().abs().max()
    assert (xt.float() - xt_ref.float()).abs().max() <= 4e-3 * xt_ref.float().abs().max()
    # independent float64 statement
    H = O.hadamard_transform(np.eye(n))  # symmetric for powers of two
    y = (parts.double().sum(0).cpu().numpy() @ H) * SV.double().cpu().numpy() * (so * n**0.5)
    xn = (res.float().cpu().numpy() + y.astype(np.float16).astype(np.float32)).astype(np.float16)
    assert np.abs(x_new.float().cpu().numpy() - xn.astype(np.float32)).max() <= 2e-3 * np.abs(xn).max()
    v = xn.astype(np.float64)
    rs = 1.0 / np.sqrt((v**2).mean(-1, keepdims=True) + eps)
    hn = (w.float().cpu().numpy() * (v * rs).astype(np.float16).astype(np.float32)).astype(np.float16).astype(np.float64)
    t = ((hn * SU.float().cpu().numpy()) @ H) * (si * n**0.5)
    assert np.abs(xt.float().cpu().numpy() - t).max() <= 4e-3 * np.abs(t).max()


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("m,k,S", [(256, 2048, None), (1024, 4096, 1), (4096, 4096, None), (512, 8192, 4),
                                   (2048, 8192, None)])
def test_matvec_with_transform_in_prologue(K, m, k, S):
    """The matvec that computes fp16(scale * H_k(su * x)) itself against the transform launch
    followed by the plain matvec (same partial-sum layout), and against a float64 statement."""
    from qtip_amd import ops
    L = make_layer(m, k, K, seed=m + k + K)
    g = torch.Generator().manual_seed(K + m)
    x = torch.randn(k, generator=g).half().cuda()
    su = dev(L["SU"]).half()
    scale = k**-0.5 / 32.0
    packed, tlut = dev(L["packed"]).reshape(-1), dev(L["tlut"]).reshape(-1)
    parts = ops.decompress_matvec_parts_rht(packed, x, su, scale, tlut, m, k, K, nparts=S)
    xt = ops.rht(x.reshape(1, k), pre=su, scale=scale, out_dtype=torch.float16)
    ref = ops.decompress_matvec_parts(packed, xt.reshape(-1), tlut, m, k, K, nparts=S)
    assert parts.shape == ref.shape
    y, r = parts.sum(0).double().cpu().numpy(), ref.sum(0).double().cpu().numpy()
    # the butterflies run in another order: x_t differs by an fp16 ulp in a few places
    assert np.abs(y - r).max() <= 2e-3 * np.abs(r).max()
    W = c_oracle.decode(L["packed"], L["tlut"], m, k, K).astype(np.float64)
    H = O.hadamard_transform(np.eye(k))
    t = ((x.double().cpu().numpy() * su.double().cpu().numpy()) @ H) * (scale * k**0.5)
    t16 = t.astype(np.float16).astype(np.float64)
    want = W @ t16
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()


def test_forward_empty_and_slabbed_batches():
    """No rows in, no rows out; more rows than one launch takes go through in slabs with the
    same result as one pass."""
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    m, k, K = 256, 512, 3
    L = make_layer(m, k, K, seed=4)
    mod = BitshiftLinear(16, 16, 16, K, 2, 9, "quantlut_sym", tlut=dev(L["tlut"]), has_kernel=True)
    hl, Kl = mh.get_hadK(k)
    hr, Kr = mh.get_hadK(m)
    args = (dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), hl, hr, Kl, Kr, 0, 8)
    empty = mod(torch.empty(0, k, dtype=torch.float16, device="cuda"), *args)
    assert empty.shape == (0, m) and empty.dtype == torch.float16
    empty3 = mod(torch.empty(2, 0, k, dtype=torch.float16, device="cuda"), *args)
    assert empty3.shape == (2, 0, m)
    x = torch.randn(2, 5, k, generator=torch.Generator().manual_seed(1)).half().cuda()
    whole = mod(x, *args)
    mod.max_rows = 4  # 10 rows -> slabs of 4, 4, 2 (the last two through other kernels than the first)
    slabbed = mod(x, *args)
    assert slabbed.shape == whole.shape == (2, 5, m)
    assert (slabbed.float() - whole.float()).abs().max() <= 2e-3 * whole.float().abs().max()


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("ms,k,S,Sp", [((512, 512, 512), 2048, None, 1), ((4096, 4096, 4096), 4096, None, 2),
                                       ((8192, 1024, 1024), 8192, 2, 2), ((11008 - 11008 % 32, 2752), 4096, 1, 1),
                                       ((64,), 2048, 4, 3), ((32, 32, 9600), 4096, 2, 1)])
def test_grouped_matvec_with_layer_boundary(K, ms, k, S, Sp):
    """Up to three matrices behind one layer boundary in one launch (separate q / k / v or
    gate / up projections): every matrix's partial sums and the new residual stream equal the
    single-matrix launch bit for bit (a row block is summed by one workgroup in a fixed order,
    whichever workgroup that is)."""
    from qtip_amd import ops
    g = torch.Generator().manual_seed(K + sum(ms) + Sp)
    layers = [make_layer(m, k, K, seed=m + k + K + i) for i, m in enumerate(ms)]
    prev = torch.randn(Sp, 1, k, generator=g).cuda()
    SV = (torch.sign(torch.randn(k, generator=g)) * (0.5 + torch.rand(k, generator=g))).cuda()
    res = torch.randn(1, k, generator=g).half().cuda()
    w = (1 + 0.1 * torch.randn(k, generator=g)).half().cuda()
    so, si, eps = 32.0 * k**-0.5, k**-0.5 / 32.0, 1e-5
    packed = [dev(L["packed"]).reshape(-1) for L in layers]
    tluts = [dev(L["tlut"]).reshape(-1) for L in layers]
    sus = [dev(L["SU"]).half() for L in layers]
    parts, x_new = ops.decompress_matvec_group_chain(packed, tluts, list(ms), k, K, prev, SV, so, res, w, eps, sus, si,
                                                     nparts=S)
    assert parts.shape[1] == sum(ms)
    off = 0
    for i, m in enumerate(ms):
        one, x_one = ops.decompress_matvec_parts_chain(packed[i], tluts[i], m, k, K, prev, SV, so, res, w, eps, sus[i],
                                                       si, nparts=parts.shape[0])
        assert torch.equal(x_one, x_new)
        assert torch.equal(parts[:, off:off + m], one), (i, m)
        off += m


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("ms,k,S", [((512, 512, 512), 5120, None), ((5120, 5120, 5120), 5120, 2), ((13824, 13824), 5120, 1),
                                    ((64,), 1024, 1), ((32, 96, 2048), 11008, 2)])
def test_grouped_plain_matvec(K, ms, k, S):
    """Up to three matrices, each on its own input, in one launch: bit-identical to the
    single-matrix launches."""
    from qtip_amd import ops
    layers = [make_layer(m, k, K, seed=m + k + K + 7 * i) for i, m in enumerate(ms)]
    packed = [dev(L["packed"]).reshape(-1) for L in layers]
    tluts = [dev(L["tlut"]).reshape(-1) for L in layers]
    xs = torch.randn(len(ms), k, generator=torch.Generator().manual_seed(k + K)).half().cuda()
    parts = ops.decompress_matvec_group(packed, [xs[i] for i in range(len(ms))], tluts, list(ms), k, K, nparts=S)
    off = 0
    for i, m in enumerate(ms):
        one = ops.decompress_matvec_parts(packed[i], xs[i], tluts[i], m, k, K, nparts=parts.shape[0])
        assert torch.equal(parts[:, off:off + m], one.reshape(parts.shape[0], m)), (i, m)
        off += m


@pytest.mark.parametrize("n", [5120, 4096, 1024, 11008, 13824])
def test_input_transforms_of_several_layers_in_one_launch(n):
    """rht_fused_pre_rows == one fused RMSNorm + transform launch per sign vector, bit for bit."""
    from qtip_amd import ops
    from qtip_amd.utils.matmul_had import get_hadK, had_bits
    g = torch.Generator().manual_seed(n)
    x = torch.randn(1, n, generator=g).half().cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).half().cuda()
    pre = torch.sign(torch.randn(3, n, generator=g) + 1e-5).half().cuda()
    hadK, order = get_hadK(n)
    bits = had_bits(hadK, order, True, "cuda") if order > 1 else None
    got = ops.rht_fused_pre_rows(x, pre, w, 1e-5, order=order, had_bits=bits, scale=n**-0.5 / 32)
    for r in range(3):
        one = ops.rht(x, order=order, had_bits=bits, pre=pre[r].contiguous(), scale=n**-0.5 / 32,
                      out_dtype=torch.float16, pre_mode=ops.PRE_RMSNORM, norm_weight=w, eps=1e-5)
        assert torch.equal(got[r], one.reshape(-1)), (n, r)


def test_forward_many_rows_decodes_and_multiplies():
    """From BitshiftLinear.dense_rows_min rows on the layer decodes to dense fp16 and multiplies
    with the BLAS library (the reference's route for every batch, bitshift.py:476-489): same
    result as the fused decompress-GEMM and as the oracle's dense layer."""
    from qtip_amd.codebook.bitshift import BitshiftLinear, BitshiftLinearKernelAG
    from qtip_amd.utils import matmul_had as mh
    m, k, K = 512, 1024, 2
    L = make_layer(m, k, K, seed=9)
    mod = BitshiftLinear(16, 16, 16, K, 2, 9, "quantlut_sym", tlut=dev(L["tlut"]), has_kernel=True)
    hl, Kl = mh.get_hadK(k)
    hr, Kr = mh.get_hadK(m)
    args = (dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), hl, hr, Kl, Kr, 0, 8)
    rows = BitshiftLinear.dense_rows_min + 9
    x = torch.randn(rows, k, generator=torch.Generator().manual_seed(2)).half()
    dense = mod(x.cuda(), *args)
    mod.dense_rows_min = 10**9
    fused = mod(x.cuda(), *args)
    assert dense.shape == fused.shape == (rows, m)
    assert_close(dense.float().cpu().numpy(), fused.float().cpu().numpy(), 5e-3, 5e-4)
    ref = O.bitshift_linear_forward(x[:4].numpy(), L["packed"], L["SU"], L["SV"], L["tlut"], K)
    assert_close(dense[:4].cpu().numpy(), ref)
    lut = mod.cb.lut.cuda() if hasattr(mod.cb, "lut") else None
    if lut is not None:
        a = BitshiftLinearKernelAG.apply(x.cuda(), dev(L["packed"]), m, k, 16, 9, K, 2, lut)
        b = BitshiftLinearKernelAG.apply(x[:8].cuda(), dev(L["packed"]), m, k, 16, 9, K, 2, lut)
        assert_close(a[:8].float().cpu().numpy(), b.float().cpu().numpy(), 5e-3, 5e-4)


@pytest.mark.parametrize("K", [2, 4])
@pytest.mark.parametrize("m,k,S,Sp", [(256, 2048, None, 1), (1024, 4096, 1, 2), (4096, 4096, None, 2), (512, 8192, 4, 1),
                                      (2048, 8192, None, 3)])
def test_matvec_with_layer_boundary_in_prologue(K, m, k, S, Sp):
    """[output transform + residual + RMSNorm + input transform] inside the matvec launch against
    the chained-transform launch followed by the plain matvec: same residual stream bit for bit
    (same arithmetic in the same order), partial sums to rounding."""
    from qtip_amd import ops
    L = make_layer(m, k, K, seed=m + k + K + 1)
    g = torch.Generator().manual_seed(K + m + Sp)
    prev = torch.randn(Sp, 1, k, generator=g).cuda()
    SV = (torch.sign(torch.randn(k, generator=g)) * (0.5 + torch.rand(k, generator=g))).cuda()
    res = torch.randn(1, k, generator=g).half().cuda()
    w = (1 + 0.1 * torch.randn(k, generator=g)).half().cuda()
    su = dev(L["SU"]).half()
    so, si, eps = 32.0 * k**-0.5, k**-0.5 / 32.0, 1e-5
    packed, tlut = dev(L["packed"]).reshape(-1), dev(L["tlut"]).reshape(-1)
    parts, x_new = ops.decompress_matvec_parts_chain(packed, tlut, m, k, K, prev, SV, so, res, w, eps, su, si, nparts=S)
    x_ref, xt_ref = ops.rht_chain(prev, SV, so, res, w, eps, su, si)
    ref = ops.decompress_matvec_parts(packed, xt_ref.reshape(-1), tlut, m, k, K, nparts=S)
    assert torch.equal(x_new, x_ref)
    assert parts.shape == ref.shape
    assert torch.equal(parts, ref)


@pytest.mark.parametrize("rcp", [1, 2])
@pytest.mark.parametrize("bs", [1, 3])
def test_forward_with_per_shard_transforms(rcp, bs):
    """rcp 1 / 2: the input / output transform acts on each of the tp_rank shards of the vector
    separately (lib/codebook/bitshift.py:437-441, 465-469), as layers quantised for tensor
    parallelism expect."""
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    m, k, K, shards = 512, 1536, 2, 8   # 1536 = 12 * 128, shard 192 = 12 * 16; 512 / 8 = 64
    L = make_layer(m, k, K, seed=rcp)
    mod = BitshiftLinear(16, 16, 16, K, 2, 9, "quantlut_sym", tlut=dev(L["tlut"]), has_kernel=True)
    g = torch.Generator().manual_seed(bs)
    x = torch.randn(bs, k, generator=g).half()
    hl, Kl = mh.get_hadK(k)
    hr, Kr = mh.get_hadK(m)
    y = mod(x.cuda(), dev(L["packed"]), dev(L["SU"]), dev(L["SV"]), hl, hr, Kl, Kr, rcp, shards).float().cpu().numpy()
    W = c_oracle.decode(L["packed"], L["tlut"], m, k, K).astype(np.float64)
    xs = x.numpy().astype(np.float64) * L["SU"].astype(np.float64)
    if rcp == 1:
        xt = O.hadamard_transform(xs.reshape(-1, k // shards), transpose=True).reshape(bs, k) / 32
    else:
        xt = O.hadamard_transform(xs, transpose=True) / 32
    z = xt.astype(np.float16).astype(np.float64) @ W.T
    if bs > 1:
        z = z.astype(np.float16).astype(np.float64)  # the batched path returns an fp16 product
    if rcp == 2:
        z = O.hadamard_transform(z.reshape(-1, m // shards)).reshape(bs, m)
    else:
        z = O.hadamard_transform(z)
    ref = z * (L["SV"].astype(np.float64) * 32)
    assert_close(y, ref, max_rel=1e-2, mean_rel=2e-3)
