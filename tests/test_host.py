"""CPU: host logic and the C-ABI surface (no kernel launches)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "qtip_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qtip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from qtip_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build with python -m qtip_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 7
    for name in declared:
        assert hasattr(handle, name), name
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared
    assert _lib.lib().qtip_abi_version() == _lib.ABI_VERSION
    assert b"shape" in _lib.lib().qtip_error_string(-1)


def test_measurement_aids_live_in_a_library_of_their_own():
    """libqtip_hip.so exports no probe; bench_probe/libqtip_probe.so exports what its header declares."""
    from qtip_amd import _lib
    import bench_probe
    main = ctypes.CDLL(_lib.LIB_PATH)
    assert os.path.exists(bench_probe.LIB_PATH), "build with python -m bench_probe"
    probe = ctypes.CDLL(bench_probe.LIB_PATH)
    text = open(os.path.join(ROOT, "bench_probe", "qtip_probe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(qtip_probe_[a-z0-9_]+)\s*\(", text)))
    assert names == ["qtip_probe_issue", "qtip_probe_stream_read"]
    for name in names:
        assert hasattr(probe, name), name
        assert not hasattr(main, name), name


def test_python_host_never_routes_through_the_shared_scratch_entry_point():
    """qtip_decompress_matvec_noalloc keeps its partial sums in one array per GPU, so overlapping
    calls race: it is for callers of the C ABI that accept that.  The package's own wrappers (which
    serve any number of streams) bind it but never call it."""
    import glob
    hits = []
    for path in glob.glob(os.path.join(ROOT, "qtip_amd", "**", "*.py"), recursive=True):
        for n, line in enumerate(open(path), 1):
            if "qtip_decompress_matvec_noalloc" in line and not path.endswith("_lib.py"):
                hits.append((path, n))
    assert hits == []


def test_argument_rejection_without_gpu():
    # rejected arguments return a negative code before anything touches the device
    from qtip_amd import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    null = ctypes.c_void_p(0)
    assert L.qtip_decompress_matvec(p, p, p, p, 33, 64, 2, null, 0, null) == -1
    assert L.qtip_decompress_matvec(p, p, p, p, 64, 64, 5, null, 0, null) == -1
    assert L.qtip_decompress_matvec(null, p, p, p, 64, 64, 2, null, 0, null) == -2
    assert L.qtip_decode(p, p, null, 64, 64, 2, null) == -2
    assert L.qtip_decompress_gemm(p, p, p, p, 64, 64, 2, 0, 0, null, 0, null) == -1
    assert L.qtip_gemm_workspace_bytes(33, 64, 2, 8) == 0
    assert L.qtip_rht(p, 0, p, 0, 1, 1, 100, 1, null, null, null, 1.0, null) == -1  # not a power of two
    assert L.qtip_rht(p, 0, p, 0, 1, 1, 12 * 64, 12, null, null, null, 1.0, null) == -2  # table missing
    assert L.qtip_rht(p, 7, p, 0, 1, 1, 64, 1, null, null, null, 1.0, null) == -5
    assert L.qtip_matvec_split(33, 64, 2) == 0 and L.qtip_matvec_split(64, 64, 7) == 0
    assert L.qtip_decompress_matvec_parts(p, p, p, p, 64, 64, 2, 0, null) in (-1, 100, 101)  # bad nparts (or no device)
    assert L.qtip_decompress_matvec_parts(null, p, p, p, 64, 64, 2, 1, null) == -2


def test_cpu_tensors_raise():
    from qtip_amd import ops
    with pytest.raises(ValueError):
        ops.decode(torch.zeros(64 * 64 * 2 // 16, dtype=torch.int16), torch.zeros(512, 2, dtype=torch.float16), 64, 64, 2)
    import qtip_amd.utils.matmul_had  # registers hadamard::hadamard (GPU implementation only)
    with pytest.raises(NotImplementedError):
        torch.ops.hadamard.hadamard(torch.zeros(2, 64), 1.0)


def test_has_kernel_gate():
    from qtip_amd.utils.kernel_check import has_kernel
    assert has_kernel('quantlut_sym', 16, 2, 2, 9, 16, 16)
    assert has_kernel('quantlut_sym', 16, 4, 2, 9, 16, 16)
    for bad in [('lut', 16, 2, 2, 9, 16, 16), ('quantlut_sym', 12, 2, 2, 9, 16, 16), ('quantlut_sym', 16, 5, 2, 9, 16, 16),
                ('quantlut_sym', 16, 1, 2, 9, 16, 16), ('quantlut_sym', 16, 2, 1, 9, 16, 16),
                ('quantlut_sym', 16, 2, 2, 10, 16, 16), ('quantlut_sym', 16, 2, 2, 9, 8, 16)]:
        assert not has_kernel(*bad)


def test_op_registry_names():
    import qtip_amd.codebook as cbk
    # every Llama-2 7B / 70B layer shape at every bit width, under the reference's naming scheme
    for m, k in [(4096, 4096), (12288, 4096), (22016, 4096), (4096, 11008), (10240, 8192), (8192, 8192),
                 (57344, 8192), (8192, 28672), (28672, 8192)]:
        for b in (2, 3, 4):
            assert (m, 1, k, b) in cbk.kdict
            assert hasattr(torch.ops.quip_lib, f"decompress_matvec_qtip_{m}_1_{k}_{b}")
    assert len([k for k in cbk.kernels if k[0] != 256]) == 61
    op = cbk.register_shape(64, 128, 3)
    assert op is cbk.kdict[(64, 1, 128, 3)]
    with pytest.raises(ValueError):
        cbk.register_shape(48, 128, 3)
    # fake (meta) implementation: shape/dtype only
    out = torch.ops.quip_lib.decompress_matvec_qtip_4096_1_4096_2(
        torch.empty(1, device="meta", dtype=torch.int16), torch.empty(1, 4096, device="meta"),
        torch.empty(512, 2, device="meta", dtype=torch.float16))
    assert out.shape == (1, 4096) and out.dtype == torch.float32


def test_quantlut_sym_matches_oracle():
    from oracle import qtip_oracle as O
    from qtip_amd.codebook.bitshift import quantlut_sym
    t = torch.randn(512, 2, generator=torch.Generator().manual_seed(0)).half()
    a = quantlut_sym(t, 16, 9).numpy().view(np.uint16)
    b = O.quantlut_sym(t.numpy()).view(np.uint16)
    assert np.array_equal(a, b)


def test_tlut_roundtrip_through_expanded_table():
    from qtip_amd.codebook.bitshift import quantlut_sym
    from qtip_amd.utils.kernel_decompress import _representatives, tlut_from_expanded
    t = torch.randn(512, 2, generator=torch.Generator().manual_seed(1)).half()
    back = tlut_from_expanded(quantlut_sym(t, 16, 9))
    seen = _representatives()[2]
    assert torch.equal(back[seen], t[seen])
    # every index some state hashes to is covered (all 512 are reachable)
    assert int(seen.sum()) == 512


def test_unpack_trellis_matches_oracle():
    from oracle import qtip_oracle as O
    from qtip_amd.codebook.bitshift import bitshift_codebook
    for K in (2, 3, 4):
        cb = bitshift_codebook(16, K, 2, 9, 'quantlut_sym', tlut=torch.zeros(512, 2, dtype=torch.float16))
        words = np.random.default_rng(K).integers(0, 65536, (6, 16 * K), dtype=np.uint16)
        got = cb.unpack_trellis(torch.from_numpy(words.view(np.int16)), 256).numpy()
        assert np.array_equal(got, O.unpack_trellis_natural(words, K))


def test_get_hadK_and_bits():
    from oracle import qtip_oracle as O
    from qtip_amd.utils import matmul_had as mh
    for n in (4096, 11008, 12288, 10240, 28672, 57344, 22016):
        had, K = mh.get_hadK(n)
        ohad, oK = O.get_hadK(n)
        assert K == oK
        if K > 1:
            assert np.array_equal(had.numpy(), ohad)
            assert np.array_equal(mh.get_hadK(n, transpose=True)[0].numpy(), ohad.T)
    with pytest.raises(AssertionError):
        mh.get_hadK(100)
    neg = np.random.default_rng(0).integers(0, 2, (20, 20)).astype(bool)
    w = mh._pack_bits(neg).view(np.uint32)
    for i in range(20):
        for j in range(20):
            b = j * 20 + i
            assert ((w[b >> 5] >> (b & 31)) & 1) == neg[i, j]


def test_had_bits_cache_follows_the_memory_not_the_object():
    """A caller's own table: a fresh view of the same memory hits the cache (no repacking, hence no
    device-to-host copy per forward), an in-place change or a new tensor misses, and an entry
    disappears with the storage it was packed from."""
    import gc
    from qtip_amd.utils import matmul_had as mh
    rng = np.random.default_rng(3)
    K = 8  # no built-in table of this order: the caller's own entry is used
    h = torch.from_numpy(np.where(rng.integers(0, 2, (K, K)) > 0, 1.0, -1.0).astype(np.float32))
    mh._bit_cache.clear()
    b0 = mh.had_bits(h, K, False, "cpu")
    n_entries = len(mh._bit_cache)
    assert mh.had_bits(h.data, K, False, "cpu") is b0          # another tensor object, same memory
    assert mh.had_bits(h.view(K, K), K, False, "cpu") is b0
    assert len(mh._bit_cache) == n_entries
    bt = mh.had_bits(h, K, True, "cpu")
    assert bt is not b0 and torch.equal(bt, torch.from_numpy(mh._pack_bits((h.numpy() < 0).T)))
    h[0, 0] = -h[0, 0]                                          # in-place edit: version bump, repacked
    b1 = mh.had_bits(h, K, False, "cpu")
    assert b1 is not b0 and torch.equal(b1, torch.from_numpy(mh._pack_bits(h.numpy() < 0)))
    h2 = h.clone()
    assert mh.had_bits(h2, K, False, "cpu") is not b1           # other memory: its own entry
    before = len(mh._bit_cache)
    del h2
    gc.collect()
    assert len(mh._bit_cache) == before - 1                     # freed storage: entry dropped
    with pytest.raises(ValueError):
        mh.had_bits(torch.zeros(K, K), K, False, "cpu")


def test_quantiser_entry_points_raise():
    from qtip_amd.codebook.bitshift import BitshiftLinear, bitshift_codebook
    cb = bitshift_codebook(16, 2, 2, 9, 'quantlut_sym')
    with pytest.raises(NotImplementedError):
        cb.quantize(None)
    with pytest.raises(NotImplementedError):
        bitshift_codebook(12, 2, 1, 16, '1mad')  # only 16-bit state windows are built
    with pytest.raises(ValueError):  # packing states needs device tensors
        cb.pack_trellis(torch.zeros(1, 128, dtype=torch.int32))
    with pytest.raises(ValueError):
        BitshiftLinear(16, 16, 16, 5, 2, 9, 'quantlut_sym', has_kernel=True)


def test_rope_scaling_follows_the_rotary_initialisers():
    """rope_inv_freq against the initialisers the reference's LlamaRotaryEmbedding uses
    (model/llama.py:39,185: transformers' ROPE_INIT_FUNCTIONS) for the static types."""
    import torch
    from qtip_amd.llama_decode import LlamaConfig, rope_inv_freq
    base = dict(hidden=4096, heads=32, rope_theta=500000.0)
    plain = rope_inv_freq(LlamaConfig(**base))
    want = 1.0 / (500000.0**(torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    assert torch.equal(plain, want)
    lin = rope_inv_freq(LlamaConfig(**base, rope_scaling={"type": "linear", "factor": 4.0}))
    assert torch.allclose(lin, want / 4.0, rtol=0, atol=0)
    l3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    got = rope_inv_freq(LlamaConfig(**base, rope_scaling=l3))
    # closed-form properties: short wavelengths untouched, long ones divided by the factor, monotone in between
    wavelen = 2 * torch.pi / want
    assert torch.equal(got[wavelen < 8192 / 4.0], want[wavelen < 8192 / 4.0])
    assert torch.allclose(got[wavelen > 8192 / 1.0], want[wavelen > 8192 / 1.0] / 8.0)
    mid = ~(wavelen < 8192 / 4.0) & ~(wavelen > 8192 / 1.0)
    assert mid.any() and bool(((got[mid] <= want[mid]) & (got[mid] >= want[mid] / 8.0)).all())
    try:
        from transformers import LlamaConfig as HFConfig
        from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    except Exception:  # the library moved the table: the closed-form checks above stand alone
        return
    hf = HFConfig(hidden_size=4096, num_attention_heads=32, rope_theta=500000.0, rope_scaling=dict(l3),
                  max_position_embeddings=131072)
    ref, att = ROPE_INIT_FUNCTIONS["llama3"](hf, "cpu")
    assert att == 1.0 and torch.allclose(got, ref, rtol=1e-6, atol=0)
    with pytest.raises(NotImplementedError):
        rope_inv_freq(LlamaConfig(**base, rope_scaling={"rope_type": "dynamic", "factor": 2.0}))


def test_sampling_helpers_follow_the_generation_script():
    """top-k restriction and the exponential-race draw of eval/interactive_gen.py:15-40."""
    from qtip_amd.llama_decode import logits_to_probs, sample
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(2, 50, generator=g)
    p = logits_to_probs(logits, temperature=0.6, top_k=5)
    assert torch.allclose(p.sum(-1), torch.ones(2))
    assert ((p > 0).sum(-1) == 5).all()
    top = logits.topk(5).indices
    assert all(set(torch.nonzero(p[i]).flatten().tolist()) == set(top[i].tolist()) for i in range(2))
    # ratios inside the kept set are those of softmax(logits / T)
    full = torch.softmax(logits / 0.6, -1)
    i0, i1 = top[0, 0], top[0, 1]
    assert abs(p[0, i0] / p[0, i1] - full[0, i0] / full[0, i1]) < 1e-4
    # top_k = 1 is greedy whatever the random draw
    torch.manual_seed(1)
    tok, _ = sample(logits[:, None, :], temperature=0.6, top_k=1)
    assert (tok.flatten() == logits.argmax(-1)).all()
    # the exponential race draws from the distribution: frequencies of a 3-way distribution
    torch.manual_seed(2)
    lg = torch.log(torch.tensor([0.7, 0.2, 0.1])).repeat(6000, 1)[:, None, :]
    tok, _ = sample(lg)
    freq = torch.bincount(tok.flatten(), minlength=3).float() / 6000
    assert (freq - torch.tensor([0.7, 0.2, 0.1])).abs().max() < 0.03


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: any other --gpus value ends with a message and a non-zero
    status before the library or a device is touched."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_generate_refuses_requests_beyond_the_cache():
    """The fused decode step keeps its position in device memory and would silently drop keys past
    the cache; the request is checked on the host before anything runs."""
    from qtip_amd.llama_decode import FUSED_MAX_CACHE_LEN, LlamaConfig, LlamaDecoder, generate
    cfg = LlamaConfig(hidden=256, heads=4, kv_heads=2, layers=1, ffn=512, vocab=64)
    model = LlamaDecoder(cfg, max_cache_len=16, device="cpu")
    ids = torch.zeros((1, 10), dtype=torch.int64)
    with pytest.raises(ValueError, match="does not fit"):
        generate(model, ids, 8)  # positions up to 16 needed, slots 0..15 exist
    with pytest.raises(ValueError, match="does not fit"):
        generate(model, torch.zeros((1, 17), dtype=torch.int64), 1)
    assert model.supports_fused_decode()
    long = LlamaDecoder(cfg, max_cache_len=FUSED_MAX_CACHE_LEN + 1, device="cpu")
    assert not long.supports_fused_decode()  # generate() then decodes module by module
    with pytest.raises(ValueError, match="fused decode step covers"):
        long.decode_fused(torch.zeros((1, 1), dtype=torch.int64), torch.tensor([0]))
