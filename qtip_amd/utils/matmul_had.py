"""Randomised-Hadamard helpers on the HIP RHT kernel.

Counterpart of lib/utils/matmul_had.py: same names and argument meaning
(get_hadK, matmul_hadU_cuda, matmul_hadUt_cuda, op hadamard::hadamard).  The
reference runs a third-party CUDA Walsh-Hadamard kernel and then a dense
K x K matmul; here both steps (and optional sign / scale vectors) are one
kernel launch.  The order-K tables are the reference's
(lib/utils/matmul_had.py:129-95715), kept as packed sign bits in
hadamard_tables.npz.
"""
import os
import weakref

import numpy as np
import torch

from .. import ops

_ORDERS = (172, 156, 140, 124, 116, 108, 60, 52, 36, 28, 20, 12)
_npz = None
_float_tables = {}
_bit_cache = {}


def _table_signs(order):
    global _npz
    if _npz is None:
        _npz = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "hadamard_tables.npz"),
                       allow_pickle=False)
    bits = np.unpackbits(_npz[f"had{order}"])[:order * order].reshape(order, order)
    return bits  # 1 = -1


def is_pow2(n):
    return (n & (n - 1) == 0) and (n > 0)


def get_hadK(n, transpose=False):
    """(hadK float tensor or None, K): first table order dividing n in the
    reference's order of preference, cofactor must be a power of two
    (lib/utils/matmul_had.py:9-63)."""
    for order in _ORDERS:
        if n % order == 0:
            assert is_pow2(n // order)
            if order not in _float_tables:
                _float_tables[order] = torch.from_numpy(1.0 - 2.0 * _table_signs(order).astype(np.float32))
            had = _float_tables[order]
            return (had.T if transpose else had), order
    assert is_pow2(n)
    return None, 1


def _pack_bits(neg):
    """(K, K) boolean array neg[i][j] (True = -1) -> int32 words, column-major:
    bit j*K+i (little-endian) holds neg[i][j], the layout the kernel reads."""
    flat = np.ascontiguousarray(np.asarray(neg, dtype=np.uint8).T).reshape(-1)
    pad = (-flat.size) % 32
    flat = np.concatenate([flat, np.zeros(pad, dtype=np.uint8)])
    words = np.packbits(flat.reshape(-1, 8)[:, ::-1], axis=1).reshape(-1, 4)
    return np.ascontiguousarray(words).view("<u4").reshape(-1).view(np.int32)


def had_bits(hadK, K, transpose, device):
    """Device int32 tensor of sign bits for the kernel, cached.

    hadK may be None (the built-in table of order K is used) or the caller's
    K x K tensor (as QuantizedLinear hands in); a caller-supplied tensor is
    packed once per (storage, transpose) and must be a +-1 matrix.
    """
    dev = torch.device(device)
    if hadK is None or (K in _float_tables and hadK.data_ptr() == _float_tables[K].data_ptr()):
        key = (K, bool(transpose), dev)
        if key not in _bit_cache:
            neg = _table_signs(K).astype(bool)
            _bit_cache[key] = torch.from_numpy(_pack_bits(neg.T if transpose else neg)).to(dev)
        return _bit_cache[key]
    # a caller's own table: keyed by the memory it occupies, so a fresh view of the same table (what
    # a module hands in on every call) hits.  The entry holds a weak reference to the storage: while
    # that storage lives its address cannot belong to another tensor, and when it is freed the entry
    # goes with it (nothing of the caller's is kept alive).  An in-place change bumps `_version`.
    st = hadK.untyped_storage()
    key = (st.data_ptr(), hadK.storage_offset(), tuple(hadK.shape), tuple(hadK.stride()), hadK.dtype,
           bool(transpose), dev)
    hit = _bit_cache.get(key)
    if hit is None or hit[0]() is not st or hit[1] != hadK._version:
        h = hadK.detach().to("cpu", torch.float32).numpy()
        if h.shape != (K, K) or not np.all(np.abs(h) == 1.0):
            raise ValueError("hadK must be a K x K matrix of +-1")
        neg = h < 0
        # a K x K table equal to the built-in one shares the built-in entry
        if K in _ORDERS and np.array_equal(neg, _table_signs(K).astype(bool)):
            bits = had_bits(None, K, transpose, dev)
        else:
            bits = torch.from_numpy(_pack_bits(neg.T if transpose else neg)).to(dev)
        if hit is None or hit[0]() is not st:
            weakref.finalize(st, _bit_cache.pop, key, None)
        hit = (weakref.ref(st), hadK._version, bits)
        _bit_cache[key] = hit
    return hit[2]


_dense_cache = {}


def _dense_sylvester(p, device):
    """H_p (Sylvester order, +-1 fp32) on the device, cached."""
    key = ("sylvester", p, torch.device(device))
    if key not in _dense_cache:
        h = torch.ones(1, 1)
        while h.shape[0] < p:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        _dense_cache[key] = h.to(device)
    return _dense_cache[key]


# a transform with a large table order over many rows runs as library GEMMs (below); these are the
# sizes from which that is faster than the transform kernel, whose order * A workgroups per row
# each read the whole row.  Measured, kernel vs GEMMs: 11008 (172 x 64) 128 rows 208 vs 103 us,
# 512 rows 809 vs 90, 2048 rows 3114 vs 280; 22016 (172 x 128) 128 rows 336 vs 102; with the small
# orders (28 x 1024, 12 x 1024, 20 x 512) the kernel stays ahead at every row count.
MANY_ROWS_MIN = 96
MANY_ROWS_MIN_ORDER = 100
_MANY_ROWS_DENSE_P = 256


def rht_many_rows(x, hadK, K, transpose, pre=None, post=None, scale=None, out_dtype=None):
    """post * scale * (H_K (x) H_p)(pre * x) over the last axis of a (rows, n) fp16 / fp32 tensor,
    evaluated the way the reference does for every input (lib/utils/matmul_had.py:105-115: a
    dense K x K matmul with the table and a Walsh-Hadamard transform of the power-of-two part) -
    fp32 library GEMMs instead of the transform kernel.  For many rows and a large table order:
    the kernel's per-row cost grows with the order, a GEMM's does not."""
    rows, n = x.shape
    p = n // K
    dev = x.device
    table = (hadK if hadK is not None else get_hadK(n)[0]).to(device=dev, dtype=torch.float32)
    M = table.T if transpose else table
    z = x.to(torch.float32)
    if pre is not None:
        z = z * pre.to(torch.float32)
    z = torch.matmul(M, z.view(rows, K, p))  # the table over the K axis, batched over the rows
    if p <= _MANY_ROWS_DENSE_P:
        z = torch.matmul(z.reshape(rows * K, p), _dense_sylvester(p, dev))
    else:  # long power-of-two parts: one workgroup of the transform kernel per p-point vector
        z = z.reshape(rows * K, p).contiguous()
        z = torch.cat([ops.rht(z[i:i + 65535], scale=1.0) for i in range(0, rows * K, 65535)], 0)
    z = z.view(rows, n) * (n**-0.5 if scale is None else scale)
    if post is not None:
        z = z * post.to(torch.float32)
    return z.to(out_dtype or x.dtype)


torch.library.define("hadamard::hadamard", "(Tensor x, float scale) -> Tensor")


@torch.library.register_fake("hadamard::hadamard")
def hadamard_abstract(x: torch.Tensor, scale: float) -> torch.Tensor:
    return torch.empty_like(x)


@torch.library.impl("hadamard::hadamard", "cuda")
def hadamard(x: torch.Tensor, scale: float) -> torch.Tensor:
    """Sylvester-ordered Walsh-Hadamard transform along the last axis times scale
    (what fast_hadamard_transform.hadamard_transform computes for the
    reference, lib/utils/matmul_had.py:99-102).  Last axis must be a power of two."""
    if x.dtype not in (torch.float16, torch.float32):
        return ops.rht(x.float().contiguous(), scale=scale).to(x.dtype)
    return ops.rht(x.contiguous(), scale=scale)


class _HadamardFn(torch.autograd.Function):
    """y = (H_K (x) H_{n/K}) x / sqrt(n) with the gradient the reference gets from the autograd
    support of its Walsh-Hadamard package plus the dense hadK matmul: the transform is linear and
    orthonormal, so grad_x = (H_K^T (x) H_{n/K}) grad_y / sqrt(n) - the same kernel with the
    order-K table transposed."""

    @staticmethod
    def forward(ctx, X, hadK, K, transpose):
        ctx.hadK, ctx.K, ctx.transpose = hadK, K, transpose
        return _hadU(X, hadK, K, transpose)

    @staticmethod
    def backward(ctx, grad):
        return _hadU(grad.contiguous(), ctx.hadK, ctx.K, not ctx.transpose), None, None, None


def _hadU(X, hadK, K, transpose):
    n = X.shape[-1]
    if K == 1:
        return torch.ops.hadamard.hadamard(X.contiguous(), n**(-0.5))
    x = X if X.dtype in (torch.float16, torch.float32) else X.float()
    rows = x.numel() // n
    if rows >= MANY_ROWS_MIN and K >= MANY_ROWS_MIN_ORDER:
        return rht_many_rows(x.reshape(rows, n), hadK, K, transpose).to(X.dtype).reshape(X.shape)
    out = ops.rht(x.contiguous(), order=K, had_bits=had_bits(hadK, K, transpose, X.device), out_dtype=x.dtype)
    return out.to(X.dtype).reshape(X.shape)


def matmul_hadU_cuda(X, hadK, K, transpose=False):
    """(H_K (x) H_{n/K}) X / sqrt(n) along the last axis (lib/utils/matmul_had.py:105-115);
    differentiable with respect to X."""
    if torch.is_grad_enabled() and X.requires_grad:
        return _HadamardFn.apply(X, hadK, K, transpose)
    return _hadU(X, hadK, K, transpose)


def matmul_hadUt_cuda(X, hadK, K):
    return matmul_hadU_cuda(X, hadK, K, transpose=True)
