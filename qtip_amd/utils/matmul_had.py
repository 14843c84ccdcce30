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
    key = (hadK.data_ptr(), hadK._version, tuple(hadK.shape), tuple(hadK.stride()), bool(transpose), dev)
    if key not in _bit_cache:
        h = hadK.detach().to("cpu", torch.float32).numpy()
        if h.shape != (K, K) or not np.all(np.abs(h) == 1.0):
            raise ValueError("hadK must be a K x K matrix of +-1")
        neg = h < 0
        _bit_cache[key] = torch.from_numpy(_pack_bits(neg.T if transpose else neg)).to(dev)
    return _bit_cache[key]


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
