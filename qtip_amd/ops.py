"""Tensor-level wrappers over the C ABI (include/qtip_hip.h).

Every function launches on the current stream of the tensors' device and
returns without synchronising.  Inputs are checked here (device, dtype,
contiguity, sizes) so that a bad argument raises instead of reaching a kernel.
"""
import ctypes
import math

import torch

from . import _lib
from ._lib import QTIP_F16, QTIP_F32, check, lib, require_cuda, stream_ptr

_DT = {torch.float16: QTIP_F16, torch.float32: QTIP_F32}

# per-device scratch for the partial sums of the split-k matvec
_WORKSPACE = {}
_WORKSPACE_BYTES = 8 << 20
_SPLIT = {}


def _workspace(device, need):
    key = device.index if device.index is not None else torch.cuda.current_device()
    ws = _WORKSPACE.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, _WORKSPACE_BYTES), dtype=torch.uint8, device=device)
        _WORKSPACE[key] = ws
    return ws


def matvec_split(m, k, bits, device):
    """Number of k splits the matvec kernel uses for this shape (cached per device)."""
    key = (m, k, bits, device.index)
    s = _SPLIT.get(key)
    if s is None:
        with torch.cuda.device(device):
            s = lib().qtip_matvec_split(m, k, bits)
        if s < 1:
            raise ValueError(f"unsupported matvec shape {m}x{k} at {bits} bits")
        _SPLIT[key] = s
    return s


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _check_packed(packed, m, k, bits):
    require_cuda(packed, "packed trellis", (torch.int16, torch.uint16, torch.int32, torch.uint8))
    if bits not in (2, 3, 4):
        raise ValueError(f"bits must be 2, 3 or 4 (got {bits})")
    if m % 32 or k % 32 or m <= 0 or k <= 0:
        raise ValueError(f"shape {m}x{k}: m and k must be positive multiples of 32")
    nbytes = packed.numel() * packed.element_size()
    if nbytes * 8 != bits * m * k:
        raise ValueError(f"packed trellis holds {nbytes} bytes, {m}x{k} at {bits} bits needs {bits * m * k // 8}")


def _check_tlut(tlut, device):
    require_cuda(tlut, "codebook (tlut)", torch.float16)
    if tlut.numel() != 1024:
        raise ValueError(f"codebook must hold 512 x 2 fp16 values (got {tuple(tlut.shape)})")
    if tlut.device != device:
        raise ValueError("codebook is on a different device")


def decode(packed, tlut, m, k, bits):
    """Kernel-packed trellis -> dense (m, k) fp16 weight matrix (bit-exact)."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    out = torch.empty((m, k), dtype=torch.float16, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decode(_ptr(out), _ptr(packed), _ptr(tlut), m, k, bits, stream_ptr(packed.device)),
              "qtip_decode")
    return out


def decompress_matvec(packed, x, tlut, m, k, bits, out=None, split_k=True):
    """out[m] fp32 = decode(packed)[m,k] @ x[k]; x is fp16 with k elements."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(x, "x", torch.float16)
    if x.numel() != k or x.device != packed.device:
        raise ValueError(f"x must hold {k} fp16 values on {packed.device}")
    if out is None:
        out = torch.empty((m,), dtype=torch.float32, device=packed.device)
    else:
        require_cuda(out, "out", torch.float32)
        if out.numel() != m:
            raise ValueError(f"out must hold {m} fp32 values")
    L = lib()
    if split_k and matvec_split(m, k, bits, packed.device) > 1:
        ws = _workspace(packed.device, 16 * m * 4)
        wsp, wsb = _ptr(ws), ws.numel()
    else:
        wsp, wsb = ctypes.c_void_p(0), 0
    with torch.cuda.device(packed.device):
        check(L.qtip_decompress_matvec(_ptr(out), _ptr(packed), _ptr(x), _ptr(tlut), m, k, bits, wsp, wsb,
                                       stream_ptr(packed.device)), "qtip_decompress_matvec")
    return out


def decompress_matvec_parts(packed, x, tlut, m, k, bits):
    """(S, m) fp32 partial sums of decode(packed) @ x over S ranges of k; their
    sum over axis 0 (in order) is the matvec.  S = matvec_split(...)."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(x, "x", torch.float16)
    if x.numel() != k or x.device != packed.device:
        raise ValueError(f"x must hold {k} fp16 values on {packed.device}")
    S = matvec_split(m, k, bits, packed.device)
    parts = torch.empty((S, m), dtype=torch.float32, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decompress_matvec_parts(_ptr(parts), _ptr(packed), _ptr(x), _ptr(tlut), m, k, bits, S,
                                                 stream_ptr(packed.device)), "qtip_decompress_matvec_parts")
    return parts


def decompress_gemm(packed, x, tlut, m, k, bits, round_f16=True):
    """(batch, m) fp32 = x[batch,k] (fp16) @ decode(packed)[m,k]^T on the matrix cores."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(x, "x", torch.float16)
    if x.dim() != 2 or x.shape[1] != k or x.device != packed.device:
        raise ValueError(f"x must be (batch, {k}) fp16 on {packed.device}")
    batch = x.shape[0]
    out = torch.empty((batch, m), dtype=torch.float32, device=packed.device)
    if batch == 0:
        return out
    with torch.cuda.device(packed.device):
        check(lib().qtip_decompress_gemm(_ptr(out), _ptr(packed), _ptr(x), _ptr(tlut), m, k, bits, batch,
                                         int(bool(round_f16)), stream_ptr(packed.device)), "qtip_decompress_gemm")
    return out


def rht(x, order=1, had_bits=None, pre=None, post=None, scale=None, out_dtype=None, in_parts=1):
    """out[r] = post * scale * (H_order (x) H_p)(pre * x[r]) over the last axis.

    x: (..., n) fp16 or fp32 (with in_parts > 1: (in_parts, ..., n), summed on load).
    had_bits: int32 device tensor of packed sign bits for order > 1.
    scale defaults to n ** -0.5.
    """
    require_cuda(x, "x", (torch.float16, torch.float32))
    n = x.shape[-1]
    rows = x.numel() // n // in_parts
    if n % order:
        raise ValueError(f"order {order} does not divide {n}")
    p = n // order
    if p & (p - 1):
        raise ValueError(f"{n} / {order} = {p} is not a power of two")
    if order > 1:
        require_cuda(had_bits, "had_bits", torch.int32)
        if had_bits.numel() * 32 < order * order:
            raise ValueError("had_bits too short")
    if pre is not None:
        require_cuda(pre, "pre", torch.float16)
        if pre.numel() != n:
            raise ValueError(f"pre must hold {n} values")
    if post is not None:
        require_cuda(post, "post", torch.float32)
        if post.numel() != n:
            raise ValueError(f"post must hold {n} values")
    out_dtype = out_dtype or x.dtype
    shape = x.shape[1:] if in_parts > 1 else x.shape
    out = torch.empty(shape, dtype=out_dtype, device=x.device)
    if rows == 0:
        return out
    if scale is None:
        scale = n ** -0.5
    with torch.cuda.device(x.device):
        # rows beyond the grid limit are processed in slices
        xf = x.reshape(in_parts, rows, n) if in_parts > 1 else x.reshape(rows, n)
        of = out.reshape(rows, n)
        step = 65535 if in_parts == 1 else rows
        if in_parts > 1 and rows > 65535:
            raise ValueError("too many rows for a split input")
        for r0 in range(0, rows, step):
            r1 = min(rows, r0 + step)
            src = xf if in_parts > 1 else xf[r0:r1]
            check(lib().qtip_rht(_ptr(of[r0:r1]), _DT[out_dtype], _ptr(src), _DT[x.dtype], in_parts, r1 - r0, n,
                                 order, _ptr(had_bits), _ptr(pre), _ptr(post), ctypes.c_float(scale),
                                 stream_ptr(x.device)), "qtip_rht")
    return out
