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

# scratch for split-k partial sums, one buffer per (device, stream): launches on one stream are
# ordered, launches on different streams must not share partial results
_WORKSPACE = {}
_WORKSPACE_BYTES = 8 << 20
_SPLIT = {}


def _workspace(device, need):
    """Scratch of at least `need` bytes for the current stream.  A request beyond the current
    buffer gets a larger one, and the smaller ones stay alive for the life of the process: a
    HIP graph recorded earlier still holds their addresses."""
    dev = device.index if device.index is not None else torch.cuda.current_device()
    key = (dev, torch.cuda.current_stream(device).cuda_stream)
    held = _WORKSPACE.setdefault(key, [])
    if not held or held[-1].numel() < need:
        held.append(torch.empty(max(need, _WORKSPACE_BYTES), dtype=torch.uint8, device=device))
    return held[-1]


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


def decompress_matvec_parts(packed, x, tlut, m, k, bits, nparts=None):
    """(S, m) fp32 partial sums of decode(packed) @ x over S ranges of k; their
    sum over axis 0 (in order) is the matvec.  S = nparts or matvec_split(...)."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(x, "x", torch.float16)
    if x.numel() != k or x.device != packed.device:
        raise ValueError(f"x must hold {k} fp16 values on {packed.device}")
    S = int(nparts) if nparts is not None else matvec_split(m, k, bits, packed.device)
    parts = torch.empty((S, m), dtype=torch.float32, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decompress_matvec_parts(_ptr(parts), _ptr(packed), _ptr(x), _ptr(tlut), m, k, bits, S,
                                                 stream_ptr(packed.device)), "qtip_decompress_matvec_parts")
    return parts


RHT_IN_MATVEC_SIZES = (2048, 4096, 8192)


def decompress_matvec_parts_rht(packed, x_raw, su, scale, tlut, m, k, bits, nparts=None):
    """(S, m) fp32 partial sums of decode(packed) @ fp16(scale * H_k(su * x_raw)): the input
    transform of the layer runs inside the matvec launch (k in RHT_IN_MATVEC_SIZES)."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(x_raw, "x", torch.float16)
    require_cuda(su, "su", torch.float16)
    if k not in RHT_IN_MATVEC_SIZES or x_raw.numel() != k or su.numel() != k:
        raise ValueError(f"x and su must hold k = {k} fp16 values, k in {RHT_IN_MATVEC_SIZES}")
    if x_raw.device != packed.device or su.device != packed.device:
        raise ValueError(f"x and su must be on {packed.device}")
    S = int(nparts) if nparts is not None else matvec_split(m, k, bits, packed.device)
    parts = torch.empty((S, m), dtype=torch.float32, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decompress_matvec_parts_rht(_ptr(parts), _ptr(packed), _ptr(x_raw), _ptr(su),
                                                     ctypes.c_float(scale), _ptr(tlut), m, k, bits, S,
                                                     stream_ptr(packed.device)), "qtip_decompress_matvec_parts_rht")
    return parts


def decompress_matvec_parts_chain(packed, tlut, m, k, bits, prev_parts, post, scale_out, residual, norm_weight, eps,
                                  su, scale_in, nparts=None):
    """(parts, x_new): the boundary between two linear layers and the second layer's matvec in
    one launch - x_new = fp16(residual + fp16(post * scale_out * H(sum(prev_parts)))),
    parts = decode(packed) @ fp16(scale_in * H(su * rmsnorm(x_new))), the (S, m) fp32 partial sums.
    prev_parts: (S_prev, k) or (S_prev, 1, k) fp32; k in RHT_IN_MATVEC_SIZES."""
    _check_packed(packed, m, k, bits)
    _check_tlut(tlut, packed.device)
    require_cuda(prev_parts, "prev_parts", torch.float32)
    require_cuda(post, "post", torch.float32)
    require_cuda(residual, "residual", torch.float16)
    require_cuda(norm_weight, "norm_weight", torch.float16)
    require_cuda(su, "su", torch.float16)
    pp = prev_parts.reshape(prev_parts.shape[0], -1)
    if k not in RHT_IN_MATVEC_SIZES or pp.shape[1] != k:
        raise ValueError(f"prev_parts must hold vectors of k = {k} values, k in {RHT_IN_MATVEC_SIZES}")
    if any(t.numel() != k for t in (post, residual, norm_weight, su)):
        raise ValueError(f"post, residual, norm_weight and su must hold k = {k} values")
    if any(t.device != packed.device for t in (pp, post, residual, norm_weight, su)):
        raise ValueError(f"all operands must be on {packed.device}")
    S = int(nparts) if nparts is not None else matvec_split(m, k, bits, packed.device)
    parts = torch.empty((S, m), dtype=torch.float32, device=packed.device)
    x_new = torch.empty((1, k), dtype=torch.float16, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decompress_matvec_parts_chain(
            _ptr(parts), _ptr(packed), _ptr(tlut), m, k, bits, S, _ptr(pp), pp.shape[0], ctypes.c_size_t(pp.stride(0)),
            _ptr(post), ctypes.c_float(scale_out), _ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), _ptr(su),
            ctypes.c_float(scale_in), _ptr(x_new), stream_ptr(packed.device)), "qtip_decompress_matvec_parts_chain")
    return parts, x_new


def decompress_matvec_group_chain(packed, tlut, m, k, bits, prev_parts, post, scale_out, residual, norm_weight, eps,
                                  su, scale_in, nparts=None):
    """decompress_matvec_parts_chain for up to three matrices that share the boundary and the
    input (separate q / k / v or gate / up projections) in one launch.  packed, tlut, m, su: lists,
    one entry per matrix.  Returns (parts (S, sum(m)) fp32 - matrix g's rows after those of
    matrix g - 1 -, x_new)."""
    n = len(packed)
    if not (1 <= n <= 3) or len(tlut) != n or len(m) != n or len(su) != n:
        raise ValueError("one to three matrices, with one table, row count and sign vector each")
    dev = packed[0].device
    for g in range(n):
        _check_packed(packed[g], m[g], k, bits)
        _check_tlut(tlut[g], dev)
        require_cuda(su[g], "su", torch.float16)
        if su[g].numel() != k or su[g].device != dev or packed[g].device != dev:
            raise ValueError(f"every su must hold k = {k} values on {dev}")
    require_cuda(prev_parts, "prev_parts", torch.float32)
    require_cuda(post, "post", torch.float32)
    require_cuda(residual, "residual", torch.float16)
    require_cuda(norm_weight, "norm_weight", torch.float16)
    pp = prev_parts.reshape(prev_parts.shape[0], -1)
    if k not in RHT_IN_MATVEC_SIZES or pp.shape[1] != k:
        raise ValueError(f"prev_parts must hold vectors of k = {k} values, k in {RHT_IN_MATVEC_SIZES}")
    if any(t.numel() != k for t in (post, residual, norm_weight)):
        raise ValueError(f"post, residual and norm_weight must hold k = {k} values")
    m_total = int(sum(m))
    S = int(nparts) if nparts is not None else matvec_split(m_total, k, bits, dev)
    parts = torch.empty((S, m_total), dtype=torch.float32, device=dev)
    x_new = torch.empty((1, k), dtype=torch.float16, device=dev)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    with torch.cuda.device(dev):
        check(lib().qtip_decompress_matvec_group_chain(
            _ptr(parts), n, ptrs(packed), ptrs(tlut), ptrs(su), (ctypes.c_int * n)(*[int(v) for v in m]), k, bits, S,
            _ptr(pp), pp.shape[0], ctypes.c_size_t(pp.stride(0)), _ptr(post), ctypes.c_float(scale_out),
            _ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), ctypes.c_float(scale_in), _ptr(x_new),
            stream_ptr(dev)), "qtip_decompress_matvec_group_chain")
    return parts, x_new


def decompress_matvec_group(packed, x, tlut, m, k, bits, nparts=None):
    """Up to three matvecs of the same k and bit width in one launch, matrix g on its own fp16
    input x[g] (k values each; rows of one tensor will do).  Returns parts (S, sum(m)) fp32."""
    n = len(packed)
    if not (1 <= n <= 3) or len(tlut) != n or len(m) != n or len(x) != n:
        raise ValueError("one to three matrices, with one table, row count and input each")
    dev = packed[0].device
    for g in range(n):
        _check_packed(packed[g], m[g], k, bits)
        _check_tlut(tlut[g], dev)
        require_cuda(x[g], "x", torch.float16)
        if x[g].numel() != k or x[g].device != dev or packed[g].device != dev:
            raise ValueError(f"every x must hold k = {k} values on {dev}")
    m_total = int(sum(m))
    if nparts is not None:
        S = int(nparts)
    else:
        S = matvec_split(m_total, k, bits, dev)
        while k * 2 > S * 28 * 1024:  # every k range of x has to fit the kernel's staging area
            S *= 2
    parts = torch.empty((S, m_total), dtype=torch.float32, device=dev)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    with torch.cuda.device(dev):
        check(lib().qtip_decompress_matvec_group(_ptr(parts), n, ptrs(packed), ptrs(x), ptrs(tlut),
                                                 (ctypes.c_int * n)(*[int(v) for v in m]), k, bits, S,
                                                 stream_ptr(dev)), "qtip_decompress_matvec_group")
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
    L = lib()
    with torch.cuda.device(packed.device):
        need = L.qtip_gemm_workspace_bytes(m, k, bits, batch)
        if need:
            ws = _workspace(packed.device, need)
            wsp, wsb = _ptr(ws), ws.numel()
        else:
            wsp, wsb = ctypes.c_void_p(0), 0
        check(L.qtip_decompress_gemm(_ptr(out), _ptr(packed), _ptr(x), _ptr(tlut), m, k, bits, batch,
                                     int(bool(round_f16)), wsp, wsb, stream_ptr(packed.device)),
              "qtip_decompress_gemm")
    return out


PRE_NONE, PRE_RMSNORM, PRE_SILU_MUL = 0, 1, 2


def rht(x, order=1, had_bits=None, pre=None, post=None, scale=None, out_dtype=None, in_parts=1, pre_mode=PRE_NONE,
        norm_weight=None, eps=0.0, residual=None):
    """out[r] = post * scale * (H_order (x) H_p)(pre * f(x[r])) (+ residual) over the last axis.

    x: (..., n) fp16 or fp32 (with in_parts > 1: (in_parts, ..., n), summed on load).
    had_bits: int32 device tensor of packed sign bits for order > 1.  scale defaults to n ** -0.5.
    pre_mode / norm_weight / eps / residual: element-wise work of the surrounding layer folded
    into the same launch (see qtip_rht_fused in include/qtip_hip.h); with PRE_SILU_MUL the last
    axis of x holds [gate | up] and n is half of it.
    """
    require_cuda(x, "x", (torch.float16, torch.float32))
    n = x.shape[-1]
    if pre_mode == PRE_SILU_MUL:
        if n % 2:
            raise ValueError("gate|up input needs an even last dimension")
        n //= 2
    rows = x.numel() // x.shape[-1] // in_parts
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
    shape = list(x.shape[1:] if in_parts > 1 else x.shape)
    shape[-1] = n
    fused = pre_mode != PRE_NONE or residual is not None
    if pre_mode == PRE_RMSNORM:
        require_cuda(norm_weight, "norm_weight", torch.float16)
        if norm_weight.numel() != n or x.dtype != torch.float16:
            raise ValueError("RMSNorm prologue needs an fp16 input and an fp16 weight of the same length")
    if pre_mode not in (PRE_NONE, PRE_RMSNORM, PRE_SILU_MUL) or (pre_mode != PRE_NONE and in_parts != 1):
        raise ValueError("bad pre_mode")
    if residual is not None:
        require_cuda(residual, "residual", torch.float16)
        if out_dtype != torch.float16 or residual.numel() != rows * n:
            raise ValueError("residual needs fp16 output and one value per output element")
    out = torch.empty(shape, dtype=out_dtype, device=x.device)
    if rows == 0:
        return out
    if scale is None:
        scale = n ** -0.5
    L = lib()
    with torch.cuda.device(x.device):
        width = x.shape[-1]
        xf = x.reshape(in_parts, rows, width) if in_parts > 1 else x.reshape(rows, width)
        of = out.reshape(rows, n)
        rf = residual.reshape(rows, n) if residual is not None else None
        step = 65535 if in_parts == 1 else rows
        if in_parts > 1 and rows > 65535:
            raise ValueError("too many rows for a split input")
        for r0 in range(0, rows, step):
            r1 = min(rows, r0 + step)
            src = xf if in_parts > 1 else xf[r0:r1]
            if fused:
                check(L.qtip_rht_fused(_ptr(of[r0:r1]), _DT[out_dtype], _ptr(src), _DT[x.dtype], in_parts, r1 - r0, n,
                                       order, _ptr(had_bits), _ptr(pre), _ptr(post), ctypes.c_float(scale), pre_mode,
                                       _ptr(norm_weight), ctypes.c_float(eps),
                                       _ptr(rf[r0:r1]) if rf is not None else _ptr(None),
                                       stream_ptr(x.device)), "qtip_rht_fused")
            else:
                check(L.qtip_rht(_ptr(of[r0:r1]), _DT[out_dtype], _ptr(src), _DT[x.dtype], in_parts, r1 - r0, n,
                                 order, _ptr(had_bits), _ptr(pre), _ptr(post), ctypes.c_float(scale),
                                 stream_ptr(x.device)), "qtip_rht")
    return out


def rht_fused_pre_rows(x, pre_rows, norm_weight, eps, order=1, had_bits=None, scale=None):
    """Input transforms of `rows` layers that read the same fp16 vector x (n values), one launch:
    row r = fp16(scale * H^T(pre_rows[r] * rmsnorm(x))).  pre_rows (rows, n) fp16.  -> (rows, n)."""
    require_cuda(x, "x", torch.float16)
    require_cuda(pre_rows, "pre_rows", torch.float16)
    require_cuda(norm_weight, "norm_weight", torch.float16)
    n = x.numel()
    if pre_rows.dim() != 2 or pre_rows.shape[1] != n or norm_weight.numel() != n or pre_rows.shape[0] > 65535:
        raise ValueError("pre_rows must be (rows, n) and norm_weight hold n values")
    p = n // order
    if n % order or p & (p - 1):
        raise ValueError(f"{n} is not {order} times a power of two")
    if order > 1:
        require_cuda(had_bits, "had_bits", torch.int32)
    out = torch.empty_like(pre_rows)
    with torch.cuda.device(x.device):
        check(lib().qtip_rht_fused_pre_rows(_ptr(out), _ptr(x), pre_rows.shape[0], n, order, _ptr(had_bits),
                                            _ptr(pre_rows), ctypes.c_float(scale if scale is not None else n ** -0.5),
                                            _ptr(norm_weight), ctypes.c_float(eps), stream_ptr(x.device)),
              "qtip_rht_fused_pre_rows")
    return out


def rht_post_rows(parts, post_rows, order=1, had_bits=None, scale=None, out_dtype=torch.float16):
    """Output transforms of `rows` layers of the same size in one launch: parts (S, rows, n) fp32
    (summed over S on load), post_rows (rows, n) fp32, one vector per row.  Returns (rows, n)."""
    require_cuda(parts, "parts", torch.float32)
    require_cuda(post_rows, "post_rows", torch.float32)
    if parts.dim() != 3 or post_rows.shape != parts.shape[1:]:
        raise ValueError("parts must be (S, rows, n) and post_rows (rows, n)")
    S, rows, n = parts.shape
    p = n // order
    if n % order or p & (p - 1) or rows > 65535:
        raise ValueError(f"{n} is not {order} times a power of two, or too many rows")
    if order > 1:
        require_cuda(had_bits, "had_bits", torch.int32)
    out = torch.empty((rows, n), dtype=out_dtype, device=parts.device)
    with torch.cuda.device(parts.device):
        check(lib().qtip_rht_post_rows(_ptr(out), _DT[out_dtype], _ptr(parts), _DT[torch.float32], S, rows, n, order,
                                       _ptr(had_bits), _ptr(post_rows),
                                       ctypes.c_float(scale if scale is not None else n ** -0.5),
                                       stream_ptr(parts.device)), "qtip_rht_post_rows")
    return out


def rht_silu_pair(parts, post, order=1, had_bits=None, scale=None):
    """fp16(fp16(silu(gate)) * up) of the transformed gate / up outputs in one launch.
    parts (S, n) fp32 with post (n,): gate and up are the halves of one transformed vector
    (returns (n / 2,)); parts (S, 2, n) with post (2, n): a transformed vector each (returns (n,))."""
    require_cuda(parts, "parts", torch.float32)
    require_cuda(post, "post", torch.float32)
    two = parts.dim() == 3
    if parts.dim() not in (2, 3) or post.shape != parts.shape[1:] or (two and parts.shape[1] != 2):
        raise ValueError("parts must be (S, n) with post (n,), or (S, 2, n) with post (2, n)")
    S, n = parts.shape[0], parts.shape[-1]
    if order > 1:
        require_cuda(had_bits, "had_bits", torch.int32)
    out = torch.empty(n if two else n // 2, dtype=torch.float16, device=parts.device)
    with torch.cuda.device(parts.device):
        check(lib().qtip_rht_silu_pair(_ptr(out), _ptr(parts), S, int(two), n, order, _ptr(had_bits), _ptr(post),
                                       ctypes.c_float(scale if scale is not None else n ** -0.5),
                                       stream_ptr(parts.device)), "qtip_rht_silu_pair")
    return out


def rht_silu_pair_ok(n, order, two_vectors):
    """Shapes qtip_rht_silu_pair takes (the vectorised form of the transform: rows of >= 8 values
    per workgroup, whole rows of the table mix for either half)."""
    p = n // order
    if n % order or p & (p - 1) or n <= 4096 or (not two_vectors and order % 2):
        return False
    pp, log_a = p, 0
    while pp > 1024:  # values per workgroup of the transform kernels
        pp >>= 1
        log_a += 1
    while pp > 64 and (order << (log_a + 1)) <= 64:
        pp >>= 1
        log_a += 1
    return pp >= 8


ATTN_MAX_KEY_SPLITS = 16


ATTN_SPLIT_FROM = 1024  # context length from which the key-range form is faster


def attention_key_splits(context):
    """Key ranges per head for decode attention over a context of `context` tokens: one workgroup
    per head below ATTN_SPLIT_FROM keys (the ranges cost a second small launch: 32 heads of 128,
    127 keys 5.8 vs 11.5 us), 8 ranges from there on (2047 keys 22.8 -> 12.9 us, 4095 keys
    40 -> 20.6 us, which is the time the 67 MB of keys and values take to arrive)."""
    return 1 if context < ATTN_SPLIT_FROM else 8


def _split_workspace(device, heads, head_dim, key_splits):
    if not 1 <= key_splits <= ATTN_MAX_KEY_SPLITS:
        raise ValueError(f"key_splits must be in 1..{ATTN_MAX_KEY_SPLITS} (got {key_splits})")
    if key_splits == 1:
        return None
    return torch.empty(heads * key_splits * (head_dim + 2), dtype=torch.float32, device=device)


def decode_attention(qkv, k_cache, v_cache, pos, inv_freq, heads, kv_heads, head_dim, key_splits=1):
    """Attention output (heads*head_dim,) fp16 of one new token: RoPE, cache write at `pos`
    (device int64 tensor with one element) and attention over cache slots 0..pos in one launch.
    k_cache / v_cache: (1, kv_heads, max_len, head_dim) fp16, updated in place."""
    require_cuda(qkv, "qkv", torch.float16)
    require_cuda(k_cache, "k_cache", torch.float16)
    require_cuda(v_cache, "v_cache", torch.float16)
    require_cuda(pos, "pos", torch.int64)
    require_cuda(inv_freq, "inv_freq", torch.float32)
    max_len = k_cache.shape[-2]
    if qkv.numel() != (heads + 2 * kv_heads) * head_dim or k_cache.numel() != kv_heads * max_len * head_dim \
            or v_cache.shape != k_cache.shape or inv_freq.numel() != head_dim // 2 or pos.numel() != 1:
        raise ValueError("decode_attention: inconsistent shapes")
    out = torch.empty(heads * head_dim, dtype=torch.float16, device=qkv.device)
    ws = _split_workspace(qkv.device, heads, head_dim, key_splits)
    with torch.cuda.device(qkv.device):
        check(lib().qtip_decode_attention(_ptr(out), _ptr(qkv), _ptr(k_cache), _ptr(v_cache), _ptr(pos),
                                          _ptr(inv_freq), heads, kv_heads, head_dim, max_len, key_splits, _ptr(ws),
                                          stream_ptr(qkv.device)), "qtip_decode_attention")
    return out


def decode_attention_rht(parts, post, scale, had_bits, order, k_cache, v_cache, pos, inv_freq, heads, kv_heads,
                         head_dim, key_splits=1):
    """decode_attention on the qkv projection's raw matvec result `parts` (S, n) fp32: the
    projection's output transform (order x power-of-two Hadamard, * post * scale, cast to fp16) runs
    in the attention kernel's prologue.  had_bits: the table's packed sign bits (None for order 1)."""
    require_cuda(parts, "parts", torch.float32)
    require_cuda(k_cache, "k_cache", torch.float16)
    require_cuda(v_cache, "v_cache", torch.float16)
    require_cuda(pos, "pos", torch.int64)
    require_cuda(inv_freq, "inv_freq", torch.float32)
    if post is not None:
        require_cuda(post, "post", torch.float32)
    if had_bits is not None:
        require_cuda(had_bits, "had_bits", torch.int32)
    n = (heads + 2 * kv_heads) * head_dim
    parts = parts.reshape(-1, n)
    max_len = k_cache.shape[-2]
    if k_cache.numel() != kv_heads * max_len * head_dim or v_cache.shape != k_cache.shape \
            or inv_freq.numel() != head_dim // 2 or pos.numel() != 1 or (post is not None and post.numel() != n) \
            or (order > 1 and had_bits is None):
        raise ValueError("decode_attention_rht: inconsistent shapes")
    out = torch.empty(heads * head_dim, dtype=torch.float16, device=parts.device)
    ws = _split_workspace(parts.device, heads, head_dim, key_splits)
    with torch.cuda.device(parts.device):
        check(lib().qtip_decode_attention_rht(_ptr(out), _ptr(parts), parts.shape[0], parts.stride(0),
                                              _ptr(post) if post is not None else None, float(scale),
                                              _ptr(had_bits) if had_bits is not None else None, int(order),
                                              _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(inv_freq), heads,
                                              kv_heads, head_dim, max_len, key_splits, _ptr(ws),
                                              stream_ptr(parts.device)),
              "qtip_decode_attention_rht")
    return out


def decode_attention_rht3(parts, post, scale, had_bits, order, k_cache, v_cache, pos, inv_freq, heads, kv_heads,
                          head_dim, key_splits=1):
    """decode_attention_rht for separate q / k / v projections: parts, post, scale, had_bits and
    order are 3-element lists (q, k, v); the three `parts` are (S, n_i) fp32 views into one
    partial-sum buffer (same number of parts and the same row stride)."""
    for i in range(3):
        require_cuda(parts[i], "parts", torch.float32, contiguous=False)
        if post[i] is not None:
            require_cuda(post[i], "post", torch.float32)
        if had_bits[i] is not None:
            require_cuda(had_bits[i], "had_bits", torch.int32)
        n = (heads if i == 0 else kv_heads) * head_dim
        if parts[i].dim() != 2 or parts[i].shape[1] != n or parts[i].stride(1) != 1 \
                or parts[i].shape[0] != parts[0].shape[0] or parts[i].stride(0) != parts[0].stride(0) \
                or (post[i] is not None and post[i].numel() != n) or (order[i] > 1 and had_bits[i] is None):
            raise ValueError("decode_attention_rht3: inconsistent shapes")
    require_cuda(k_cache, "k_cache", torch.float16)
    require_cuda(v_cache, "v_cache", torch.float16)
    require_cuda(pos, "pos", torch.int64)
    require_cuda(inv_freq, "inv_freq", torch.float32)
    max_len = k_cache.shape[-2]
    if k_cache.numel() != kv_heads * max_len * head_dim or v_cache.shape != k_cache.shape \
            or inv_freq.numel() != head_dim // 2 or pos.numel() != 1:
        raise ValueError("decode_attention_rht3: inconsistent shapes")
    dev = parts[0].device
    out = torch.empty(heads * head_dim, dtype=torch.float16, device=dev)
    ws = _split_workspace(dev, heads, head_dim, key_splits)
    vp = lambda ts: (ctypes.c_void_p * 3)(*[t.data_ptr() if t is not None else None for t in ts])
    with torch.cuda.device(dev):
        check(lib().qtip_decode_attention_rht3(_ptr(out), vp(parts), parts[0].shape[0], parts[0].stride(0), vp(post),
                                               (ctypes.c_float * 3)(*[float(v) for v in scale]), vp(had_bits),
                                               (ctypes.c_int * 3)(*[int(v) for v in order]), _ptr(k_cache),
                                               _ptr(v_cache), _ptr(pos), _ptr(inv_freq), heads, kv_heads, head_dim,
                                               max_len, key_splits, _ptr(ws), stream_ptr(dev)),
              "qtip_decode_attention_rht3")
    return out


def rmsnorm(x, weight, eps):
    """weight * fp16(x * rsqrt(mean(x^2) + eps)) for one fp16 vector (model/llama.py:129-135)."""
    require_cuda(x, "x", torch.float16)
    require_cuda(weight, "weight", torch.float16)
    if x.numel() != weight.numel():
        raise ValueError("rmsnorm: x and weight differ in length")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        check(lib().qtip_rmsnorm(_ptr(out), _ptr(x), _ptr(weight), float(eps), x.numel(), stream_ptr(x.device)),
              "qtip_rmsnorm")
    return out


def greedy_pick(logits, tok, pos, history=None, history_base=0):
    """tok[0] = argmax(logits) (fp16 logits of one position, first index among equal maxima),
    history[pos - history_base] = tok when that slot exists, pos += 1 - the per-token bookkeeping
    of a greedy generation loop (eval/interactive_gen.py:43-69) in one launch, in place."""
    require_cuda(logits, "logits", torch.float16)
    require_cuda(tok, "tok", torch.int64)
    require_cuda(pos, "pos", torch.int64)
    if history is not None:
        require_cuda(history, "history", torch.int64)
    if tok.numel() != 1 or pos.numel() != 1:
        raise ValueError("greedy_pick: tok and pos hold one element each")
    with torch.cuda.device(logits.device):
        check(lib().qtip_greedy_pick(_ptr(logits), logits.numel(), _ptr(tok), _ptr(pos),
                                     _ptr(history) if history is not None else None,
                                     history.numel() if history is not None else 0, int(history_base),
                                     stream_ptr(logits.device)), "qtip_greedy_pick")


SAMPLE_PICK_MAX_TOP_K = 64


def sample_pick(logits, temperature, top_k, seed, counter, tok, pos, history=None, history_base=0):
    """Draw tok[0] from softmax(logits / temperature) restricted to the top_k largest logits
    (None: all), as eval/interactive_gen.py:15-40 does, with the bookkeeping of greedy_pick, in
    one launch.  counter: device int64 draw counter (advanced in place); seed: host integer."""
    require_cuda(logits, "logits", torch.float16)
    require_cuda(tok, "tok", torch.int64)
    require_cuda(pos, "pos", torch.int64)
    require_cuda(counter, "counter", torch.int64)
    if history is not None:
        require_cuda(history, "history", torch.int64)
    k = 0 if top_k is None else int(top_k)
    if tok.numel() != 1 or pos.numel() != 1 or counter.numel() != 1 or not (0 <= k <= SAMPLE_PICK_MAX_TOP_K):
        raise ValueError("sample_pick: tok, pos and counter hold one element each, top_k at most 64")
    with torch.cuda.device(logits.device):
        check(lib().qtip_sample_pick(_ptr(logits), logits.numel(), ctypes.c_float(temperature), k,
                                     ctypes.c_uint(int(seed) & 0xffffffff), _ptr(counter), _ptr(tok), _ptr(pos),
                                     _ptr(history) if history is not None else None,
                                     history.numel() if history is not None else 0, int(history_base),
                                     stream_ptr(logits.device)), "qtip_sample_pick")


# ---- packing tools ---------------------------------------------------------------------------

def repack(packed, m, k, bits, to_kernel=True):
    """Natural packing <-> kernel packing of a 16x16-tile, V=2 trellis (same shape and dtype out).
    to_kernel=True is the re-pack of lib/algo/finetune.py:196-201, False its inverse
    (lib/utils/kernel_decompress.py:19-24)."""
    _check_packed(packed, m, k, bits)
    out = torch.empty_like(packed)
    with torch.cuda.device(packed.device):
        check(lib().qtip_repack(_ptr(out), _ptr(packed), m, k, bits, 1 if to_kernel else 0,
                                stream_ptr(packed.device)), "qtip_repack")
    return out


def _check_natural(packed, T, K, V):
    require_cuda(packed, "packed", (torch.int16, torch.uint16))
    if V not in (1, 2) or K * V > 16 or T % V or (T * K) % 16:
        raise ValueError(f"unsupported natural packing T={T} K={K} V={V}")
    nw = T * K // 16
    if packed.numel() % nw:
        raise ValueError(f"packed holds {packed.numel()} words, not a multiple of {nw} per tile")
    return packed.numel() // nw


def unpack_trellis(packed, T, K, V):
    """Natural packing (ntiles, T*K/16) int16/uint16 -> (ntiles, T/V) int32 states
    (lib/codebook/bitshift.py:329-353)."""
    ntiles = _check_natural(packed, T, K, V)
    states = torch.empty((ntiles, T // V), dtype=torch.int32, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_unpack_trellis(_ptr(states), _ptr(packed), ntiles, T, K, V, stream_ptr(packed.device)),
              "qtip_unpack_trellis")
    return states


def pack_trellis(states, K, V):
    """(ntiles, T/V) states -> natural packing (ntiles, T*K/16) uint16
    (lib/codebook/bitshift.py:294-327).  Raises, like the reference's assert, when consecutive
    states do not overlap by 16 - K*V bits (this check synchronises with the device)."""
    require_cuda(states, "states", torch.int32)
    if states.dim() != 2:
        raise ValueError("states must be (ntiles, T/V)")
    ntiles, ns = states.shape
    T = ns * V
    if V not in (1, 2) or K * V > 16 or (T * K) % 16:
        raise ValueError(f"unsupported natural packing T={T} K={K} V={V}")
    packed = torch.empty((ntiles, T * K // 16), dtype=torch.uint16, device=states.device)
    bad = torch.zeros(1, dtype=torch.int32, device=states.device)
    with torch.cuda.device(states.device):
        check(lib().qtip_pack_trellis(_ptr(packed), _ptr(states), ntiles, T, K, V, _ptr(bad),
                                      stream_ptr(states.device)), "qtip_pack_trellis")
    nbad = int(bad.item())
    if nbad:
        raise ValueError(f"pack_trellis: {nbad} consecutive state pairs are not a bitshift trellis walk")
    return packed


def decode_natural(packed, lut, m, n, td_x, td_y, K, V):
    """Natural packing -> dense (m, n) in the dtype of `lut`, the expanded (V, 65536) table of the
    codebook (fp16 or fp32): get_hatW(unpack_trellis(.)) of lib/codebook/bitshift.py:329-381."""
    T = td_x * td_y
    ntiles = _check_natural(packed, T, K, V)
    if m % td_x or n % td_y or ntiles != (m // td_x) * (n // td_y) or td_y % V:
        raise ValueError(f"packed does not describe a {m}x{n} matrix of {td_x}x{td_y} tiles")
    require_cuda(lut, "lut", (torch.float16, torch.float32))
    if lut.shape != (V, 65536) or lut.device != packed.device:
        raise ValueError(f"lut must be ({V}, 65536) on {packed.device}")
    out = torch.empty((m, n), dtype=lut.dtype, device=packed.device)
    with torch.cuda.device(packed.device):
        check(lib().qtip_decode_natural(_ptr(out), _ptr(packed), _ptr(lut), _DT[lut.dtype], m, n, td_x, td_y, K, V,
                                        stream_ptr(packed.device)), "qtip_decode_natural")
    return out


def rht_chain(parts, post, scale_out, residual, norm_weight, eps, pre, scale_in):
    """(x_new, xt) for one hidden-size vector per row, one launch:
    x_new = fp16(residual + fp16(post * scale_out * H(sum(parts)))),
    xt = fp16(scale_in * H(pre * rmsnorm(x_new))).  parts: (S, rows, n) fp32, n in {2048, 4096, 8192}."""
    require_cuda(parts, "parts", torch.float32)
    require_cuda(residual, "residual", torch.float16)
    require_cuda(norm_weight, "norm_weight", torch.float16)
    if parts.dim() != 3:
        raise ValueError("parts must be (S, rows, n)")
    S, rows, n = parts.shape
    if n not in (2048, 4096, 8192) or residual.numel() != rows * n or norm_weight.numel() != n:
        raise ValueError("rht_chain: unsupported or inconsistent shapes")
    if post is not None:
        require_cuda(post, "post", torch.float32)
    if pre is not None:
        require_cuda(pre, "pre", torch.float16)
    x_new = torch.empty((rows, n), dtype=torch.float16, device=parts.device)
    xt = torch.empty((rows, n), dtype=torch.float16, device=parts.device)
    with torch.cuda.device(parts.device):
        check(lib().qtip_rht_chain(_ptr(xt), _ptr(x_new), _ptr(parts), S, rows, n, _ptr(post), ctypes.c_float(scale_out),
                                   _ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), _ptr(pre),
                                   ctypes.c_float(scale_in), stream_ptr(parts.device)), "qtip_rht_chain")
    return x_new, xt
