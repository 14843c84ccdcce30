"""CPU oracle for the QTIP quantized-linear inference path (TEST INFRASTRUCTURE ONLY).

This file is a checker.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.  The shipped package (qtip_amd/)
never imports anything from oracle/ and has no CPU fallback.

Everything here is numpy and restates the algorithms of Cornell-RelaxML/qtip
for the HYB code (L=16, tlut_bits=9, V=2, 16x16 tiles, K in {2,3,4}).  Each
function cites the reference file:line it follows (paths relative to the
reference checkout).

Pinning status of each function (what, other than itself, fixes its result):

  quantlut_sym            closed form + hand-computed known answers + brute
                          force over all 65536 states against the device
                          statement of the hash (qtip-kernels/src/inference.cu:349-359).
  unpack_trellis_natural  pack/unpack round trip, overlap invariant
  pack_trellis_natural    (lib/codebook/bitshift.py:307-309), bit-flip locality.
  decode_natural          cross-checked against decode_kernel_lanes through
  repack_for_kernel       the repack + _PERMUTE (three descriptions of the same
  decode_kernel_tensor    layout in the reference must agree), plus the
  decode_kernel_lanes     reference's zero-stream known-answer test
                          (qtip-kernels/src/test.cu:23-58).
  hadamard_transform      scipy.linalg.hadamard (Sylvester) for the power-of-two
                          part, np.kron with the order-K table for the general
                          case, orthogonality / involution invariants.
                          The reference calls the third-party CUDA package
                          fast_hadamard_transform==1.0.4.post1 here, which is
                          not vendored: last-ulp summation order is
                          "parity unpinned" and checked by tolerance only.
  bitshift_linear_forward dense W_eff formula of lib/codebook/bitshift.py:389-413
                          (the reference's own "manifest" form).
  unpack_trellis_generic  any (T, K, V): equal to unpack_trellis_natural for the 16x16,
  pack_trellis_generic    V=2 case; round trip; bit-level definition by Python-int
  decode_natural_generic  string slicing in the tests; the 16x16/V=2 case equals decode_natural.
  code_1mad / code_2mad   byte-sum codes: scalar Python-int recomputation, exact moments
                          (mean 0, variance 1 over all 2^32 inputs follows from the byte-sum
                          construction; sqrt(21845) = 147.8005...), value grid k/147.8.
  code_3inst              scalar Python-int + struct('e') recomputation of hand-picked states.
  quantlut                closed form; equals quantlut_sym up to the sign of element 0.
"""
from __future__ import annotations

import math
import os

import numpy as np

L_BITS = 16
TLUT_BITS = 9
TILE = 16
STATES_PER_TILE = 128

# ----------------------------------------------------------------------------
# a1. HYB codebook expansion
# ----------------------------------------------------------------------------


def hyb_hash(states: np.ndarray):
    """(lut index, sign bit) of 16-bit states.

    lib/codebook/bitshift.py:72-77: p = s*(s+1); sign = (p >> 15) & 1;
    index = (p >> (16 - 9 - 1)) & 511.
    """
    s = states.astype(np.uint64)
    p = s * (s + 1)
    return ((p >> np.uint64(6)) & np.uint64(511)).astype(np.int64), \
        ((p >> np.uint64(15)) & np.uint64(1)).astype(np.int64)


def quantlut_sym(tlut: np.ndarray) -> np.ndarray:
    """Expanded (65536, 2) fp16 table from the (512, 2) fp16 tunable table.

    lib/codebook/bitshift.py:72-80: element 0 of the pair is negated where the
    sign bit of the hash is set; element 1 is taken as is.
    """
    tlut = np.asarray(tlut, dtype=np.float16).reshape(512, 2)
    q, sg = hyb_hash(np.arange(1 << L_BITS))
    out = tlut[q].copy()
    # multiply by (1 - 2*sign) in fp16: exact (sign flip), keeps -0.0 semantics
    out[:, 0] = out[:, 0] * (1 - 2 * sg).astype(np.float16)
    return out


# ----------------------------------------------------------------------------
# a2/a4. natural packing (one circular bitstream per 16x16 tile)
# ----------------------------------------------------------------------------


def unpack_trellis_natural(words: np.ndarray, K: int) -> np.ndarray:
    """(ntiles, 16K) uint16 natural stream -> (ntiles, 128) int32 states.

    lib/codebook/bitshift.py:329-353: bits are taken MSB first from each
    word, the first L-KV bits are appended again (tail biting) and state i is
    the 16-bit window at bit offset i*K*V.
    """
    words = np.ascontiguousarray(words).view(np.uint16).reshape(-1, 16 * K)
    nt = words.shape[0]
    bits = ((words[:, :, None] >> (15 - np.arange(16, dtype=np.uint16))) & 1)
    bits = bits.reshape(nt, 256 * K).astype(np.int64)
    kv = 2 * K
    ext = np.concatenate([bits, bits[:, :L_BITS - kv]], axis=1)
    weights = 1 << np.arange(15, -1, -1, dtype=np.int64)
    states = np.empty((nt, STATES_PER_TILE), dtype=np.int32)
    for i in range(STATES_PER_TILE):
        states[:, i] = (ext[:, i * kv:i * kv + 16] * weights).sum(axis=1)
    return states


def pack_trellis_natural(states: np.ndarray, K: int) -> np.ndarray:
    """(ntiles, 128) states -> (ntiles, 16K) uint16 natural stream.

    lib/codebook/bitshift.py:294-327.  Raises if consecutive states do not
    overlap by L-KV bits (the reference asserts the same, :307-309).
    """
    states = np.asarray(states, dtype=np.int64)
    nt, T = states.shape
    kv = 2 * K
    low = (1 << (L_BITS - kv)) - 1
    if not np.all((states[:, :-1] & low) == (states[:, 1:] >> kv)):
        raise ValueError("states are not a bitshift trellis walk")
    bits = np.zeros((nt, T * kv + L_BITS - kv), dtype=np.uint8)
    bits[:, :16] = (states[:, :1] >> np.arange(15, -1, -1)) & 1
    for i in range(1, T):
        fresh = states[:, i] & ((1 << kv) - 1)
        bits[:, 16 + (i - 1) * kv:16 + i * kv] = \
            (fresh[:, None] >> np.arange(kv - 1, -1, -1)) & 1
    bits = bits[:, :T * kv]  # the dropped tail repeats the head (:317)
    w = bits.reshape(nt, -1, 16).astype(np.uint32)
    words = (w << np.arange(15, -1, -1, dtype=np.uint32)).sum(axis=2)
    return words.astype(np.uint16)


# within-tile order used when quantising for the kernel:
# lib/algo/ldlq.py:10-13 (sequence position p holds row-major tile element PERMUTE[p])
PERMUTE = np.arange(256).reshape(2, 8, 2, 4, 2).transpose(1, 3, 2, 0, 4).reshape(-1)
INV_PERMUTE = np.empty(256, dtype=np.int64)
INV_PERMUTE[PERMUTE] = np.arange(256)


def decode_natural(words: np.ndarray, lut: np.ndarray, m: int, n: int, K: int,
                   kernel_order: bool) -> np.ndarray:
    """Natural stream -> (m, n) fp16 matrix.

    lib/codebook/bitshift.py:199-201 (recons) and :378-381 (get_hatW): state s
    gives sequence positions 2s, 2s+1; tiles are numbered row-major over
    (m/16, n/16).  With kernel_order the sequence was permuted by PERMUTE
    before quantisation (lib/algo/ldlq.py:56-61), so tile.flat[PERMUTE[p]] = seq[p].
    """
    states = unpack_trellis_natural(words, K)
    seq = lut[states].reshape(-1, 256)  # (ntiles, 256) in sequence order
    if kernel_order:
        tiles = np.empty_like(seq)
        tiles[:, PERMUTE] = seq
    else:
        tiles = seq
    return np.ascontiguousarray(
        tiles.reshape(m // 16, n // 16, 16, 16).transpose(0, 2, 1, 3).reshape(m, n))


def repack_for_kernel(words: np.ndarray, m: int, n: int, K: int) -> np.ndarray:
    """Natural (ntiles, 16K) uint16 -> kernel-packed int16 of the same shape.

    lib/algo/finetune.py:196-201: byte-swap every word (stream order bytes),
    split the tile's 32K bytes into 32 chunks of K bytes, interleave the four
    tiles of a 2x2 tile block as [lane][kh][mh], reverse each K-byte chunk.
    """
    by = np.ascontiguousarray(words).view(np.uint16).reshape(-1, 16 * K)
    by = by.view(np.uint8).reshape(-1, 2)[:, ::-1]  # big-endian byte stream
    by = by.reshape(m // 32, 2, n // 32, 2, 32, K)  # [i0, mh, i1, kh, lane, K]
    by = by.transpose(0, 2, 4, 3, 1, 5)[..., ::-1]  # [i0, i1, lane, kh, mh, K]
    return np.ascontiguousarray(by).reshape(-1).view(np.int16).reshape(-1, 16 * K)


def kernel_to_natural(packed: np.ndarray, m: int, n: int, K: int) -> np.ndarray:
    """Inverse of repack_for_kernel (lib/utils/kernel_decompress.py:19-24)."""
    by = np.ascontiguousarray(packed).reshape(-1).view(np.uint8)
    by = by.reshape(m // 32, n // 32, 32, 2, 2, K)[..., ::-1]
    by = by.transpose(0, 4, 1, 3, 2, 5)  # [i0, mh, i1, kh, lane, K]
    by = np.ascontiguousarray(by).reshape(-1, 2)[:, ::-1]
    return np.ascontiguousarray(by).reshape(-1).view(np.uint16).reshape(-1, 16 * K)


# ----------------------------------------------------------------------------
# a3. kernel-packed stream -> dense matrix, two independent statements
# ----------------------------------------------------------------------------


def decode_kernel_tensor(packed: np.ndarray, lut: np.ndarray, m: int, k: int,
                         K: int) -> np.ndarray:
    """Follows lib/utils/kernel_decompress.py:4-55 step by step.

    un-interleave to per-tile uint16 words (:19-24), pair every word with its
    circular successor (:29-35), take the 16-bit window at every 2K-th bit
    offset (:38-46), look the states up (:49) and undo the fragment order (:52-54).
    """
    words = kernel_to_natural(packed, m, k, K).astype(np.uint32)  # (ntiles, 16K)
    nxt = np.roll(words, -1, axis=1)
    win = (words << 16) | nxt  # 32-bit window starting at each word
    # bit offsets inside a word: all multiples of 2K land at (16w + o); collect
    # the 128 states in stream order
    nt = words.shape[0]
    pos = np.arange(STATES_PER_TILE) * 2 * K
    w_idx, o = pos // 16, pos % 16
    states = (win[:, w_idx] >> (16 - o).astype(np.uint32)) & 0xFFFF
    frag = lut[states]  # (ntiles, 128, 2)
    t = frag.reshape(m // 16, k // 16, 8, 4, 2, 2, 2)
    # axes: [tm, tn, r8, c4, chalf, rhalf, e] -> rows (tm, rhalf, r8), cols (tn, chalf, c4, e)
    t = t.transpose(0, 5, 2, 1, 4, 3, 6)
    return np.ascontiguousarray(t).reshape(m, k)


def decode_kernel_states_lanes(packed: np.ndarray, m: int, k: int, K: int) -> np.ndarray:
    """Lane-level statement of the device decode: states[i0,i1,lane,kh,mh,j].

    qtip-kernels/src/inference.cu:94-166 (load + neighbour fix-up) and
    :340-346 (window shifts): a lane's chunk is K bytes read little-endian,
    the window is chunk || top16(next lane's chunk) and state j starts 2K*j
    bits below the top.
    """
    by = np.ascontiguousarray(packed).reshape(-1).view(np.uint8)
    by = by.reshape(m // 32, k // 32, 32, 2, 2, K).astype(np.uint64)
    own = np.zeros(by.shape[:-1], dtype=np.uint64)
    for b in range(K):
        own |= by[..., b] << np.uint64(8 * b)
    nxt = np.roll(own, -1, axis=2) >> np.uint64(8 * K - 16)
    win = (own << np.uint64(16)) | nxt
    st = [(win >> np.uint64(8 * K - 2 * K * j)) & np.uint64(0xFFFF) for j in range(4)]
    return np.stack(st, axis=-1).astype(np.int64)


def decode_kernel_lanes(packed: np.ndarray, lut: np.ndarray, m: int, k: int,
                        K: int) -> np.ndarray:
    """Kernel-packed stream -> (m, k) fp16 using the lane-level statement.

    Placement of a lane's four states follows the A-fragment of
    mma.m16n8k16 that the reference feeds them to (inference.cu:364-373):
    j=0 -> (r, c..c+1), j=1 -> (r+8, .), j=2 -> (r, c+8..), j=3 -> (r+8, c+8..)
    with r = lane/4 and c = 2*(lane%4).
    """
    st = decode_kernel_states_lanes(packed, m, k, K)  # [i0,i1,lane,kh,mh,j]
    vals = lut[st]  # [..., j, e]
    i0, i1, lane, kh, mh, j, e = np.meshgrid(
        np.arange(m // 32), np.arange(k // 32), np.arange(32), np.arange(2),
        np.arange(2), np.arange(4), np.arange(2), indexing="ij", sparse=True)
    row = 32 * i0 + 16 * mh + lane // 4 + 8 * (j % 2)
    col = 32 * i1 + 16 * kh + 2 * (lane % 4) + 8 * (j // 2) + e
    out = np.empty((m, k), dtype=np.float16)
    out[np.broadcast_to(row, vals.shape), np.broadcast_to(col, vals.shape)] = vals
    return out


def decode_kernel(packed, tlut, m, k, K):
    """Convenience: kernel-packed stream + raw (512,2) table -> (m,k) fp16."""
    return decode_kernel_lanes(packed, quantlut_sym(tlut), m, k, K)


# ----------------------------------------------------------------------------
# a5. decompress-matvec
# ----------------------------------------------------------------------------


def decompress_matvec(packed, x, tlut, m, k, K) -> np.ndarray:
    """out[m] = hatW[m,k] . x[k], fp16 operands, products exact, fp64 sums.

    qtip-kernels/src/inference.cu:364-373 accumulates fp16 x fp16 products in
    fp32; the oracle sums in fp64 so that the tolerance in the tests measures
    the device's fp32 accumulation error and nothing else.
    """
    w = decode_kernel(packed, tlut, m, k, K).astype(np.float64)
    xv = np.asarray(x, dtype=np.float16).reshape(k).astype(np.float64)
    return w @ xv


# ----------------------------------------------------------------------------
# a7. randomized Hadamard transform
# ----------------------------------------------------------------------------

_HAD_ORDERS = (172, 156, 140, 124, 116, 108, 60, 52, 36, 28, 20, 12)
_TABLES = None


def _load_tables():
    global _TABLES
    if _TABLES is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), os.pardir,
                            "qtip_amd", "utils", "hadamard_tables.npz")
        z = np.load(path, allow_pickle=False)
        _TABLES = {}
        for o in _HAD_ORDERS:
            bits = np.unpackbits(z[f"had{o}"])[:o * o].reshape(o, o)
            _TABLES[o] = (1.0 - 2.0 * bits).astype(np.float64)  # bit set = -1
    return _TABLES


def get_hadK(n: int):
    """(table or None, K).  lib/utils/matmul_had.py:9-63: first order in
    172,156,...,12 that divides n; the cofactor must be a power of two."""
    for o in _HAD_ORDERS:
        if n % o == 0:
            p = n // o
            if p & (p - 1):
                raise AssertionError(f"{n} = {o} * {p}: cofactor not a power of two")
            return _load_tables()[o], o
    if n <= 0 or n & (n - 1):
        raise AssertionError(f"{n} is not a supported Hadamard size")
    return None, 1


def fwht(a: np.ndarray) -> np.ndarray:
    """Unnormalised Sylvester (natural-order) Walsh-Hadamard along the last axis.

    Same butterfly recursion as lib/utils/matmul_had.py:70-80 (pairs at the
    coarsest split first); any stage order gives the same matrix.
    """
    a = np.array(a, dtype=np.float64)
    n = a.shape[-1]
    h = 1
    while h < n:
        v = a.reshape(*a.shape[:-1], n // (2 * h), 2, h)
        a = np.concatenate([v[..., 0, :] + v[..., 1, :], v[..., 0, :] - v[..., 1, :]],
                           axis=-1).reshape(*a.shape[:-1], n)
        h *= 2
    return a


def hadamard_transform(x: np.ndarray, transpose: bool = False) -> np.ndarray:
    """y = (H_K (x) H_{n/K}) x / sqrt(n) along the last axis, in fp64.

    lib/utils/matmul_had.py:105-115: view (.., K, n/K), Sylvester transform on
    the last axis, then the order-K table (its transpose for the "Ut" form)
    applied on the K axis.
    """
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[-1]
    had, K = get_hadK(n)
    y = fwht(x.reshape(*x.shape[:-1], K, n // K))
    if K > 1:
        hk = had.T if transpose else had
        y = np.einsum("ij,...jc->...ic", hk, y)
    return y.reshape(x.shape) / math.sqrt(n)


# ----------------------------------------------------------------------------
# a8/a9. whole layer
# ----------------------------------------------------------------------------


def bitshift_linear_forward(inp, packed, SU, SV, tlut, K, return_parts=False, matvec_fn=None):
    """Restates BitshiftLinear.forward, eval mode, rcp=0
    (lib/codebook/bitshift.py:415-472) with its cast points:

      x1 = fp32(inp) * SU ; x2 = H_L^T x1 / sqrt(n) ; x3 = x2 / 32 ;
      x4 = fp16(x3) ; y0 = hatW x4 ; y1 = H_R y0 / sqrt(m) ;
      out = fp16(y1 * (SV * 32)).

    Transforms and sums are evaluated in fp64 on the bit-exact fp16 weights,
    so the result is the value the device's fp32 pipeline approximates.  For
    more than one row the reference rounds y0 to fp16 once (:489); that
    rounding is applied here as well.

    matvec_fn(x4_row) -> (m,) float64, if given, supplies hatW x4 row by row
    (the C restatement for the full-size matrices, where a dense float64 copy
    of hatW would not fit in memory).
    """
    SU = np.asarray(SU)
    SV = np.asarray(SV)
    n, m = SU.shape[0], SV.shape[0]
    x0 = np.asarray(inp, dtype=np.float16).reshape(-1, n)
    x1 = x0.astype(np.float32) * SU.astype(np.float32)
    x2 = hadamard_transform(x1, transpose=True)
    x4 = (x2 / 32.0).astype(np.float32).astype(np.float16)
    if matvec_fn is not None:
        y0 = np.stack([np.asarray(matvec_fn(row), dtype=np.float64) for row in x4])
    else:
        w = decode_kernel(packed, tlut, m, n, K).astype(np.float64)
        y0 = x4.astype(np.float64) @ w.T
    if x0.shape[0] > 1:
        y0 = y0.astype(np.float16).astype(np.float64)
    y1 = hadamard_transform(y0, transpose=False)
    y2 = y1 * (SV.astype(np.float64) * 32.0)
    out = y2.astype(np.float16).reshape(*np.shape(inp)[:-1], m)
    if return_parts:
        return out, dict(x4=x4, y0=y0, y1=y1, y2=y2)
    return out


def dense_equivalent(packed, SU, SV, tlut, K, decode_fn=None):
    """W_eff with out = inp @ W_eff^T (no activation rounding), following the
    reference's own dense form (lib/codebook/bitshift.py:389-413 and
    quantize_llama/manifest_model.py:38-50):
    W_eff = diag(SV*32) . H_R . (hatW/32) . H_L^T . diag(SU).
    decode_fn(packed, tlut, m, n, K): a faster restatement of decode_kernel (the C one)."""
    SU = np.asarray(SU, dtype=np.float64)
    SV = np.asarray(SV, dtype=np.float64)
    n, m = SU.shape[0], SV.shape[0]
    w = (decode_fn or decode_kernel)(packed, tlut, m, n, K).astype(np.float64) / 32.0
    # rows of w are vectors over n: apply H_L (not transposed) to each row,
    # since (w H_L^T)[i,:] = H_L-transform of row i with the transposed table
    # swapped: (w @ HL^T) = (HL @ w^T)^T
    a = hadamard_transform(w, transpose=False)  # (HL @ w^T)^T, shape (m, n)
    b = hadamard_transform(a.T, transpose=False).T  # HR applied over the m axis
    return (SV[:, None] * 32.0) * b * SU[None, :]


# ----------------------------------------------------------------------------
# f3. generic natural packing (any tile size T, K bits, V weights per state) and
#     the other decode modes of the codebook
# ----------------------------------------------------------------------------


def unpack_trellis_generic(words: np.ndarray, T: int, K: int, V: int) -> np.ndarray:
    """(ntiles, T*K/16) uint16 -> (ntiles, T/V) int32 states, lib/codebook/bitshift.py:329-353
    for any tile size: circular stream of T*K bits, state i = 16-bit window at bit i*K*V."""
    nw = T * K // 16
    words = np.ascontiguousarray(words).view(np.uint16).reshape(-1, nw)
    nt = words.shape[0]
    bits = ((words[:, :, None] >> (15 - np.arange(16, dtype=np.uint16))) & 1).reshape(nt, T * K).astype(np.int64)
    kv = K * V
    ext = np.concatenate([bits, bits[:, :L_BITS - kv]], axis=1) if kv < L_BITS else bits
    weights = 1 << np.arange(15, -1, -1, dtype=np.int64)
    ns = T // V
    states = np.empty((nt, ns), dtype=np.int32)
    for i in range(ns):
        states[:, i] = (ext[:, i * kv:i * kv + 16] * weights).sum(axis=1)
    return states


def pack_trellis_generic(states: np.ndarray, K: int, V: int) -> np.ndarray:
    """(ntiles, T/V) states -> (ntiles, T*K/16) uint16, lib/codebook/bitshift.py:294-327: all 16
    bits of state 0, then the K*V fresh bits of every later state, cut to T*K bits."""
    states = np.asarray(states, dtype=np.int64)
    nt, ns = states.shape
    kv = K * V
    low = (1 << (L_BITS - kv)) - 1
    if not np.all((states[:, :-1] & low) == (states[:, 1:] >> kv)):
        raise ValueError("states are not a bitshift trellis walk")
    bits = np.zeros((nt, ns * kv + L_BITS - kv), dtype=np.uint8)
    bits[:, :16] = (states[:, :1] >> np.arange(15, -1, -1)) & 1
    for i in range(1, ns):
        fresh = states[:, i] & ((1 << kv) - 1)
        bits[:, 16 + (i - 1) * kv:16 + i * kv] = (fresh[:, None] >> np.arange(kv - 1, -1, -1)) & 1
    bits = bits[:, :ns * kv]
    w = bits.reshape(nt, -1, 16).astype(np.uint32)
    return (w << np.arange(15, -1, -1, dtype=np.uint32)).sum(axis=2).astype(np.uint16)


def decode_natural_generic(words, lut, m, n, td_x, td_y, K, V):
    """Natural stream -> (m, n) in lut's dtype; lut is (V, 65536).  lib/codebook/bitshift.py:199-201
    (recons) and :378-381 (get_hatW): sequence position i*V + v of a tile is its row-major element."""
    st = unpack_trellis_generic(words, td_x * td_y, K, V)  # (ntiles, T/V)
    seq = np.stack([lut[v][st] for v in range(V)], axis=-1).reshape(-1, td_x * td_y)
    return np.ascontiguousarray(
        seq.reshape(m // td_x, n // td_y, td_x, td_y).transpose(0, 2, 1, 3).reshape(m, n))


def _byte_sum(x):
    return ((x & 255) + ((x >> 8) & 255) + ((x >> 16) & 255) + ((x >> 24) & 255)).astype(np.int64)


def code_1mad(states: np.ndarray) -> np.ndarray:
    """lib/codebook/bitshift.py:17-26, uint64 arithmetic reduced mod 2^32."""
    x = (np.asarray(states, dtype=np.uint64) * np.uint64(34038481) + np.uint64(76625530)) & np.uint64(0xFFFFFFFF)
    return ((_byte_sum(x) - 510).astype(np.float32) / np.float32(147.800537109375)).astype(np.float32)


def code_2mad(states: np.ndarray) -> np.ndarray:
    """lib/codebook/bitshift.py:29-40."""
    M = np.uint64(0xFFFFFFFF)
    x = (np.asarray(states, dtype=np.uint64) * np.uint64(264435761) + np.uint64(1013904223)) & M
    x = (((x * np.uint64(1664525)) >> np.uint64(32)) + x) & M
    return ((_byte_sum(x) - 510).astype(np.float32) / np.float32(147.800537109375)).astype(np.float32)


def code_3inst(states: np.ndarray) -> np.ndarray:
    """lib/codebook/bitshift.py:43-59: the two 16-bit halves of ((x*a+b) & 0x8FFF8FFF) ^ 0x3B603B60
    read as fp16 and added in fp16."""
    M = np.uint64(0xFFFFFFFF)
    x = (np.asarray(states, dtype=np.uint64) * np.uint64(89226354) + np.uint64(64248484)) & M
    res = (x & np.uint64(0x8FFF8FFF)) ^ np.uint64(996162400)
    top = (res >> np.uint64(16)).astype(np.uint16).view(np.float16)
    bot = (res & np.uint64(0xFFFF)).astype(np.uint16).view(np.float16)
    return (top + bot).astype(np.float32)


def quantlut(tlut: np.ndarray) -> np.ndarray:
    """lib/codebook/bitshift.py:62-69: tlut[(s*(s+1) >> (16-nbits)) & (2^nbits - 1)] for all states."""
    nbits = int(np.log2(tlut.shape[0]))
    s = np.arange(1 << L_BITS, dtype=np.int64)
    idx = ((s * (s + 1)) >> (16 - nbits)) & ((1 << nbits) - 1)
    return tlut[idx]
