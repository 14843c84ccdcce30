"""Kernel-packed trellis -> dense weight matrix, on the GPU.

Counterpart of lib/utils/kernel_decompress.py:4-55.  The reference builds the
matrix out of a chain of torch tensor ops on an expanded 65536-entry table;
here one HIP kernel walks the bitstream and looks weights up in LDS.
"""
import torch

from .. import ops

_REP_STATES = None  # for every 9-bit LUT index: a state that hashes to it, and that state's sign


def _representatives():
    global _REP_STATES
    if _REP_STATES is None:
        s = torch.arange(1 << 16, dtype=torch.int64)
        p = s * (s + 1)
        q = (p >> 6) & 511
        sg = (p >> 15) & 1
        rep = torch.zeros(512, dtype=torch.int64)
        neg = torch.zeros(512, dtype=torch.bool)
        seen = torch.zeros(512, dtype=torch.bool)
        # prefer a representative whose sign bit is clear
        for want in (1, 0):
            idx = torch.nonzero(sg == want).flatten()
            rep[q[idx]] = idx
            neg[q[idx]] = bool(want)
            seen[q[idx]] = True
        _REP_STATES = (rep, neg, seen)
    return _REP_STATES


def tlut_from_expanded(expanded_lut):
    """Recover the 512 x 2 tunable table from the (65536, 2) expanded one
    (inverse of quantlut_sym, lib/codebook/bitshift.py:72-80).  Indices no
    state hashes to cannot occur in a stream and are left at zero."""
    rep, neg, seen = _representatives()
    dev = expanded_lut.device
    t = expanded_lut[rep.to(dev)].clone()
    t[:, 0] = torch.where(neg.to(dev), -t[:, 0], t[:, 0])
    t[~seen.to(dev)] = 0
    return t.to(torch.float16).contiguous()


def decode_compressed(L, S, R, V, m, k, compressed, expanded_lut):
    """Same signature as the reference (V is log2 of the vector size, i.e. 1).

    compressed: flat int16/uint16 kernel-packed stream of R*m*k/16 words;
    expanded_lut: (65536, 2) fp16.  Returns the (m, k) fp16 matrix.
    """
    if (L, S, V) != (16, 9, 1) or R not in (2, 3, 4):
        raise NotImplementedError(f"no kernel for L={L} S={S} R={R} V=2**{V}")
    if expanded_lut.shape != (1 << L, 2):
        raise ValueError(f"expanded_lut must be ({1 << L}, 2), got {tuple(expanded_lut.shape)}")
    return ops.decode(compressed.reshape(-1), tlut_from_expanded(expanded_lut), m, k, R)
