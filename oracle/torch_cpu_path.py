"""CPU baseline: the reference's CPU-capable path for one layer, restated in torch.

TEST / MEASUREMENT INFRASTRUCTURE ONLY (used by bench.py's cpu_baseline leg
and tests); never imported by qtip_amd.

What the reference runs when no kernel is available is a chain of torch tensor
ops that turns the kernel-packed stream into a dense fp16 matrix
(lib/utils/kernel_decompress.py:4-55) followed by a dense matmul
(lib/codebook/bitshift.py:489).  This restatement does the same three stages
(un-interleave the 2x2 tile blocks, build 16-bit windows, gather from the
expanded 65536-entry table, undo the fragment order) with torch CPU ops and
multiplies in fp32 (torch's CPU fp16 matmul is avoided; the products are
exact either way).  It gathers only the 128 windows per tile that are used,
where the reference materialises all 16 shifts of every word, so it is a
somewhat faster CPU path than the reference's own.
"""
import time

import torch


def expand_lut(tlut):
    s = torch.arange(1 << 16, dtype=torch.int64)
    p = s * (s + 1)
    lut = tlut.reshape(512, 2)[(p >> 6) & 511].clone()
    neg = ((p >> 15) & 1).bool()
    lut[neg, 0] = -lut[neg, 0]
    return lut


def decode_dense(packed, lut, m, k, K):
    by = packed.reshape(-1).view(torch.uint8).reshape(m // 32, k // 32, 32, 2, 2, K)
    by = by.flip(-1).permute(0, 4, 1, 3, 2, 5).reshape(m // 16 * (k // 16), 16 * K, 2)
    words = (by[..., 0].to(torch.int32) << 8) | by[..., 1].to(torch.int32)
    win = (words << 16) | torch.roll(words, -1, dims=1)
    pos = torch.arange(128) * 2 * K
    states = (win[:, pos // 16] >> (16 - pos % 16)) & 0xFFFF
    frag = lut[states.long()]
    t = frag.reshape(m // 16, k // 16, 8, 4, 2, 2, 2).permute(0, 5, 2, 1, 4, 3, 6)
    return t.reshape(m, k)


def time_layer(packed, x, tlut, m, k, K, reps=1, threads=None):
    """Returns dict(decode_s, matmul_s, out) for decode + matvec on the host."""
    if threads:
        torch.set_num_threads(threads)
    lut = expand_lut(tlut)
    best_d = best_m = float("inf")
    out = None
    for _ in range(reps):
        t0 = time.perf_counter()
        w = decode_dense(packed, lut, m, k, K)
        t1 = time.perf_counter()
        out = w.float() @ x.reshape(k, 1).float()
        t2 = time.perf_counter()
        best_d, best_m = min(best_d, t1 - t0), min(best_m, t2 - t1)
    return dict(decode_s=best_d, matmul_s=best_m, out=out.reshape(-1), weights=w)
