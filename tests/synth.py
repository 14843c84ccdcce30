"""Seeded synthetic layer tensors shared by the tests (numpy, CPU)."""
import numpy as np


def make_layer(m, k, K, seed=0, scale=None):
    """Uniform-random kernel-packed bitstream (any circular bitstream is a valid
    tail-biting trellis walk), N(0,1) fp16 table, +-1 sign vectors, x ~ N(0,1)."""
    rng = np.random.default_rng(seed)
    packed = rng.integers(-32768, 32768, size=(m // 16 * k // 16, 16 * K), dtype=np.int16)
    tlut = rng.standard_normal((512, 2)).astype(np.float16)
    SU = np.sign(rng.standard_normal(k) + 1e-5).astype(np.float16)
    sc = scale if scale is not None else 1.0 / np.sqrt(k)
    SV = (np.sign(rng.standard_normal(m) + 1e-5) * sc).astype(np.float32)
    x = rng.standard_normal((1, k)).astype(np.float16)
    return dict(packed=packed, tlut=tlut, SU=SU, SV=SV, x=x, m=m, k=k, K=K)


def rounding_case():
    """A 64 x 64, 2-bit layer built by hand so that the fp16 rounding of the matmul result - which the
    reference applies for more than one row (fp16 GEMM output, lib/codebook/bitshift.py:489) and not
    for a single row (fp32 matvec op, :443-448) - changes the layer's output from 6.0 to 8.0.

    Stream: every chunk of the tile-row half mh = 0 is 0x0000, every chunk of mh = 1 is 0x1111, so
    rows r with r % 32 < 16 decode state 0x0000 everywhere (hash 0 -> entry 0, no sign) and the other
    rows state 0x1111 (0x1111 * 0x1112 = 0x1235432 -> low 16 bits 0x5432 -> entry 336, sign bit 0).
    Table: entry 0 = (64, 3/64), entry 336 = (-64, 0), everything else 0.
    Input 256 * e_0 with SU = 1: H x / 8 / 32 = 1.0 in every position, so
      y0[r] = 32 * (64 + 3/64) = 2049.5   (fp16: 2050)   for r % 32 < 16
      y0[r] = 32 * (-64)       = -2048                  otherwise,
    all sums exact in fp32.  Output element 0 = sum(y0) / 8 * (SV * 32) with SV = 1/32:
      (32 * 2049.5 - 32 * 2048) / 8 = 6.0 without the rounding, (32 * 2050 - 32 * 2048) / 8 = 8.0 with it.
    """
    m = k = 64
    K = 2
    blk = np.zeros((m // 32, k // 32, 32, 2, 2, K), dtype=np.uint8)  # [i0][i1][lane][kh][mh][byte]
    blk[:, :, :, :, 1, :] = 0x11
    packed = blk.reshape(-1).view(np.int16).reshape(m // 16 * k // 16, 16 * K)
    tlut = np.zeros((512, 2), dtype=np.float16)
    tlut[0] = (64.0, 3.0 / 64.0)
    tlut[336] = (-64.0, 0.0)
    SU = np.ones(k, dtype=np.float16)
    SV = np.full(m, 1.0 / 32.0, dtype=np.float32)
    x = np.zeros((1, k), dtype=np.float16)
    x[0, 0] = 256.0
    return dict(packed=packed, tlut=tlut, SU=SU, SV=SV, x=x, m=m, k=k, K=K)
