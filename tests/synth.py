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
