"""torch custom ops of the bs=1 decompress-matvec, under the reference's names.

The reference defines one op per compiled shape,
`quip_lib::decompress_matvec_qtip_{m}_{n}_{k}_{bits}(Tensor compressed, Tensor x,
Tensor codebook) -> Tensor` (lib/codebook/__init__.py:4-93), each bound to a
separately instantiated CUDA kernel.  The HIP kernel takes its shape at run
time, so all names share one implementation; any further shape can be added
with `register_shape`.
"""
import torch

from .. import ops

# (m, k) -> bit widths registered by the reference (lib/codebook/__init__.py:4-66)
_SHAPES = {
    (1024, 3072): (4,), (8192, 3072): (4,), (3072, 8192): (4,), (3072, 3072): (4,),
    (53248, 16384): (2, 3, 4), (16384, 53248): (2, 3, 4), (1024, 16384): (2, 3, 4),
    (16384, 16384): (2, 3, 4), (4096, 14336): (2, 3, 4), (14336, 4096): (2, 3, 4),
    (1024, 4096): (2, 3, 4), (4096, 4096): (2, 3, 4), (4096, 11008): (2, 3, 4),
    (11008, 4096): (2, 3, 4), (12288, 4096): (2, 3, 4), (22016, 4096): (2, 3, 4),
    (8192, 8192): (2, 3, 4), (10240, 8192): (2, 3, 4), (57344, 8192): (2, 3, 4),
    (8192, 1024): (2, 3, 4), (8192, 28672): (2, 3, 4), (28672, 8192): (2, 3, 4),
    (1024, 8192): (2, 3, 4),
    (256, 256): (2, 3, 4),  # native-only test shape (qtip-kernels/src/qtip_torch.cu:157-164)
}

kernels = [(m, 1, k, b) for (m, k), bits in _SHAPES.items() for b in bits]
kdict = {}


def _make(m, k, bits):
    name = f"decompress_matvec_qtip_{m}_1_{k}_{bits}"
    qual = f"quip_lib::{name}"
    torch.library.define(qual, "(Tensor compressed, Tensor x, Tensor codebook) -> Tensor")

    @torch.library.register_fake(qual)
    def _abstract(compressed, x, codebook):
        return torch.zeros(1, m, dtype=torch.float32, device=x.device)

    @torch.library.impl(qual, "cuda")
    def _impl(compressed, x, codebook):
        # reference glue (lib/codebook/__init__.py:85-92): x.to(fp16), flat
        # codebook, (1, m) fp32 result; no zero-fill is needed here because
        # the kernel overwrites every element
        xh = x.to(torch.float16).contiguous()
        out = ops.decompress_matvec(compressed.reshape(-1), xh.reshape(-1), codebook.reshape(-1).contiguous(),
                                    m, k, bits)
        return out.view(1, m)

    kdict[(m, 1, k, bits)] = getattr(torch.ops.quip_lib, name)


def register_shape(m, k, bits):
    """Make `torch.ops.quip_lib.decompress_matvec_qtip_{m}_1_{k}_{bits}` available."""
    if m % 32 or k % 32 or bits not in (2, 3, 4):
        raise ValueError("need m % 32 == 0, k % 32 == 0 and bits in {2,3,4}")
    if (m, 1, k, bits) not in kdict:
        _make(m, k, bits)
    return kdict[(m, 1, k, bits)]


for _m, _n, _k, _b in kernels:
    _make(_m, _k, _b)
