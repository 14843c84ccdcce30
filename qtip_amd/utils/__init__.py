from .kernel_check import has_kernel
from .kernel_decompress import decode_compressed
from .matmul_had import get_hadK, is_pow2, matmul_hadU_cuda, matmul_hadUt_cuda


def dtype_from_str(s):
    import torch
    return {'torch.float32': torch.float32, 'torch.float16': torch.float16, 'torch.bfloat16': torch.bfloat16}[str(s)]
