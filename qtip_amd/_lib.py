"""ctypes binding of libqtip_hip.so (the C ABI declared in include/qtip_hip.h).

There is no CPU or pure-PyTorch fallback: if the shared library is missing or
a launcher reports an error, the call raises.
"""
import ctypes
import os

import torch  # must be imported first so that its bundled HIP runtime is the one libqtip_hip.so binds to

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("QTIP_HIP_LIBRARY") or os.path.join(_HERE, "libqtip_hip.so")

QTIP_F16 = 0
QTIP_F32 = 1
ABI_VERSION = 20

_lib = None


class QtipLibraryError(RuntimeError):
    pass


_SIGNATURES = {
    "qtip_abi_version": (ctypes.c_int, []),
    "qtip_init": (ctypes.c_int, []),
    "qtip_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "qtip_decode": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_void_p]),
    "qtip_matvec_split": (ctypes.c_int, [ctypes.c_int] * 3),
    "qtip_matvec_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 3),
    "qtip_decompress_matvec_parts": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "qtip_decompress_matvec_parts_rht": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_float, ctypes.c_void_p] +
                                         [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "qtip_decompress_matvec_parts_chain": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 +
                                           [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_float,
                                            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_float,
                                            ctypes.c_void_p, ctypes.c_void_p]),
    "qtip_decompress_matvec_group_chain": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 4 +
                                           [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t,
                                            ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_float, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p]),
    "qtip_decompress_matvec_group": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 4 +
                                     [ctypes.c_int] * 3 + [ctypes.c_void_p]),
    "qtip_decompress_matvec": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 +
                               [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "qtip_decompress_matvec_noalloc": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "qtip_gemm_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 4),
    "qtip_decompress_gemm": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 +
                             [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "qtip_rht": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]),
    "qtip_rht_post_rows": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_float, ctypes.c_void_p]),
    "qtip_rht_silu_pair": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
                                          ctypes.c_void_p]),
    "qtip_rht_fused_pre_rows": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                               ctypes.c_float, ctypes.c_void_p]),
    "qtip_rht_fused": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_float,
                                      ctypes.c_void_p, ctypes.c_void_p]),
    "qtip_rht_chain": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_float,
                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                      ctypes.c_float, ctypes.c_void_p]),
    "qtip_decode_attention": (ctypes.c_int, [ctypes.c_void_p] * 6 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2),
    "qtip_decode_attention_rht": (ctypes.c_int, [ctypes.c_void_p] * 2 + [ctypes.c_int, ctypes.c_size_t,
                                                 ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_int] +
                                  [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2),
    "qtip_decode_attention_rht3": (ctypes.c_int, [ctypes.c_void_p] * 2 + [ctypes.c_int, ctypes.c_size_t] +
                                   [ctypes.c_void_p] * 8 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2),
    "qtip_rmsnorm": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_float, ctypes.c_int, ctypes.c_void_p]),
    "qtip_greedy_pick": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 3 +
                         [ctypes.c_long, ctypes.c_long, ctypes.c_void_p]),
    "qtip_sample_pick": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_uint] +
                         [ctypes.c_void_p] * 4 + [ctypes.c_long, ctypes.c_long, ctypes.c_void_p]),
    "qtip_repack": (ctypes.c_int, [ctypes.c_void_p] * 2 + [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "qtip_unpack_trellis": (ctypes.c_int, [ctypes.c_void_p] * 2 + [ctypes.c_long] + [ctypes.c_int] * 3 +
                            [ctypes.c_void_p]),
    "qtip_pack_trellis": (ctypes.c_int, [ctypes.c_void_p] * 2 + [ctypes.c_long] + [ctypes.c_int] * 3 +
                          [ctypes.c_void_p] * 2),
    "qtip_decode_natural": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 7 + [ctypes.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib():
    """The loaded library (loads on first use)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise QtipLibraryError(
                f"{LIB_PATH} not found: build it with `python -m qtip_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        got = handle.qtip_abi_version()
        if got != ABI_VERSION:
            raise QtipLibraryError(f"libqtip_hip.so ABI {got}, Python side expects {ABI_VERSION}: rebuild")
        _lib = handle
    return _lib


_INITIALISED = set()


def init_device(device=None):
    """qtip_init() for `device` (default: the current one), once per device and process: the
    library's one-time set-up, kept out of any later stream capture."""
    dev = torch.cuda.current_device() if device is None else torch.device(device).index
    if dev is None:
        dev = torch.cuda.current_device()
    if dev not in _INITIALISED:
        with torch.cuda.device(dev):
            check(lib().qtip_init(), "qtip_init")
        _INITIALISED.add(dev)


def check(code, what):
    if code != 0:
        msg = lib().qtip_error_string(code).decode()
        raise QtipLibraryError(f"{what} failed ({code}): {msg}")


def stream_ptr(device):
    """Current stream of `device` as the launchers take it; also the point where a device the
    library has not met yet gets its one-time set-up (every launch passes through here)."""
    init_device(device)
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_cuda(t, name, dtype=None, contiguous=True):
    """Argument checks of the reference's tensor shim (qtip-kernels/src/qtip_torch.cu:21-46):
    device tensor, contiguous, expected dtype; raises instead of terminating."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (got device {t.device})")
    if contiguous and not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise TypeError(f"{name} has dtype {t.dtype}, expected {dtype}")
    return t
