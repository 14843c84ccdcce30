"""Measurement aids of bench.py (libqtip_probe.so, declared in bench_probe/qtip_probe.h): the
stream-read ceiling of the box, the issue rate of the instructions of the 2-bit decode and its
loop without memory.  Not part of the qtip_amd package: nothing under qtip_amd/ imports this."""
import ctypes
import os
import subprocess
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libqtip_probe.so")
SRC = os.path.join(HERE, "qtip_probe.hip")

# the product sources compiled with -DQTIP_STAMPS: wave 0 of every matvec workgroup records a few
# readings of the constant clock (bench.py --timeline prints them); never loaded by default
STAMPED_LIB_PATH = os.path.join(HERE, "libqtip_hip_stamped.so")

OPS_PER_ITER = 88
KINDS = {"v_and_b32": 0, "v_add_u32": 1, "v_lshrrev_b32": 2, "v_lshlrev_b32": 3, "v_pk_mad_u16": 4,
         "v_mad_u32_u16": 5, "v_perm_b32": 6, "v_pk_lshrrev_b16": 7, "v_mov_b32_dpp": 8, "v_dot2c_f32_f16": 9,
         "ds_read_b32": 10, "v_mfma_f32_16x16x32_f16": 11, "decode_loop": 100, "decode_loop_valu": 101}

_lib = None


class ProbeError(RuntimeError):
    pass


def build(verbose=True):
    """hipcc --offload-arch=gfx950 of qtip_probe.hip into libqtip_probe.so, in-tree."""
    cmd = [os.environ.get("HIPCC", "hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", SRC, "-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def build_stamped(verbose=True):
    """The timeline build of libqtip_hip.so (same sources and flags, plus -DQTIP_STAMPS)."""
    from qtip_amd import build as qbuild
    cmd = [os.environ.get("HIPCC", "hipcc")] + qbuild.HIPCC_FLAGS + ["-DQTIP_STAMPS"] + qbuild.SRCS + \
        ["-o", STAMPED_LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l))
    os.replace(STAMPED_LIB_PATH + ".tmp", STAMPED_LIB_PATH)
    return STAMPED_LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ProbeError(f"{LIB_PATH} not found: build it with `python -m bench_probe`")
        h = ctypes.CDLL(LIB_PATH)
        h.qtip_probe_stream_read.restype = ctypes.c_int
        h.qtip_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        h.qtip_probe_issue.restype = ctypes.c_int
        h.qtip_probe_issue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        _lib = h
    return _lib


def _check(rc, what):
    if rc != 0:
        raise ProbeError(f"{what} failed ({rc})")


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def stream_read(src):
    """Read the tensor once with the matvec's kind of loads; returns the per-wave folded words."""
    if not (isinstance(src, torch.Tensor) and src.is_cuda and src.is_contiguous()):
        raise ValueError("src must be a contiguous GPU tensor")
    cus = torch.cuda.get_device_properties(src.device).multi_processor_count
    sink = torch.empty(16 * cus, dtype=torch.int32, device=src.device)
    with torch.cuda.device(src.device):
        _check(lib().qtip_probe_stream_read(sink.data_ptr(), src.data_ptr(), src.numel() * src.element_size(),
                                            _stream(src.device)), "qtip_probe_stream_read")
    return sink


def issue(kind, iters, tlut, sink=None):
    """One launch of the instruction-rate probe: `kind` a key of KINDS.  The caller times it."""
    if kind not in KINDS:
        raise ValueError(f"unknown probe kind {kind!r}")
    if not (isinstance(tlut, torch.Tensor) and tlut.is_cuda and tlut.dtype == torch.float16 and tlut.numel() == 1024):
        raise ValueError("tlut holds 512 x 2 fp16 values on the GPU")
    cus = torch.cuda.get_device_properties(tlut.device).multi_processor_count
    if sink is None:
        sink = torch.empty(1024 * cus, dtype=torch.int32, device=tlut.device)
    with torch.cuda.device(tlut.device):
        _check(lib().qtip_probe_issue(KINDS[kind], int(iters), tlut.data_ptr(), sink.data_ptr(), _stream(tlut.device)),
               "qtip_probe_issue")
    return sink
