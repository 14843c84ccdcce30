"""BitshiftLinear on the HIP kernels: the drop-in for lib/codebook/bitshift.py.

Kept from the reference: class names, constructor and forward signatures,
attribute names (`cb`, `scale`, `internal_dtype`, `has_kernel`), tensor
layouts and the cast points of the forward pass.  The quantiser side of
`bitshift_codebook` (Viterbi, `quantize`, `update`) is not part of the
inference path and raises NotImplementedError.  Every decode mode of the
reference is available on the natural-packing path; the fused kernels cover
the HYB code ('quantlut_sym', has_kernel).
"""
import math

import torch
from torch import nn

from .. import ops
from ..utils.kernel_check import has_kernel as _has_kernel
from ..utils.matmul_had import (MANY_ROWS_MIN, MANY_ROWS_MIN_ORDER, had_bits, matmul_hadU_cuda, matmul_hadUt_cuda,
                                rht_many_rows)


def quantlut_sym(tlut, L, nbits):
    """HYB expansion of the tunable table to all 2**L states
    (lib/codebook/bitshift.py:72-80): index bits 6..14 of s*(s+1) (for
    nbits = 9), element 0 negated when bit 15 is set."""
    with torch.no_grad():
        s = torch.arange(1 << L, device=tlut.device)
        p = (s + 1) * s
        flip = 1 - ((p >> 15) & 1) * 2
        idx = (p >> (16 - nbits - 1)) & ((1 << nbits) - 1)
    lut = tlut[idx]
    lut[:, 0] = lut[:, 0] * flip
    return lut


def _byte_sum_code(x):
    """Sum of the four bytes of a 32-bit word, centred and scaled to unit variance: the value map
    shared by the computed codes '1mad' and '2mad' (lib/codebook/bitshift.py:17-40)."""
    y = sum((x >> sh) & 255 for sh in (0, 8, 16, 24)) - 510
    return y.to(torch.float32) / 147.800537109375


def decode_1mad(x):
    """'1mad' computed code (lib/codebook/bitshift.py:17-26): one 32-bit multiply-add, byte sum."""
    m32 = (1 << 32) - 1
    x = ((x.to(torch.int64) & m32) * 34038481 + 76625530) & m32
    return _byte_sum_code(x)


def decode_2mad(x):
    """'2mad' computed code (lib/codebook/bitshift.py:29-40): LCG step, multiply-high add, byte sum."""
    m32 = (1 << 32) - 1
    x = ((x.to(torch.int64) & m32) * 264435761 + 1013904223) & m32
    x = (((x * 1664525) >> 32) + x) & m32
    return _byte_sum_code(x)


def decode_3inst(x):
    """'3inst' computed code (lib/codebook/bitshift.py:43-59): multiply-add, keep sign and 12
    mantissa/exponent bits of each half, xor a constant exponent pattern in, add the two fp16s."""
    m32 = (1 << 32) - 1
    x = ((x.to(torch.int64) & m32) * 89226354 + 64248484) & m32
    keep = (1 << 15) + ((1 << 12) - 1)
    res = (x & ((keep << 16) + keep)) ^ 996162400
    halves = torch.stack([res >> 16, res & 0xFFFF]).to(torch.int32)
    fp = (halves - ((halves >= 1 << 15).to(torch.int32) << 16)).to(torch.int16).view(torch.float16)
    return (fp[0] + fp[1]).float()


def quantlut(tlut, L, nbits):
    """Expansion of a tunable table without the sign trick (lib/codebook/bitshift.py:62-69)."""
    with torch.no_grad():
        s = torch.arange(1 << L, device=tlut.device)
        idx = (((s + 1) * s) >> (16 - nbits)) & ((1 << nbits) - 1)
    return tlut[idx]


_COMPUTED = {'1mad': decode_1mad, '2mad': decode_2mad, '3inst': decode_3inst}


class bitshift_codebook(nn.Module):
    """Decode side of the reference class (lib/codebook/bitshift.py:83-201, 294-353): holds the
    expanded table `lut` (V, 2**L) of the chosen decode mode ('lut', '1mad', '2mad', '3inst',
    'quantlut', 'quantlut_sym'), maps states to weights (`recons`) and converts between states and
    the natural packing.  The quantiser side (Viterbi search) raises NotImplementedError."""

    def __init__(self, L=16, K=2, V=2, tlut_bits=16, decode_mode='lut', tlut=None):
        super().__init__()
        self.idx_dtype = torch.int32
        self.opt_scale = 1
        self.L, self.K, self.V = L, K, V
        self.tlut_bits = tlut_bits
        self.decode_mode = decode_mode
        if L != 16:
            raise NotImplementedError("only L = 16 trellises are built (16-bit state windows)")
        if decode_mode in _COMPUTED:
            if V != 1:
                raise ValueError(f"decode_mode {decode_mode!r} needs V == 1")
            self.register_buffer('lut', _COMPUTED[decode_mode](torch.arange(2**L)).unsqueeze(0))
        elif decode_mode in ('lut', 'quantlut', 'quantlut_sym'):
            if tlut is None:
                self.register_buffer('tlut', self._default_tlut())
                self.register_buffer('lut', self._expand().T.contiguous())
            else:
                self.tlut = tlut
                self.recons_lut()
        else:
            raise ValueError(f"unknown decode_mode {decode_mode!r}")
        self.version = 0

    def _default_tlut(self):
        """Start tables of lib/codebook/bitshift.py:106-168 (a checkpoint overwrites them)."""
        n, V = 2**self.tlut_bits, self.V
        if self.decode_mode == 'lut':
            if self.tlut_bits != self.L:
                raise ValueError("decode_mode 'lut' needs tlut_bits == L")
            return torch.randn(n, V)
        if self.decode_mode == 'quantlut':
            if V == 1:
                return (torch.erfinv((torch.arange(n) + 0.5) / n * 2 - 1) * 2.0**0.5).unsqueeze(-1)
            if V == 2:
                R = ((n / (n - torch.arange(n))).log() * 2).sqrt()
                return torch.stack([R * torch.arange(n).sin(), R * torch.arange(n).cos()], dim=-1)
            raise ValueError("quantlut needs V in {1, 2}")
        if V != 2:
            raise ValueError("quantlut_sym needs V == 2")
        # the reference fits a k-means table to Gaussian samples here; start from a seeded
        # Gaussian table with the same normalisation instead
        g = torch.Generator().manual_seed(0)
        t = torch.randn(n, V, generator=g)
        return (t / t.std(unbiased=False)) * 0.9682458365518543

    def _expand(self):
        if self.decode_mode == 'lut':
            return self.tlut
        if self.decode_mode == 'quantlut':
            return quantlut(self.tlut, self.L, self.tlut_bits)
        return quantlut_sym(self.tlut, self.L, self.tlut_bits)

    def recons_lut(self):
        if self.decode_mode not in _COMPUTED:
            self.lut = self._expand().T.contiguous()

    def recons(self, encoded, **kwargs):
        return self.lut[:, encoded.int().to(self.lut.device)].to(encoded.device)

    def unpack_trellis(self, packed, T):
        """Natural (non-kernel) packing -> (ntiles, T/V) int32 states
        (lib/codebook/bitshift.py:329-353): state i is the 16-bit window at bit offset i*K*V of
        the tile's circular bitstream.  Device tensors go through the HIP kernel; host tensors
        (checkpoint conversion before upload) use the same window formula in torch."""
        if packed.is_cuda:
            return ops.unpack_trellis(packed.contiguous(), T, self.K, self.V)
        words = packed.view(torch.uint16).to(torch.int32).reshape(-1, T * self.K // 16)
        nxt = torch.roll(words, -1, dims=1)
        win = (words << 16) | nxt
        kv = self.K * self.V
        pos = torch.arange(T // self.V, device=packed.device) * kv
        w_idx, off = pos // 16, pos % 16
        return ((win[:, w_idx] >> (16 - off)) & 0xFFFF).to(torch.int32)

    def pack_trellis(self, trellis):
        """(ntiles, T/V) states -> natural packing, uint16 (lib/codebook/bitshift.py:294-327),
        on the device that holds `trellis` (a GPU tensor is required)."""
        return ops.pack_trellis(trellis.to(torch.int32).contiguous(), self.K, self.V)

    def quantize(self, *a, **k):
        raise NotImplementedError("quantisation (Viterbi) is outside the inference path")

    viterbi = update = quantize_seq = quantize


class BitshiftLinear(nn.Module):

    max_rows = 65535  # rows per launch of the transform / GEMM kernels (grid limit)
    # from this many rows on the dense decode + library GEMM is faster than the fused
    # decompress-GEMM, which runs in passes of 32 rows (measured crossover 128-192 rows for the
    # Llama-2 7B and 70B matrices at 2 and 4 bits)
    dense_rows_min = 160

    def __init__(self, td_x, td_y, L, K, V, tlut_bits, decode_mode, dtype=torch.float16, tlut=None,
                 has_kernel=False):
        super().__init__()
        self.td_x = td_x
        self.td_y = td_y
        self.V = V
        self.cb = bitshift_codebook(L, K, V, tlut_bits, decode_mode, tlut=tlut)
        self.internal_dtype = dtype
        self.has_kernel = has_kernel
        self.scale = 32
        if has_kernel and not _has_kernel(decode_mode, L, K, V, tlut_bits, td_x, td_y):
            raise ValueError("has_kernel=True for a configuration the kernels do not cover")

    # -- dense weights -----------------------------------------------------
    def get_hatW(self, unpacked_trellis, m, n):
        """States in the natural packing -> (m, n) (lib/codebook/bitshift.py:378-381)."""
        return self.cb.recons(unpacked_trellis).transpose(0, 1).transpose(1, 2).reshape(
            m // self.td_x, n // self.td_y, self.td_x, self.td_y).transpose(1, 2).reshape(m, n)

    def get_hatW_natural(self, packed_trellis, m, n):
        """Natural packing -> (m, n) in one launch for any decode mode: what
        get_hatW(cb.unpack_trellis(.)) computes (lib/codebook/bitshift.py:329-381)."""
        lut = self.cb.lut
        if lut.dtype not in (torch.float16, torch.float32):
            lut = lut.float()
        lut = lut.to(packed_trellis.device).contiguous()
        return ops.decode_natural(packed_trellis.contiguous(), lut, m, n, self.td_x, self.td_y, self.cb.K, self.V)

    def get_hatW_kernel(self, trellis, m, n):
        """Kernel-packed trellis -> (m, n) fp16 on the HIP decode kernel
        (lib/codebook/bitshift.py:383-387)."""
        return ops.decode(trellis.reshape(-1), self._tlut16(trellis.device), m, n, self.cb.K)

    def _tlut16(self, device):
        t = self.cb.tlut
        if t.dtype != torch.float16 or t.device != device or not t.is_contiguous():
            t = t.to(device=device, dtype=torch.float16).contiguous()
        return t

    def cache_hatW(self, packed_trellis, had_left, had_right, K_left, K_right, m, n, rcp, tp_rank):
        """Dense transformed weight for mode='train-fixW' (lib/codebook/bitshift.py:389-413)."""
        if self.has_kernel:
            hatW = self.get_hatW_kernel(packed_trellis, m, n)
        else:
            hatW = self.get_hatW_natural(packed_trellis, m, n)
        hatW = hatW.float() / self.scale
        if rcp == 1:
            self.hatW = matmul_hadU_cuda(
                matmul_hadU_cuda(hatW.reshape(tp_rank * m, n // tp_rank), had_left, K_left).reshape(m, n).T.contiguous(),
                had_right, K_right).T.contiguous().to(self.internal_dtype)
        elif rcp == 2:
            self.hatW = matmul_hadU_cuda(
                matmul_hadU_cuda(hatW, had_left, K_left).T.contiguous().reshape(tp_rank * n, m // tp_rank), had_right,
                K_right).reshape(n, m).T.contiguous().to(self.internal_dtype)
        else:
            self.hatW = matmul_hadU_cuda(
                matmul_hadU_cuda(hatW, had_left, K_left).T.contiguous(), had_right,
                K_right).T.contiguous().to(self.internal_dtype)

    # -- forward -------------------------------------------------------------
    def forward(self, input, trellis, SU, SV, had_left, had_right, K_left, K_right, rcp, tp_rank,
                mode='eval', **kwargs):
        """y = (H_R [hatW fp16(H_L^T (x * SU) / 32)]) * (SV * 32), cast to input.dtype
        (lib/codebook/bitshift.py:415-472).  Launches: RHT-in, matvec or GEMM, RHT-out."""
        n, m = len(SU), len(SV)
        if mode == 'train-fixW':
            x = input.view(-1, n).to(torch.float32) * SU
            x = (x.to(self.internal_dtype) @ self.hatW.T).float()
            x = x.to(SV.device) * (SV * self.scale)
            return x.view(*input.shape[:-1], m).to(input.dtype)
        if mode not in ('eval', 'train-recons'):
            raise NotImplementedError(f"mode {mode!r}")
        if mode == 'train-recons':
            self.cb.recons_lut()
        rcp = int(rcp)
        tp_rank = int(tp_rank)
        if torch.is_grad_enabled() and (input.requires_grad or SU.requires_grad or SV.requires_grad):
            return self._forward_autograd(input, trellis, SU, SV, had_left, had_right, K_left, K_right, rcp,
                                          tp_rank, mode)
        dev = input.device
        x = input.reshape(-1, n)
        bs = x.shape[0]
        if bs == 0:
            return input.new_empty(*input.shape[:-1], m)
        if bs > self.max_rows:  # the launchers take at most 65535 rows: go through in slabs
            outs = [self.forward(x[i:i + self.max_rows], trellis, SU, SV, had_left, had_right, K_left, K_right,
                                 rcp, tp_rank, mode=mode, **kwargs) for i in range(0, bs, self.max_rows)]
            return torch.cat(outs, dim=0).view(*input.shape[:-1], m)

        # ---- input transform: fp16(H_L^T (x * SU) / sqrt(n) / 32)
        fused_in = (rcp != 1 and SU.dtype == torch.float16 and x.dtype in (torch.float16, torch.float32))
        # one token, power-of-two input size: the matvec kernel transforms its input itself
        in_matvec = (fused_in and bs == 1 and self.has_kernel and K_left == 1 and x.dtype == torch.float16
                     and n in ops.RHT_IN_MATVEC_SIZES)
        if in_matvec:
            xt = None
        elif fused_in and bs >= MANY_ROWS_MIN and K_left >= MANY_ROWS_MIN_ORDER:
            xt = rht_many_rows(x, had_left, K_left, True, pre=SU, scale=(n**-0.5) / self.scale,
                               out_dtype=torch.float16)
        elif fused_in:
            xt = ops.rht(x.contiguous(), order=K_left,
                         had_bits=had_bits(had_left, K_left, True, dev) if K_left > 1 else None,
                         pre=SU.contiguous(), scale=(n**-0.5) / self.scale, out_dtype=torch.float16)
        else:
            xf = x.to(torch.float32) * SU
            if rcp == 1:
                xf = xf.reshape(-1, n // tp_rank)
            nn_ = xf.shape[-1]
            xt = ops.rht(xf.contiguous(), order=K_left,
                         had_bits=had_bits(had_left, K_left, True, dev) if K_left > 1 else None,
                         scale=(nn_**-0.5) / self.scale, out_dtype=torch.float16).reshape(bs, n)

        # ---- quantised matmul
        in_parts = 1
        if self.has_kernel:
            tl = self._tlut16(dev)
            if in_matvec:
                y = ops.decompress_matvec_parts_rht(trellis.reshape(-1), x.reshape(-1), SU.contiguous(),
                                                    (n**-0.5) / self.scale, tl.reshape(-1), m, n, self.cb.K)
                in_parts = y.shape[0]
            elif bs == 1:
                # same kernel as the quip_lib::decompress_matvec_qtip_* op; the k-split
                # partial sums (if any) are added by the output transform on load
                y = ops.decompress_matvec_parts(trellis.reshape(-1), xt.reshape(-1), tl.reshape(-1), m, n, self.cb.K)
                in_parts = y.shape[0]
            elif bs < self.dense_rows_min:
                y = ops.decompress_gemm(trellis.reshape(-1), xt, tl, m, n, self.cb.K, round_f16=True)
            else:
                # many rows: decode once to dense fp16 and let the BLAS library multiply, which is
                # what the reference does for every batch (bitshift.py:476-489)
                hatW = ops.decode(trellis.reshape(-1), tl.reshape(-1), m, n, self.cb.K)
                y = (xt @ hatW.T).float()
                del hatW
        else:
            if mode == 'eval':
                hatW = self.get_hatW_natural(trellis, m, n)
            else:  # the owning module already turned the trellis into states
                hatW = self.get_hatW(trellis, m, n)
            y = (xt.to(hatW.dtype) @ hatW.T).float()

        # ---- output transform: (H_R y / sqrt(m)) * SV * 32, cast
        fused_out = (rcp != 2 and SV.dtype == torch.float32 and SV.device == dev
                     and input.dtype in (torch.float16, torch.float32))
        if fused_out and bs >= MANY_ROWS_MIN and K_right >= MANY_ROWS_MIN_ORDER and in_parts == 1:
            out = rht_many_rows(y.reshape(bs, m), had_right, K_right, False, post=SV,
                                scale=(m**-0.5) * self.scale, out_dtype=input.dtype)
        elif fused_out:
            out = ops.rht(y if in_parts > 1 else y.reshape(bs, m), order=K_right,
                          had_bits=had_bits(had_right, K_right, False, dev) if K_right > 1 else None,
                          post=SV.contiguous(), scale=(m**-0.5) * self.scale, out_dtype=input.dtype,
                          in_parts=in_parts)
        else:
            if in_parts > 1:
                y = y.sum(0, keepdim=True)
            yy = y.reshape(-1, m // tp_rank) if rcp == 2 else y
            mm = yy.shape[-1]
            yt = ops.rht(yy.contiguous(), order=K_right,
                         had_bits=had_bits(had_right, K_right, False, dev) if K_right > 1 else None,
                         scale=mm**-0.5, out_dtype=torch.float32).reshape(bs, m)
            out = (yt.to(SV.device) * (SV * self.scale)).to(input.dtype)
        return out.view(*input.shape[:-1], m)


    def _forward_autograd(self, input, trellis, SU, SV, had_left, had_right, K_left, K_right, rcp, tp_rank, mode):
        """The same forward as a chain of differentiable steps, as the reference runs it when
        fine-tuning (lib/codebook/bitshift.py:428-472): gradients reach the input and the sign
        vectors SU / SV; the trellis is fixed and the table gets no gradient on the kernel path
        (BitshiftLinearKernelAG returns None for it, :491-505)."""
        n, m = len(SU), len(SV)
        x = input.reshape(-1, n).to(torch.float32) * SU
        if rcp == 1:
            x = matmul_hadUt_cuda(x.reshape(-1, n // tp_rank), had_left, K_left).reshape(x.shape) / self.scale
        else:
            x = matmul_hadUt_cuda(x, had_left, K_left) / self.scale
        if self.has_kernel:
            x = BitshiftLinearKernelAG.apply(x, trellis, m, n, self.cb.L, self.cb.tlut_bits, self.cb.K, self.V,
                                             self.cb.lut).float()
        else:
            hatW = self.get_hatW_natural(trellis, m, n) if mode == 'eval' else self.get_hatW(trellis, m, n)
            x = (x.to(hatW.dtype) @ hatW.T).float()
        if rcp == 2:
            x = matmul_hadU_cuda(x.reshape(-1, m // tp_rank), had_right, K_right).reshape(x.shape)
        else:
            x = matmul_hadU_cuda(x, had_right, K_right)
        x = x.to(SV.device) * (SV * self.scale)
        return x.view(*input.shape[:-1], m).to(input.dtype)


class BitshiftLinearKernelAG(torch.autograd.Function):
    """x @ decode(trellis)^T with the weights re-decoded in backward
    (lib/codebook/bitshift.py:476-505).  Forward uses the fused
    decompress-GEMM; backward decodes to a dense matrix and uses a dense GEMM."""

    @staticmethod
    def forward(ctx, input, trellis, m, n, L, tlut_bits, K, V, lut):
        from ..utils.kernel_decompress import tlut_from_expanded
        tlut = tlut_from_expanded(lut.T)
        ctx.save_for_backward(trellis, tlut)
        ctx.shape = (m, n, K)
        x = input.to(torch.float16).reshape(-1, n).contiguous()
        if x.shape[0] == 1:
            y = ops.decompress_matvec(trellis.reshape(-1), x.reshape(-1), tlut.reshape(-1), m, n, K).view(1, m)
            y = y.to(torch.float16)
        elif x.shape[0] < BitshiftLinear.dense_rows_min:
            y = ops.decompress_gemm(trellis.reshape(-1), x, tlut.reshape(-1), m, n, K, round_f16=True).to(torch.float16)
        else:
            y = x @ ops.decode(trellis.reshape(-1), tlut.reshape(-1), m, n, K).T
        return y.view(*input.shape[:-1], m)

    @staticmethod
    def backward(ctx, grad_output):
        trellis, tlut = ctx.saved_tensors
        m, n, K = ctx.shape
        hatW = ops.decode(trellis.reshape(-1), tlut.reshape(-1), m, n, K)
        grad_input = grad_output.to(hatW.dtype) @ hatW
        return grad_input, None, None, None, None, None, None, None, None
