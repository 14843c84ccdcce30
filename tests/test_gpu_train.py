"""Training-side parity: gradients of the differentiable forward against a float64 dense model."""
import numpy as np
import pytest
import torch

from oracle import qtip_oracle as O
from synth import make_layer

pytestmark = pytest.mark.gpu


def _matrix(n, transpose):
    return torch.from_numpy(O.hadamard_transform(np.eye(n), transpose=transpose).T.copy())  # y = M @ x


@pytest.mark.parametrize("m,k,bs", [(128, 256, 4), (192, 128, 1), (96, 160, 3)])
def test_gradients_of_input_and_sign_vectors(m, k, bs):
    from qtip_amd.codebook.bitshift import BitshiftLinear
    from qtip_amd.utils import matmul_had as mh
    dev = torch.device("cuda:0")
    K = 2
    L = make_layer(m, k, K, seed=m + k)
    tlut = torch.from_numpy(L["tlut"]).to(dev)
    mod = BitshiftLinear(16, 16, 16, K, 2, 9, "quantlut_sym", tlut=tlut, has_kernel=True)
    tr = torch.from_numpy(L["packed"]).to(dev)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(bs, k, generator=g).half().to(dev).requires_grad_(True)
    SU = torch.from_numpy(L["SU"]).to(dev).requires_grad_(True)
    SV = torch.from_numpy(L["SV"]).to(dev).requires_grad_(True)
    hl, Kl = mh.get_hadK(k)
    hr, Kr = mh.get_hadK(m)
    y = mod(x, tr, SU, SV, hl, hr, Kl, Kr, 0, 8, mode="train-recons")
    w = torch.randn(bs, m, generator=g).to(dev)
    (y.float() * w).sum().backward()

    # float64 dense model of lib/codebook/bitshift.py:428-472
    W = torch.from_numpy(O.decode_kernel(L["packed"], L["tlut"], m, k, K).astype(np.float64))
    A, B = _matrix(k, True), _matrix(m, False)
    xd = x.detach().cpu().double().requires_grad_(True)
    SUd = SU.detach().cpu().double().requires_grad_(True)
    SVd = SV.detach().cpu().double().requires_grad_(True)
    yd = (((xd * SUd) @ A.T / 32) @ W.T @ B.T) * (SVd * 32)
    (yd * w.cpu().double()).sum().backward()

    def close(a, b, tol):
        a, b = a.detach().cpu().double(), b.detach().double()
        return float((a - b).abs().max() / b.abs().max()) <= tol

    assert close(y, yd, 1e-2)
    assert close(x.grad, xd.grad, 2e-2)
    assert close(SU.grad, SUd.grad, 2e-2)
    assert close(SV.grad, SVd.grad, 2e-2)
    assert x.grad.dtype == torch.float16 and SV.grad.dtype == torch.float32


def test_hadamard_function_gradient_is_the_transposed_transform():
    from qtip_amd.utils import matmul_had as mh
    dev = torch.device("cuda:0")
    for n in (256, 160, 96):  # 160 = 20 * 8 and 96 = 12 * 8: tables that are not symmetric
        had, K = mh.get_hadK(n)
        x = torch.randn(5, n, device=dev, requires_grad=True)
        y = mh.matmul_hadU_cuda(x, had, K)
        gy = torch.randn(5, n, device=dev)
        (y * gy).sum().backward()
        M = _matrix(n, False).float().to(dev)
        assert torch.allclose(y.detach(), x.detach() @ M.T, atol=1e-4)
        assert torch.allclose(x.grad, gy @ M, atol=1e-4)
        # and it inverts: hadUt(hadU(x)) = x
        z = mh.matmul_hadUt_cuda(y.detach(), had, K)
        assert torch.allclose(z, x.detach(), atol=1e-4)


def test_train_fixW_mode_matches_eval():
    from qtip_amd.linear.quantized_linear import QuantizedLinear
    dev = torch.device("cuda:0")
    m, k, K = 128, 256, 3
    L = make_layer(m, k, K, seed=9)
    outs = {}
    for mode in ("eval", "train-fixW"):
        lin = QuantizedLinear(k, m, 16, 16, 16, K, 2, 9, "quantlut_sym", mode=mode).to(dev)
        with torch.no_grad():
            lin.trellis.copy_(torch.from_numpy(L["packed"]))
            lin.tlut.copy_(torch.from_numpy(L["tlut"]))
            lin.SU.copy_(torch.from_numpy(L["SU"]))
            lin.SV.copy_(torch.from_numpy(L["SV"]))
        x = torch.randn(4, k, generator=torch.Generator().manual_seed(2)).half().to(dev)
        outs[mode] = lin(x).float()
    err = (outs["eval"] - outs["train-fixW"]).abs().max() / outs["eval"].abs().max()
    assert err < 2e-2
