"""GPU parity of the dense-math seam (cfp_gemm_*) and the unfused elementwise
kernels against fp64 matmuls (textbook GEMM), 1e-4 relative."""
import numpy as np
import pytest

from parity_util import GRU, HIDDEN, OBS, TOL_FP32, assert_close

pytestmark = pytest.mark.gpu


def _r(shape, cuda, seed, scale=1.0):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(cuda)


@pytest.mark.parametrize("m,cols,k", [(768, 500, 256), (44, 96, 256), (43, 1, 256),
                                      (768, 16384, 256), (100, 33, 77)])
def test_gemm_fwd(pkg, cuda, m, cols, k):
    import torch
    W, x = _r((m, k), cuda, 1, 0.1), _r((cols, k), cuda, 2)
    y = pkg.policy.gemm_fwd(W, x)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), (x.double() @ W.double().T).cpu().numpy(), TOL_FP32, "gemm_fwd")


@pytest.mark.parametrize("cols", [1, 100, 4096])
def test_gemm_enc_fwd(pkg, cuda, cols):
    import torch
    W, x = _r((OBS, HIDDEN), cuda, 3, 0.05), _r((cols, OBS), cuda, 4, 5.0)
    h = pkg.policy.gemm_enc_fwd(W, x)
    torch.cuda.synchronize()
    assert_close(h.cpu().numpy(), (x.double() @ W.double()).cpu().numpy(), TOL_FP32, "gemm_enc_fwd")


@pytest.mark.parametrize("m3,cols", [(768, 777), (43, 130), (768, 8192)])
def test_gemm_dh(pkg, cuda, m3, cols):
    import torch
    W, d = _r((m3, HIDDEN), cuda, 5, 0.1), _r((cols, m3), cuda, 6)
    dh = pkg.policy.gemm_dh(W, d)
    torch.cuda.synchronize()
    assert_close(dh.cpu().numpy(), (d.double() @ W.double()).cpu().numpy(), TOL_FP32, "gemm_dh")


@pytest.mark.parametrize("rows,cols", [(768, 5000), (43, 300), (843, 2048), (768, 31), (768, 65536)])
def test_gemm_dw_accumulates(pkg, cuda, rows, cols):
    import torch
    x, d = _r((cols, HIDDEN), cuda, 7), _r((cols, rows), cuda, 8)
    dW = torch.full((rows, HIDDEN), 0.5, device=cuda)
    pkg.policy.gemm_dw(x, d, dW)
    torch.cuda.synchronize()
    want = 0.5 + (d.double().T @ x.double())
    assert_close(dW.cpu().numpy(), want.cpu().numpy(), TOL_FP32, "gemm_dw")
    # split-K sums in a fixed order: run-to-run bitwise stable
    dW2 = torch.full((rows, HIDDEN), 0.5, device=cuda)
    pkg.policy.gemm_dw(x, d, dW2)
    torch.cuda.synchronize()
    assert torch.equal(dW, dW2)


def test_gemv_dwv(pkg, cuda):
    import torch
    x, dv = _r((5000, HIDDEN), cuda, 9), _r((5000,), cuda, 10)
    out = torch.ones(HIDDEN, device=cuda)
    pkg.policy.gemv_dwv(x, dv, out)
    torch.cuda.synchronize()
    assert_close(out.cpu().numpy(), (1.0 + x.double().T @ dv.double()).cpu().numpy(), TOL_FP32, "gemv_dwv")


def test_unfused_epilogue_and_bias(pkg, cuda):
    """k_add_bias / k_mingru_epi_fwd equivalents against the closed form in fp64."""
    import torch
    cols = 300
    pre, x = _r((cols, GRU), cuda, 11, 2.0), _r((cols, HIDDEN), cuda, 12)
    st0 = _r((cols, HIDDEN), cuda, 13, 0.5)
    term = (torch.rand(cols, device=cuda) < 0.3).float()
    state = st0.clone(); rs = torch.zeros_like(st0)
    h = pkg.policy.mingru_epi_fwd(pre, x, state, term, r_state_store=rs)
    torch.cuda.synchronize()
    p64, x64 = pre.double(), x.double()
    s = torch.where(term[:, None] != 0, torch.zeros_like(p64[:, :HIDDEN]), st0.double())
    zh, zg, zp = p64[:, :HIDDEN], p64[:, HIDDEN:2 * HIDDEN], p64[:, 2 * HIDDEN:]
    gh = torch.where(zh >= 0, zh + 0.5, torch.sigmoid(zh))
    out = s + torch.sigmoid(zg) * (gh - s)
    pg = torch.sigmoid(zp)
    assert_close(state.cpu().numpy(), out.cpu().numpy(), TOL_FP32, "epi state")
    assert_close(h.cpu().numpy(), (pg * out + (1 - pg) * x64).cpu().numpy(), TOL_FP32, "epi h")
    assert torch.equal(rs, s.float())
    b = _r((HIDDEN,), cuda, 14)
    hb = x.clone()
    pkg.policy.add_bias(hb, b)
    torch.cuda.synchronize()
    assert torch.equal(hb, x + b)
