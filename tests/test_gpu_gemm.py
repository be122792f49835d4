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


def _check_split_errors(errs):
    """errs[mode] = max |got - fp64| / sum_k |a_k b_k|.  Mode 1 (nine exact partial
    products) must sit at the fp32 MFMA kernel's level (mode 0); mode 2 (six) may add
    its documented 2^-23 per product on top; mode 3 (eight: only lo*lo left out, below
    2^-30 of a product) is held to the bar of mode 1."""
    assert errs[1] <= 3.0 * errs[0] + 1e-7, errs
    assert errs[1] < 2e-6, errs
    assert errs[3] <= 3.0 * errs[0] + 1e-7 and errs[3] < 2e-6, errs
    assert abs(errs[3] - errs[1]) <= 2.0 ** -28, errs
    assert errs[2] <= 3.0 * errs[0] + 1e-7 + 2.0 ** -23, errs


def test_gemm_split_mode_is_checked(pkg, cuda):
    with pytest.raises(pkg._lib.CfpError, match="mode must be 0..3"):
        pkg.policy.set_gemm_split(4)
    assert pkg.policy.lib().cfp_get_gemm_split() == 1


@pytest.mark.parametrize("rows,cols", [(768, 4096), (768, 1000), (128, 8), (75, 2048), (43, 520),
                                       (843, 264)])
def test_gemm_dw_split_is_as_accurate_as_fp32_mfma(pkg, cuda, rows, cols):
    """fp32 operands as bf16 triples, nine partial products each: the error against
    fp64 must stay at the level of the fp32 MFMA kernel's.  A missing partial product
    would show as a relative error of 2^-16 (hi*lo) or 2^-8 (hi*mid), far above it."""
    import torch
    x, d = _r((cols, HIDDEN), cuda, 21), _r((cols, rows), cuda, 22)
    want = (d.double().T @ x.double())
    scale = (d.double().abs().T @ x.double().abs())
    errs = {}
    assert pkg.policy.lib().cfp_get_gemm_split() == 1
    for mode in (1, 2, 3, 0):
        pkg.policy.set_gemm_split(mode)
        dW = torch.zeros(rows, HIDDEN, device=cuda)
        pkg.policy.gemm_dw(x, d, dW)
        torch.cuda.synchronize()
        errs[mode] = ((dW.double() - want).abs() / scale).max().item()
    pkg.policy.set_gemm_split(1)
    _check_split_errors(errs)


@pytest.mark.parametrize("m3,cols", [(768, 8192), (768, 32), (768, 4000 * 32), (48, 288)])
def test_gemm_dh_split_is_as_accurate_as_fp32_mfma(pkg, cuda, m3, cols):
    """Same bar for dh = dpre . W on bf16 triples (W split into an MFMA-ordered mirror,
    dpre in registers).  The accumulating form (layer 0 of the update, onto the highway
    term) has no entry point of its own and is covered by the trainer's parity tests."""
    import torch
    W, d = _r((m3, HIDDEN), cuda, 23, 0.1), _r((cols, m3), cuda, 24)
    want = d.double() @ W.double()
    scale = d.double().abs() @ W.double().abs()
    errs = {}
    for mode in (1, 2, 3, 0):
        pkg.policy.set_gemm_split(mode)
        out = pkg.policy.gemm_dh(W, d)
        torch.cuda.synchronize()
        errs[mode] = ((out.double() - want).abs() / scale).max().item()
    pkg.policy.set_gemm_split(1)
    _check_split_errors(errs)


@pytest.mark.parametrize("m,cols,k", [(768, 8192, 256), (256, 64, 32), (768, 32000, 256)])
def test_gemm_fwd_split_is_as_accurate_as_fp32_mfma(pkg, cuda, m, cols, k):
    """The gate-forward shape y = x . W^T on the dh kernel, 256 rows of W at a time."""
    import torch
    W, x = _r((m, k), cuda, 26, 0.1), _r((cols, k), cuda, 27)
    want = x.double() @ W.double().T
    scale = x.double().abs() @ W.double().abs().T
    errs = {}
    for mode in (1, 2, 3, 0):
        pkg.policy.set_gemm_split(mode)
        out = pkg.policy.gemm_fwd(W, x)
        torch.cuda.synchronize()
        errs[mode] = ((out.double() - want).abs() / scale).max().item()
    pkg.policy.set_gemm_split(1)
    _check_split_errors(errs)


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


# ---- bf16-input / fp32-accumulate seam (cfp_set_gemm_bf16) ---------------------------
@pytest.fixture
def bf16_gemms(pkg):
    pkg.policy.set_gemm_bf16(True)
    yield
    pkg.policy.set_gemm_bf16(False)


def _grid(t):
    """fp32 tensor rounded to the bf16 grid (so that the kernel's own rounding is exact)."""
    import torch
    return t.to(torch.bfloat16).to(torch.float32)


@pytest.mark.parametrize("exact", [True, False])
def test_bf16_gemms(pkg, cuda, bf16_gemms, exact):
    """All four GEMM shapes with bf16 inputs.  exact=True: operands already on the
    bf16 grid, every product is exact and the result must match fp64 to fp32
    summation accuracy (pins fragment layout and the LDS transposition of both
    operand orientations, vector and scalar load paths, edge tiles, split-K);
    exact=False: arbitrary fp32 operands, 2e-2 relative to fp64 and 1e-4 against
    fp64 on the bf16-rounded operands (the rounding is to nearest even)."""
    import torch
    from parity_util import TOL_BF16

    def check(got, a, b, what, base=None):
        ref = a.double() @ b.double()
        ref_q = _grid(a).double() @ _grid(b).double()
        if base is not None:
            ref, ref_q = ref + base, ref_q + base
        assert_close(got.cpu().numpy(), ref_q.cpu().numpy(), 1e-4, what + " vs bf16-rounded fp64")
        if not exact:
            assert_close(got.cpu().numpy(), ref.cpu().numpy(), TOL_BF16, what + " vs fp64")

    prep = _grid if exact else (lambda t: t)
    for m, cols, k in [(768, 500, 256), (44, 96, 256), (100, 33, 77), (768, 16384, 256)]:
        W, x = prep(_r((m, k), cuda, 1, 0.1)), prep(_r((cols, k), cuda, 2))
        check(pkg.policy.gemm_fwd(W, x), x, W.T, f"bf16 gemm_fwd {m}x{cols}x{k}")
    for cols in (1, 100, 4096):
        W, x = prep(_r((OBS, HIDDEN), cuda, 3, 0.05)), prep(_r((cols, OBS), cuda, 4, 5.0))
        check(pkg.policy.gemm_enc_fwd(W, x), x, W, f"bf16 gemm_enc_fwd {cols}")
    for m3, cols in [(768, 777), (43, 130), (768, 8192)]:
        W, d = prep(_r((m3, HIDDEN), cuda, 5, 0.1)), prep(_r((cols, m3), cuda, 6))
        check(pkg.policy.gemm_dh(W, d), d, W, f"bf16 gemm_dh {m3}x{cols}")
    for rows, cols in [(768, 5000), (43, 300), (843, 2048), (768, 31), (768, 65536)]:
        x, d = prep(_r((cols, HIDDEN), cuda, 7)), prep(_r((cols, rows), cuda, 8))
        dW = torch.full((rows, HIDDEN), 0.5, device=cuda)
        pkg.policy.gemm_dw(x, d, dW)
        check(dW, d.T, x, f"bf16 gemm_dw {rows}x{cols}", base=0.5)
    torch.cuda.synchronize()


def test_bf16_switch_is_off_by_default_and_reversible(pkg, cuda):
    import torch
    W, x = _r((768, 256), cuda, 1, 0.1), _r((300, 256), cuda, 2)
    assert pkg.lib().cfp_get_gemm_bf16() == 0
    y0 = pkg.policy.gemm_fwd(W, x)
    pkg.policy.set_gemm_bf16(True)
    y1 = pkg.policy.gemm_fwd(W, x)
    pkg.policy.set_gemm_bf16(False)
    y2 = pkg.policy.gemm_fwd(W, x)
    torch.cuda.synchronize()
    assert torch.equal(y0, y2) and not torch.equal(y0, y1)
