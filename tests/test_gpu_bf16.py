"""GPU parity of the bf16-input / fp32-accumulate forward (cfp_policy_set_gemm_bf16)
through the C ABI.

Three kinds of checks:
  * against the fp64 oracle on the same fp32 weights: 2e-2 in the relative
    Frobenius norm for hidden states, logits and values (parity_util explains why
    the per-entry metric of the fp32 tests cannot apply to bf16 inputs);
  * against an fp64 evaluation of the same bf16-rounded operands
    (parity_util.numpy_forward_bf16_f64): 1e-3 in the relative Frobenius norm and
    5e-2 per entry -- the kernel computes the bf16-input / fp32-accumulate
    function itself; what is left are the rare activations that sit on a bf16
    rounding boundary and round the other way in fp32 than in fp64;
  * operand-layout pins: with weights and activations that are exactly
    representable in bf16 every product is exact, so the kernel must agree with
    fp64 to fp32 summation accuracy (1e-5) -- a transposed or permuted MFMA
    operand cannot pass this.
The recurrent state and r_state stay fp32; the post-zero state record is exact."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import (ACTIONS, HIDDEN, TOL_BF16, assert_close, bf16_round, expand_records,
                         fro_err, numpy_forward_bf16_f64, random_params, split_params,
                         synth_records_host, synth_classic_records_host)

TOL_EMUL_FRO = 1e-3
TOL_EMUL_ENTRY = 5e-2


def _fro_close(got, ref, what, tol=TOL_BF16):
    e = fro_err(got, ref)
    assert np.all(np.isfinite(np.asarray(got))), f"{what}: non-finite values"
    assert e <= tol, f"{what}: relative Frobenius error {e:.3e} exceeds {tol:.1e}"
    return e


def _emul_close(got, emul, what):
    e = _fro_close(got, emul, what + " vs fp64 on bf16-rounded operands", TOL_EMUL_FRO)
    assert_close(got, emul, TOL_EMUL_ENTRY, what + " vs fp64 on bf16-rounded operands")
    return e

pytestmark = pytest.mark.gpu
L = 3


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def _bf16_grid(a):
    """fp32 values rounded to the nearest bf16, returned as fp32."""
    return bf16_round(a).astype(np.float32)


@pytest.mark.parametrize("n,layers,term_p", [(32, 3, 0.0), (96, 3, 0.3), (256, 2, 0.5), (1024, 3, 0.1)])
def test_bf16_forward_within_tolerance(pkg, cuda, n, layers, term_p):
    import torch
    params = random_params(layers, 300 + n)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    pol.set_gemm_bf16(True)
    assert pol.gemm_bf16
    rng = np.random.default_rng(n + 1)
    rec_h = synth_records_host(n, 6, n)
    state_h = (0.5 * rng.standard_normal((layers, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < term_p).astype(np.float32)
    ref = ob.forward_f64(params, layers, expand_records(rec_h), state_h, term_h)
    state = _t(state_h, cuda)
    r_state = torch.zeros(layers, n, HIDDEN, device=cuda)
    h_enc = torch.zeros(n, HIDDEN, device=cuda)
    h3 = torch.zeros(n, HIDDEN, device=cuda)
    av = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state, r_state_t=r_state, h_enc=h_enc, h3=h3)
    torch.cuda.synchronize()
    av_h = av.cpu().numpy()
    got = {"h_enc": h_enc.cpu().numpy(), "h3": h3.cpu().numpy(), "state": state.cpu().numpy(),
           "logits": av_h[:, :ACTIONS], "values": av_h[:, ACTIONS]}
    emul = numpy_forward_bf16_f64(params, layers, expand_records(rec_h), state_h, term_h)
    errs = []
    for k, v in got.items():
        errs.append(_fro_close(v, ref[k], f"bf16 {k} vs fp64 oracle"))
        _emul_close(v, emul[k], f"bf16 {k}")
    assert np.array_equal(r_state.cpu().numpy(), ref["r_state"].astype(np.float32))
    # the bf16 kernel really ran: its error is far above the fp32 kernel's
    assert max(errs) > 2e-4
    pol.close()


def test_bf16_switch_back_to_fp32_is_bitwise_the_fp32_kernel(pkg, cuda):
    import torch
    n = 64
    pol = pkg.Policy(n, L, seed=5)
    rec = pkg.policy.synth_records(n, 3, 0)
    term = torch.zeros(n, device=cuda)
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    st_a, st_b, st_c = st0.clone(), st0.clone(), st0.clone()
    av_a = pol.forward(rec, term, st_a).clone()
    pol.set_gemm_bf16(True)
    av_b = pol.forward(rec, term, st_b).clone()
    pol.set_gemm_bf16(False)
    av_c = pol.forward(rec, term, st_c).clone()
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_c) and torch.equal(st_a, st_c)
    assert not torch.equal(av_a, av_b)
    pol.close()


def test_bf16_encoder_operand_layout_exact(pkg, cuda):
    """Record bytes are exact in bf16; with W_enc on a coarse dyadic grid and the tail
    floats on the bf16 grid, h_enc must match fp64 to summation accuracy."""
    import torch
    n = 64
    rng = np.random.default_rng(41)
    params = random_params(L, 42)
    w = split_params(params, L)
    w["W_enc"][...] = rng.integers(-8, 9, size=w["W_enc"].shape).astype(np.float32) / 64.0
    rec_h = synth_records_host(n, 8, 1)
    tail = np.ascontiguousarray(rec_h[:, 792:]).view(np.float32)
    rec_h[:, 792:] = _bf16_grid(tail).view(np.uint8).reshape(n, -1)
    pol = pkg.Policy(n, L, seed=1)
    pol.set_params(params)
    pol.set_gemm_bf16(True)
    h_enc = pol.encode_step(_t(rec_h, cuda)).clone()
    torch.cuda.synchronize()
    x = expand_records(rec_h).astype(np.float64)
    ref = x @ w["W_enc"].astype(np.float64) + w["b_enc"].astype(np.float64)
    assert_close(h_enc.cpu().numpy(), ref, 1e-5, "bf16 encoder, exact operands")
    pol.close()


def test_bf16_gate_and_head_operand_layout_exact(pkg, cuda):
    """One layer with W_gru / W_a / W_v and the layer input on bf16-exact grids."""
    import torch
    n, layers = 96, 1
    rng = np.random.default_rng(43)
    params = random_params(layers, 44)
    w = split_params(params, layers)
    w["W_gru"][...] = rng.integers(-8, 9, size=w["W_gru"].shape).astype(np.float32) / 128.0
    w["W_a"][...] = rng.integers(-8, 9, size=w["W_a"].shape).astype(np.float32) / 64.0
    w["W_v"][...] = rng.integers(-8, 9, size=w["W_v"].shape).astype(np.float32) / 64.0
    x0_h = _bf16_grid(rng.standard_normal((n, HIDDEN)).astype(np.float32))
    state_h = (0.5 * rng.standard_normal((layers, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < 0.2).astype(np.float32)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    pol.set_gemm_bf16(True)
    state = _t(state_h, cuda)
    h3 = pol.gru_chain(_t(x0_h, cuda), state, _t(term_h, cuda)).clone()
    # head on a bf16-exact input
    hin = _bf16_grid(rng.standard_normal((n, HIDDEN)).astype(np.float32))
    av = pol.head(_t(hin, cuda)).clone()
    torch.cuda.synchronize()
    # fp64 evaluation of the layer
    W = w["W_gru"][0].astype(np.float64)
    z = x0_h.astype(np.float64) @ W.T
    zh, zg, zp = z[:, :HIDDEN], z[:, HIDDEN:2 * HIDDEN], z[:, 2 * HIDDEN:]
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    st = np.where(term_h[:, None] != 0, 0.0, state_h[0].astype(np.float64))
    out = st + sig(zg) * (np.where(zh >= 0, zh + 0.5, sig(zh)) - st)
    p = sig(zp)
    h_ref = p * out + (1 - p) * x0_h
    assert_close(state.cpu().numpy()[0], out, 1e-5, "bf16 gate GEMM, exact operands: state")
    assert_close(h3.cpu().numpy(), h_ref, 1e-5, "bf16 gate GEMM, exact operands: h")
    logits = hin.astype(np.float64) @ w["W_a"].astype(np.float64).T + w["b_a"]
    values = hin.astype(np.float64) @ w["W_v"].astype(np.float64) + w["b_v"][0]
    av_h = av.cpu().numpy()
    assert_close(av_h[:, :ACTIONS], logits, 1e-5, "bf16 head, exact operands: logits")
    assert_close(av_h[:, ACTIONS], values, 1e-5, "bf16 head, exact operands: values")
    pol.close()


def test_bf16_classic_variant(pkg, cuda):
    """Classic game: the gather encoder stays fp32, gate and head GEMMs run bf16."""
    import torch
    n = 128
    params = random_params(L, 51, obs=1345, actions=17)
    pol = pkg.Policy(n, L, seed=1, variant="classic")
    pol.set_params(params)
    pol.set_gemm_bf16(True)
    rng = np.random.default_rng(52)
    rec_h = synth_classic_records_host(n, 4, 2)
    state_h = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < 0.2).astype(np.float32)
    ref = ob.classic_forward_f64(params, L, ob.classic_expand(rec_h), state_h, term_h)
    state = _t(state_h, cuda)
    h_enc = torch.zeros(n, HIDDEN, device=cuda)
    av = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state, h_enc=h_enc)
    torch.cuda.synchronize()
    av_h = av.cpu().numpy()
    assert_close(h_enc.cpu().numpy(), ref["h_enc"], 1e-4, "classic bf16: fp32 gather encoder")
    emul = numpy_forward_bf16_f64(params, L, ob.classic_expand(rec_h), state_h, term_h, obs=1345,
                                  actions=17, quantize_encoder=False)
    for k, v in (("state", state.cpu().numpy()), ("logits", av_h[:, :17]), ("values", av_h[:, 17])):
        _fro_close(v, ref[k], f"classic bf16 {k} vs fp64 oracle")
        _emul_close(v, emul[k], f"classic bf16 {k}")
    pol.close()
