"""GPU parity of the classic-game policy (gathered-column encoder over 148-byte
records, MinGRU x3, actor 17 / value 1) against the fp64 oracle; 1e-4 relative."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import (HIDDEN, TOL_FP32, assert_close, random_params,
                         synth_classic_records_host)

pytestmark = pytest.mark.gpu
L = 3


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def test_classic_synth_records_device_equals_host(pkg, cuda):
    import torch
    for n, seed, step in ((32, 1, 0), (1000, 9, 4)):
        d = pkg.policy.synth_classic_records(n, seed, step)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy(), synth_classic_records_host(n, seed, step))


@pytest.mark.parametrize("n,term_p", [(32, 0.0), (160, 0.3)])
def test_classic_forward_matches_oracle(pkg, cuda, n, term_p):
    import torch
    params = random_params(L, 70 + n, obs=1345, actions=17)
    pol = pkg.Policy(n, L, seed=1, variant="classic")
    assert pol.param_count == params.size == 939026
    pol.set_params(params)
    rng = np.random.default_rng(n)
    rec_h = synth_classic_records_host(n, 11, 2)
    state_h = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < term_p).astype(np.float32)
    ref = ob.classic_forward_f64(params, L, ob.classic_expand(rec_h), state_h, term_h)
    state = _t(state_h, cuda)
    h_enc = torch.zeros(n, HIDDEN, device=cuda); h3 = torch.zeros(n, HIDDEN, device=cuda)
    av = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state, h_enc=h_enc, h3=h3)
    torch.cuda.synchronize()
    assert av.shape == (n, 18)
    assert_close(h_enc.cpu().numpy(), ref["h_enc"], TOL_FP32, "classic h_enc")
    assert_close(h3.cpu().numpy(), ref["h3"], TOL_FP32, "classic h3")
    assert_close(state.cpu().numpy(), ref["state"], TOL_FP32, "classic state")
    assert_close(av.cpu().numpy()[:, :17], ref["logits"], TOL_FP32, "classic logits")
    assert_close(av.cpu().numpy()[:, 17], ref["values"], TOL_FP32, "classic values")
    # encode_step alone (encode_obs_kernel) gives the same h_enc
    he = pol.encode_step(_t(rec_h, cuda))
    torch.cuda.synchronize()
    assert torch.equal(he, h_enc)
    pol.close()


def test_classic_full_size_properties(pkg, cuda):
    """Config 5: 1 048 576 envs, one step.  Sampled tiles run alone reproduce their
    rows bit for bit and match the oracle; chunked == unchunked."""
    import torch
    n = 1 << 20
    pol = pkg.Policy(n, L, seed=1, variant="classic")
    params = pol.get_params()
    rec = pkg.policy.synth_classic_records(n, 13, 0)
    term = torch.zeros(n, device=cuda)
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    st_a = st0.clone()
    av_a = pol.forward(rec, term, st_a).clone()
    st_b = st0.clone()
    av_b = pol.forward(rec, term, st_b, chunk=65536)
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_b) and torch.equal(st_a, st_b) and torch.isfinite(av_a).all()
    tiles = [0, 1, 16383, 32767, 20000]
    idx = torch.cat([torch.arange(t * 32, t * 32 + 32) for t in tiles]).to(cuda)
    small = pkg.Policy(len(idx), L, seed=1, variant="classic")
    sub_st = st0[:, idx].contiguous()
    av_s = small.forward(rec[idx].contiguous(), term[idx].contiguous(), sub_st)
    torch.cuda.synchronize()
    assert torch.equal(av_s, av_a[idx]) and torch.equal(sub_st, st_a[:, idx])
    ref = ob.classic_forward_f64(params, L, ob.classic_expand(rec[idx].cpu().numpy()),
                                 st0[:, idx].cpu().numpy(), None)
    assert_close(av_s.cpu().numpy()[:, :17], ref["logits"], TOL_FP32, "classic sample logits")
    assert_close(sub_st.cpu().numpy(), ref["state"], TOL_FP32, "classic sample state")
    small.close(); pol.close()
