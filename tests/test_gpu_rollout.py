"""GPU tests of the rollout-side entry points through the C ABI: categorical
sampling (cfp_value_sample), reward/done recording (cfp_record_rd), the policy
half of a rollout step (cfp_rollout_step) and the bootstrap value
(cfp_train_bootstrap).

The uniform behind each draw is computed directly from Philox4x32-10 with curand_init's
(seed, subsequence, offset) mapping; the CPU oracle's version of it is held to rocRAND's
engine in tests/test_oracle_policy.py, and the device's to the oracle's here.  Given
the uniform, actions and log-probabilities follow cf_nn_sample_action
(craftax_full.cu:9147-9165) and are checked against its C restatement.  Actions
must agree except where u*total lies within 1e-6 (relative) of a cumulative-sum
boundary, where a one-ulp difference between device and host expf may tip the
comparison; log-probabilities within 1e-5 absolute."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import ACTIONS, HIDDEN, random_params, synth_records_host

pytestmark = pytest.mark.gpu
L = 3
SALT = 0xA5A5A5A5A5A5A5A5


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def _uniforms(seed, step, n):
    return ob.philox_uniforms(int(seed) ^ SALT, range(n), step)


def _check_draws(av_h, act, lp, val, seed, step):
    n = av_h.shape[0]
    A = av_h.shape[1] - 1
    u = _uniforms(seed, step, n)
    ref_act, ref_lp, margin = ob.sample_actions(av_h[:, :A], u)
    bad = act != ref_act
    assert np.all(margin[bad] < 1e-6), f"{bad.sum()} draws differ away from a boundary"
    assert bad.mean() < 1e-3
    ok = ~bad
    assert np.max(np.abs(lp[ok] - ref_lp[ok])) < 1e-5
    assert np.array_equal(val, av_h[:, A])


@pytest.mark.parametrize("n,A,scale", [(4096, 43, 1.0), (1000, 43, 6.0), (2048, 17, 2.0),
                                       (16384 + 37, 43, 3.0), (20000, 17, 2.0)])
def test_value_sample_matches_restatement(pkg, cuda, n, A, scale):
    import torch
    rng = np.random.default_rng(n + A)
    av_h = (scale * rng.standard_normal((n, A + 1))).astype(np.float32)
    ctr = torch.tensor([7], dtype=torch.int64, device=cuda)
    env_act = torch.zeros(n, device=cuda)
    act, lp, val = pkg.policy.value_sample(_t(av_h, cuda), 1234, step_ctr=ctr, env_actions=env_act)
    torch.cuda.synchronize()
    act_h = act.cpu().numpy()
    _check_draws(av_h, act_h, lp.cpu().numpy(), val.cpu().numpy(), 1234, 7)
    assert np.array_equal(env_act.cpu().numpy(), act_h.astype(np.float32))
    # same inputs -> same draws; another step -> other draws; no counter -> step 0
    act2, _, _ = pkg.policy.value_sample(_t(av_h, cuda), 1234, step_ctr=ctr)
    ctr.fill_(8)
    act3, _, _ = pkg.policy.value_sample(_t(av_h, cuda), 1234, step_ctr=ctr)
    act0, lp0, val0 = pkg.policy.value_sample(_t(av_h, cuda), 1234)
    torch.cuda.synchronize()
    assert torch.equal(act, act2) and not torch.equal(act, act3)
    _check_draws(av_h, act0.cpu().numpy(), lp0.cpu().numpy(), val0.cpu().numpy(), 1234, 0)


def test_value_sample_both_kernels_agree(pkg, cuda):
    """Batches below 16 384 envs run sixteen lanes per env, larger ones one thread per env;
    both do the order-dependent sums in ascending order, so env e of a large launch draws
    what env e of a small launch over the same rows draws, bit for bit."""
    import torch
    for A in (43, 17):
        n = 16384 + 517
        av = _t((2.5 * np.random.default_rng(A).standard_normal((n, A + 1))).astype(np.float32), cuda)
        ctr = torch.tensor([11], dtype=torch.int64, device=cuda)
        act_l, lp_l, val_l = pkg.policy.value_sample(av, 77, step_ctr=ctr)
        act_s, lp_s, val_s = pkg.policy.value_sample(av[:4096].contiguous(), 77, step_ctr=ctr)
        torch.cuda.synchronize()
        assert torch.equal(act_l[:4096], act_s) and torch.equal(lp_l[:4096], lp_s)
        assert torch.equal(val_l[:4096], val_s)


def test_value_sample_distribution(pkg, cuda):
    """One logit vector replicated over 2^20 envs: empirical action frequencies
    match softmax within five binomial standard deviations (pins that the
    uniforms are uniform and the inversion unbiased)."""
    import torch
    n, A = 1 << 20, 43
    rng = np.random.default_rng(3)
    logits = (1.5 * rng.standard_normal(A)).astype(np.float32)
    av = torch.empty(n, A + 1, device=cuda)
    av[:, :A] = _t(logits, cuda)
    av[:, A] = 0.25
    act, lp, val = pkg.policy.value_sample(av, 99)
    torch.cuda.synchronize()
    p = np.exp(logits.astype(np.float64) - logits.max())
    p /= p.sum()
    freq = np.bincount(act.cpu().numpy(), minlength=A) / n
    sd = np.sqrt(p * (1 - p) / n)
    assert np.all(np.abs(freq - p) < 5 * sd + 1e-9)
    assert torch.all(val == 0.25)


def test_record_rd(pkg, cuda):
    import torch
    n = 1000
    rng = np.random.default_rng(1)
    rew = rng.standard_normal(n).astype(np.float32)
    term = (rng.random(n) < 0.3).astype(np.float32) * rng.choice([1.0, 2.0], n).astype(np.float32)
    r_rew = torch.full((n,), -7.0, device=cuda)
    r_done = torch.full((n,), 9, dtype=torch.uint8, device=cuda)
    pkg.policy.record_rd(_t(rew, cuda), _t(term, cuda), r_rew, r_done)
    torch.cuda.synchronize()
    assert np.array_equal(r_rew.cpu().numpy(), rew)
    assert np.array_equal(r_done.cpu().numpy(), (term != 0).astype(np.uint8))


@pytest.mark.parametrize("n,small", [(256, False), (8192, False), (256, True), (4096, True),
                                     (8224, False), (16416, False)])
def test_rollout_step_and_bootstrap(pkg, cuda, n, small):
    """cfp_rollout_step == forward on the live state + sampling with the device step
    counter, written into the slab rows; cfp_train_bootstrap values the next
    records on a copy of the live state.  The cases cover the four forms of the step:
    one launch on 32-env tiles, one per workgroup, that also draws and bumps (256 and
    8192 envs: at most one tile per CU), the same on 16-env tiles (small), forward +
    sampler that bumps the counter in its own launch (8224 envs = 257 tiles), forward +
    row sampler + bump kernel (16 416)."""
    import torch
    T, seed = 4, 4321
    params = random_params(L, 21, scale=0.5)
    pol = pkg.Policy(n, L, seed=1)
    pol.set_params(params)
    twin = pkg.Policy(n, L, seed=1)      # same weights, driven by hand
    twin.set_params(params)
    pol.set_small_tiles(small)
    twin.set_small_tiles(small)
    tr = pkg.Trainer(pol, T)
    rng = np.random.default_rng(22)
    pol.state.zero_()
    twin_state = torch.zeros(L, n, HIDDEN, device=cuda)
    env_act = torch.zeros(n, device=cuda)
    for t in range(T):
        rec = _t(synth_records_host(n, 5, t), cuda)
        term = _t((rng.random(n) < 0.2).astype(np.float32) if t else np.zeros(n, np.float32), cuda)
        r_state_ref = torch.zeros(L, n, HIDDEN, device=cuda)
        av = twin.forward(rec, term, twin_state, r_state_t=r_state_ref).clone()
        tr.rollout_step(t, rec, term, seed, env_actions=env_act)
        torch.cuda.synchronize()
        assert int(tr.buf("step_ctr").cpu()[0]) == t + 1
        assert torch.equal(pol.state, twin_state)
        assert torch.equal(tr.buf("r_state")[t], r_state_ref)
        assert torch.equal(tr.buf("r_obs")[t], rec)
        act = tr.buf("r_act")[t].cpu().numpy()
        _check_draws(av.cpu().numpy(), act, tr.buf("r_logprob")[t].cpu().numpy(),
                     tr.buf("r_value")[t].cpu().numpy(), seed, t)
        assert np.array_equal(env_act.cpu().numpy(), act.astype(np.float32))
    # bootstrap: value of the next records, live state untouched
    rec = _t(synth_records_host(n, 5, T), cuda)
    term = _t((rng.random(n) < 0.2).astype(np.float32), cuda)
    live_before = pol.state.clone()
    tr.bootstrap(rec, term)
    st_copy = twin_state.clone()
    av = twin.forward(rec, term, st_copy)
    torch.cuda.synchronize()
    assert torch.equal(pol.state, live_before)
    assert torch.equal(tr.buf("v_boot"), av[:, ACTIONS])
    tr.close(); pol.close(); twin.close()


@pytest.mark.parametrize("classic", [False, True])
def test_reference_weight_init(pkg, cuda, classic):
    """cfp_policy_init_reference: segment s, element i = (2u - 1) * bound with u the
    Philox uniform of (seed, subsequence s, offset i) -- checked against the oracle's
    restatement at the segment boundaries and on a random sample, plus the bounds
    and the uniform's moments per segment; the forward then runs on these weights."""
    import torch
    n = 64
    pol = pkg.Policy(n, L, seed=1, variant="classic" if classic else "full")
    before = pol.get_params()
    pol.init_reference(1234)
    w = pol.get_params()
    assert not np.array_equal(w, before)
    obs, actions = (1345, 17) if classic else (843, 43)
    be, bh = np.float32(1.0) / np.sqrt(np.float32(obs)), np.float32(1.0) / np.sqrt(np.float32(256))
    counts = [obs * 256, 256, L * 768 * 256, actions * 256, actions, 256, 1]
    bounds = [be, be, bh, bh, bh, bh, bh]
    assert sum(counts) == w.size
    rng = np.random.default_rng(3)
    off = 0
    lib = ob.cfo()
    for s, (cnt, b) in enumerate(zip(counts, bounds)):
        seg = w[off:off + cnt]
        assert np.all(np.abs(seg) <= b)
        idx = np.unique(np.concatenate([[0, cnt - 1], rng.integers(0, cnt, 64)]))
        for i in idx:
            u = np.float32(lib.cfo_philox_uniform(1234, s, int(i)))
            assert seg[i] == (np.float32(2.0) * u - np.float32(1.0)) * np.float32(b), (s, i)
        if cnt >= 4096:
            assert abs(seg.mean()) < 0.05 * b and abs(seg.var() / (b * b / 3.0) - 1.0) < 0.05
        off += cnt
    rec = (pkg.policy.synth_classic_records(n, 3, 0) if classic else pkg.policy.synth_records(n, 3, 0))
    av = pol.forward(rec, torch.zeros(n, device=cuda), pol.state)
    torch.cuda.synchronize()
    assert torch.isfinite(av).all()
    pol.close()


@pytest.mark.parametrize("n,small", [(256, False), (512, True)])
def test_rollout_round_replays_from_a_graph(pkg, cuda, n, small):
    """A round of rollout steps captured once and replayed (the reference captures its
    rollout the same way): the step counter lives in device memory and is bumped inside
    the launch that draws, so every replay must continue the eager twin's stream of
    draws -- same actions, log-probabilities, values, state and counter after each
    replay, with eager work and synchronisations in between."""
    import torch
    T, seed = 3, 99
    params = random_params(L, 31, scale=0.5)
    twins = []
    for _ in range(2):
        pol = pkg.Policy(n, L, seed=1)
        pol.set_params(params)
        pol.set_small_tiles(small)
        pol.state.zero_()
        twins.append((pol, pkg.Trainer(pol, T)))
    (pol_e, tr_e), (pol_g, tr_g) = twins
    recs = [_t(synth_records_host(n, 7, t), cuda) for t in range(T)]
    term = _t((np.random.default_rng(3).random(n) < 0.2).astype(np.float32), cuda)
    acts = [torch.zeros(n, device=cuda) for _ in range(2)]

    def round_(tr, a):
        for t in range(T):
            tr.rollout_step(t, recs[t], term, seed, env_actions=a)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            round_(tr_g, acts[1])
    torch.cuda.synchronize()
    for i in range(3):
        round_(tr_e, acts[0])
        with torch.cuda.stream(side):
            graph.replay()
        torch.cuda.synchronize()
        junk = torch.randn(1 << 16, device=cuda).sum().item()   # eager work between replays
        assert np.isfinite(junk)
        assert int(tr_g.buf("step_ctr").cpu()[0]) == (i + 1) * T == int(tr_e.buf("step_ctr").cpu()[0])
        for name in ("r_act", "r_logprob", "r_value", "r_state"):
            assert torch.equal(tr_e.buf(name), tr_g.buf(name)), f"replay {i}: {name}"
        assert torch.equal(pol_e.state, pol_g.state) and torch.equal(acts[0], acts[1])
    # successive rounds drew from different offsets of the stream
    first = tr_e.buf("r_act").clone()
    round_(tr_e, acts[0]); torch.cuda.synchronize()
    assert not torch.equal(first, tr_e.buf("r_act"))
    for pol, tr in twins:
        tr.close(); pol.close()
