"""GPU parity of the PPO update (cfp_train_*) against the fp64 oracle
(oracle/policy_bwd_ref.c), which is itself pinned by finite differences.

Tolerance: gradients, losses, advantages within 1e-4 relative (parity_util.rel_err,
per parameter segment) of the fp64 evaluation of the same fp32 inputs."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import (ACTIONS, GRU, HIDDEN, OBS, TOL_FP32, assert_close, random_params,
                         rel_err, synth_records_host)

pytestmark = pytest.mark.gpu
L = 3


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def _segments(layers):
    sizes = [("W_enc", OBS * HIDDEN), ("b_enc", HIDDEN), ("W_gru", layers * GRU * HIDDEN),
             ("W_a", ACTIONS * HIDDEN), ("b_a", ACTIONS), ("W_v", HIDDEN), ("b_v", 1)]
    off = 0
    for name, cnt in sizes:
        yield name, slice(off, off + cnt)
        off += cnt


def _collect(pkg, cuda, n, T, seed, done_p, scale=0.3, layers=L, **cfg):
    """Synthetic rollout: records from the counter generator, r_state written by the
    device's own forward (zero initial state, zeroed after a done), the rest of
    the slabs random."""
    import torch
    params = random_params(layers, seed, scale=scale)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    tr = pkg.Trainer(pol, T, **cfg)
    rng = np.random.default_rng(seed + 1)
    r_done = (rng.random((T, n)) < done_p).astype(np.uint8)
    pol.state.zero_()
    for t in range(T):
        rec = _t(synth_records_host(n, seed, t), cuda)
        term = _t(r_done[t - 1].astype(np.float32) if t else np.zeros(n, np.float32), cuda)
        tr.record_step(t, rec, term)
    host = dict(
        r_act=rng.integers(0, ACTIONS, (T, n)).astype(np.int32),
        r_logprob=(-np.log(ACTIONS) + 0.1 * rng.standard_normal((T, n))).astype(np.float32),
        adv=rng.standard_normal((T, n)).astype(np.float32),
        ret=rng.standard_normal((T, n)).astype(np.float32), r_done=r_done)
    for k, v in host.items():
        tr.buf(k).copy_(_t(v, cuda))
    tr.adv_stats()
    torch.cuda.synchronize()
    host["r_obs"] = tr.buf("r_obs").cpu().numpy()
    host["r_state"] = tr.buf("r_state").cpu().numpy()
    return params, pol, tr, host


KINK_MARGIN = 5e-7


def _collect_off_the_kink(pkg, cuda, n, T, seed, done_p, layers=L, **cfg):
    """_collect on `seed`, moved on to seed + 1000, + 2000 ... while some gate pre-activation
    zh of the batch lies within KINK_MARGIN of zero.  The candidate function's derivative
    jumps from 1/4 to 1 at zh = 0 (craftax_full.cu:9357), so the gradient of such a batch is
    discontinuous there and an fp32 evaluation may land on either side (seed 153 of the
    eight consecutive ones below has a zh of 6e-8: one unit's row of dW_gru then differs by
    1e-2 from the fp64 value in every GEMM mode alike).  The margin is a few fp32 roundings
    of a zh (mean |zh| is 0.4 to 0.8 over 4e5 values a batch, so one batch in four has a
    value inside it); both the exact and the bf16-operand zh are looked at.  The criterion
    looks at the batch, not at any result."""
    for k in range(16):
        params, pol, tr, host = _collect(pkg, cuda, n, T, seed + 1000 * k, done_p, layers=layers, **cfg)
        batch, keep = ob.make_batch(T, n, 0, n, layers, T, **host)
        margin = min(ob.ppo_min_abs_zh(params, batch), ob.ppo_min_abs_zh(params, batch, bf16_ops=True))
        if margin >= KINK_MARGIN:
            return params, pol, tr, host, seed + 1000 * k
        print(f"seed {seed + 1000 * k}: min |zh| = {margin:.1e}, a batch on the kink; moving on")
        tr.close(); pol.close()
    raise AssertionError("no batch off the kink")


@pytest.mark.parametrize("n,T,minibatches,bptt_split,bwd_win,done_p",
                         [(64, 8, 1, 1, 0, 0.1), (64, 8, 2, 2, 3, 0.15), (32, 6, 1, 3, 1, 0.0),
                          # window lengths 7, 4 and 5: every remainder of the reverse sweep's
                          # three-step rounds after at least one full round
                          (32, 7, 1, 1, 0, 0.2), (32, 8, 1, 2, 4, 0.1), (32, 5, 1, 1, 0, 0.1)])
def test_backward_matches_oracle(pkg, cuda, n, T, minibatches, bptt_split, bwd_win, done_p):
    import torch
    params, pol, tr, host = _collect(pkg, cuda, n, T, 50 + n + T, done_p,
                                     minibatches=minibatches, bptt_split=bptt_split,
                                     bwd_win=bwd_win)
    mb = n // minibatches
    stats = tr.buf("stats").cpu().numpy()
    a64 = host["adv"].astype(np.float64)
    assert np.allclose(stats, [a64.sum(), (a64 * a64).sum()], rtol=1e-12)
    for m in range(minibatches):
        tr.buf("grads").zero_()
        tr.zero_loss()
        tr.backward(m * mb, mb)
        torch.cuda.synchronize()
        g = tr.buf("grads").cpu().numpy()
        l3 = tr.buf("loss_acc").cpu().numpy()
        batch, keep = ob.make_batch(T, n, m * mb, mb, L, T // bptt_split, **host)
        g_ref, l3_ref = ob.ppo_backward_f64(params, batch)
        for name, sl in _segments(L):
            assert_close(g[sl], g_ref[sl], TOL_FP32, f"minibatch {m} d{name}")
        assert np.allclose(l3, l3_ref, rtol=1e-4), (l3, l3_ref)
    tr.close(); pol.close()


def test_backward_matches_oracle_at_a_mid_size(pkg, cuda):
    """The largest batch the fp64 oracle is asked for: 256 envs x 8 steps (2048 samples,
    truncation after 4 steps, two windows of 1024 columns), four times the cases above and on
    the way to the 4096 x 64 shape that is held by properties only: 256 envs fill a workgroup
    of the dh GEMM and sixteen of the head kernel's.  The batch is taken off the candidate
    function's kink like the bf16 ones: with 1.6 million gate pre-activations a batch has a
    value within the margin of zero more often than not (at 8192 samples every batch has, and
    a comparison with one fp64 evaluation stops being well-posed: an attempt at 512 x 16
    differed by 7e-4 in the one row of dW_gru a flipped derivative reaches)."""
    import torch
    n, T = 256, 8
    params, pol, tr, host, seed = _collect_off_the_kink(pkg, cuda, n, T, 4321, 0.08, L,
                                                        bptt_split=2, bwd_win=4)
    print(f"batch of seed {seed}")
    tr.buf("grads").zero_()
    tr.zero_loss()
    tr.backward(0, n)
    torch.cuda.synchronize()
    g = tr.buf("grads").cpu().numpy()
    l3 = tr.buf("loss_acc").cpu().numpy()
    batch, keep = ob.make_batch(T, n, 0, n, L, T // 2, **host)
    g_ref, l3_ref = ob.ppo_backward_f64(params, batch)
    for name, sl in _segments(L):
        assert_close(g[sl], g_ref[sl], TOL_FP32, f"d{name}")
    assert np.allclose(l3, l3_ref, rtol=1e-4), (l3, l3_ref)
    tr.close(); pol.close()


@pytest.mark.parametrize("layers", [1, 2])
def test_backward_matches_oracle_with_fewer_layers(pkg, cuda, layers):
    """Which of the trainer's two streams runs the dependent chain, the heads' own
    gradients, dW_enc and its last rows depends on the parity of the layer count, and
    they share split workspaces and column-sum scratch across those streams: one- and
    two-layer policies, two windows (4 + 2 steps), against the fp64 oracle, and twice for
    the same bits."""
    import torch
    n, T = 64, 6
    params, pol, tr, host = _collect(pkg, cuda, n, T, 300 + layers, 0.1, layers=layers, bwd_win=4)
    batch, keep = ob.make_batch(T, n, 0, n, layers, T, **host)
    g_ref, l3_ref = ob.ppo_backward_f64(params, batch)
    outs = []
    for _ in range(2):
        tr.buf("grads").zero_(); tr.zero_loss()
        tr.backward(0, n)
        torch.cuda.synchronize()
        outs.append(tr.buf("grads").cpu().numpy().copy())
    assert np.array_equal(outs[0], outs[1])
    for name, sl in _segments(layers):
        assert_close(outs[0][sl], g_ref[sl], TOL_FP32, f"{layers} layers d{name}")
    assert np.allclose(tr.buf("loss_acc").cpu().numpy(), l3_ref, rtol=1e-4)
    tr.close(); pol.close()


def test_backward_is_bitwise_reproducible_and_stale_state_semantics(pkg, cuda):
    """Fixed-order reductions: two passes give identical bits.  The recompute
    uses the STORED state at every step even when it is not what the live
    recurrence would give (stale states after an Adam step): perturb r_state and
    compare with the oracle, which follows the same rule."""
    import torch
    n, T = 32, 5
    params, pol, tr, host = _collect(pkg, cuda, n, T, 77, 0.1)
    rs = host["r_state"] + 0.05 * np.random.default_rng(5).standard_normal(host["r_state"].shape).astype(np.float32)
    tr.buf("r_state").copy_(_t(rs, cuda))
    host["r_state"] = rs
    outs = []
    for _ in range(2):
        tr.buf("grads").zero_()
        tr.backward(0, n)
        torch.cuda.synchronize()
        outs.append(tr.buf("grads").cpu().numpy().copy())
    assert np.array_equal(outs[0], outs[1])
    batch, keep = ob.make_batch(T, n, 0, n, L, T, **host)
    g_ref, _ = ob.ppo_backward_f64(params, batch)
    for name, sl in _segments(L):
        assert_close(outs[0][sl], g_ref[sl], TOL_FP32, f"stale-state d{name}")
    tr.close(); pol.close()


def test_loss_matches_oracle_and_gradcheck_gate(pkg, cuda):
    """cfp_train_loss vs the oracle's live-recurrence loss, then the reference's
    gradcheck gate (craftax_full.cu:13854-13907): central differences of the
    device loss on the largest-|g| parameters; fail if diff > 2e-4 and rel > 3e-2."""
    import torch
    n, T = 32, 6
    params, pol, tr, host = _collect(pkg, cuda, n, T, 91, 0.1, bptt_split=2)
    batch, keep = ob.make_batch(T, n, 0, n, L, T // 2, **host)
    want, l3_ref = ob.ppo_loss_f64(params, batch)
    got = tr.loss()
    assert np.allclose(got[:3], l3_ref, rtol=1e-4), (got, l3_ref)
    assert abs(got[3] - want) <= 1e-4 * abs(want)
    tr.buf("grads").zero_()
    tr.backward(0, n)
    torch.cuda.synchronize()
    g = tr.buf("grads").cpu().numpy().copy()
    for i in np.argsort(-np.abs(g))[:4]:
        eps = 1e-3
        pp = params.copy(); pp[i] += eps
        pm = params.copy(); pm[i] -= eps
        pol.set_params(pp); lp = tr.loss()[3]
        pol.set_params(pm); lm = tr.loss()[3]
        fd = (lp - lm) / (float(pp[i]) - float(pm[i]))
        diff = abs(fd - g[i]); rel = diff / max(abs(fd), abs(g[i]), 1e-12)
        assert not (diff > 2e-4 and rel > 3e-2), (int(i), fd, float(g[i]))
    tr.close(); pol.close()


def test_gae_and_adam_match_oracle(pkg, cuda):
    import torch
    n, T = 64, 12
    pol = pkg.Policy(n, L, seed=3)
    tr = pkg.Trainer(pol, T)
    rng = np.random.default_rng(4)
    vals = rng.standard_normal((T, n)).astype(np.float32)
    rew = rng.standard_normal((T, n)).astype(np.float32)
    done = (rng.random((T, n)) < 0.1).astype(np.uint8)
    vboot = rng.standard_normal(n).astype(np.float32)
    for k, v in (("r_value", vals), ("r_reward", rew), ("r_done", done), ("v_boot", vboot)):
        tr.buf(k).copy_(_t(v, cuda))
    tr.gae()
    torch.cuda.synchronize()
    adv = np.zeros((T, n)); ret = np.zeros((T, n))
    ob.cfo().cfo_gae_f64(vals.ctypes.data, rew.ctypes.data, done.ctypes.data, vboot.ctypes.data,
                         adv.ctypes.data, ret.ctypes.data, n, T, 0.99, 0.95)
    adv_d = tr.buf("adv").cpu().numpy()
    assert_close(adv_d, adv, TOL_FP32, "gae adv")
    assert_close(tr.buf("ret").cpu().numpy(), ret, TOL_FP32, "gae ret")
    a64 = adv_d.astype(np.float64)
    assert np.allclose(tr.buf("stats").cpu().numpy(), [a64.sum(), (a64 * a64).sum()], rtol=1e-12)
    # three Adam steps with known gradients
    p64 = pol.get_params().astype(np.float64)
    m = np.zeros_like(p64); v = np.zeros_like(p64)
    for step in range(1, 4):
        g = (rng.standard_normal(p64.size) * 10.0 ** rng.integers(-4, 1, p64.size)).astype(np.float32)
        tr.buf("grads").copy_(_t(g, cuda))
        tr.adam()
        g64 = g.astype(np.float64)
        ob.cfo().cfo_adam_f64(p64.ctypes.data, g64.ctypes.data, m.ctypes.data, v.ctypes.data,
                              p64.size, step, 3e-4, 0.9, 0.999, 1e-8)
        torch.cuda.synchronize()
        assert not tr.buf("grads").any()                      # Adam zeroes the arena
    got = pol.get_params().astype(np.float64)
    assert np.max(np.abs(got - p64)) < 2e-6, np.max(np.abs(got - p64))
    tr.close(); pol.close()


def test_trainer_argument_checks(pkg, cuda):
    pol = pkg.Policy(64, L, seed=3)
    with pytest.raises(pkg._lib.CfpError, match="minibatches must divide"):
        pkg.Trainer(pol, 8, minibatches=3)
    with pytest.raises(pkg._lib.CfpError, match="bptt_split must divide"):
        pkg.Trainer(pol, 8, bptt_split=3)
    with pytest.raises(pkg._lib.CfpError, match="multiple of 32"):
        pkg.Trainer(pol, 8, minibatches=4)                    # 16 envs per minibatch
    pol.close()


def test_config4_shape_properties(pkg, cuda):
    """The PPO-update config at full size (4096 envs x 64 steps = 262 144 samples):
    too large for the oracle, so size-independent properties: the update is
    linear over envs (full-batch gradient = mean of the two half-batch
    gradients, each normalised by its own size), finite and reproducible, also while
    other work competes for the memory system."""
    import torch
    n, T = 4096, 64
    pol = pkg.Policy(n, L, seed=1)
    tr = pkg.Trainer(pol, T)
    assert tr.window * tr.mb == 262144
    term0 = torch.zeros(n, device=cuda)
    for t in range(T):
        tr.record_step(t, pkg.policy.synth_records(n, 5, t), term0)
    g = torch.Generator(device="cpu").manual_seed(1)
    tr.buf("r_act").copy_(torch.randint(0, ACTIONS, (T, n), generator=g, dtype=torch.int32).to(cuda))
    tr.buf("r_logprob").fill_(float(-np.log(ACTIONS)))
    tr.buf("adv").copy_(torch.randn(T, n, generator=g).to(cuda))
    tr.buf("ret").copy_(torch.randn(T, n, generator=g).to(cuda))
    tr.adv_stats()
    tr.buf("grads").zero_(); tr.backward(0, n); torch.cuda.synchronize()
    g_full = tr.buf("grads").clone()
    assert torch.isfinite(g_full).all()
    # the reverse sweep waits for its own loads with counted s_waitcnt: the same backward
    # racing a long run of device copies on another stream must give the same bits
    side = torch.cuda.Stream()
    big = torch.empty(1 << 28, dtype=torch.uint8, device=cuda)
    tr.buf("grads").zero_(); torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(150):
            big[: 1 << 27].copy_(big[1 << 27:])
    tr.backward(0, n); torch.cuda.synchronize()
    assert torch.equal(tr.buf("grads"), g_full), "backward depends on timing"
    del big
    tr.buf("grads").zero_(); tr.backward(0, n // 2); tr.backward(n // 2, n // 2)
    torch.cuda.synchronize()
    g_halves = tr.buf("grads").clone() * 0.5
    for name, sl in _segments(L):
        assert_close(g_halves[sl].cpu().numpy(), g_full[sl].cpu().numpy(), TOL_FP32,
                     f"linearity d{name}")
    tr.close(); pol.close()


def test_config4_shape_bf16_storage_properties(pkg, cuda):
    """bf16 GEMM inputs with bf16 storage of the window workspace at the full size of the
    PPO-update config (4096 envs x 64 steps, one 262 144-column window): finite, the same
    bits twice, and every gradient segment within the bf16 tolerance (relative Frobenius
    norm) of the same update with fp32 storage."""
    import torch
    from parity_util import TOL_BF16, fro_err
    n, T = 4096, 64
    pol = pkg.Policy(n, L, seed=1)
    tr = pkg.Trainer(pol, T)
    term0 = torch.zeros(n, device=cuda)
    for t in range(T):
        tr.record_step(t, pkg.policy.synth_records(n, 5, t), term0)
    g = torch.Generator(device="cpu").manual_seed(1)
    tr.buf("r_act").copy_(torch.randint(0, ACTIONS, (T, n), generator=g, dtype=torch.int32).to(cuda))
    tr.buf("r_logprob").fill_(float(-np.log(ACTIONS)))
    tr.buf("adv").copy_(torch.randn(T, n, generator=g).to(cuda))
    tr.buf("ret").copy_(torch.randn(T, n, generator=g).to(cuda))
    tr.adv_stats()
    pkg.policy.set_gemm_bf16(True)
    try:
        grads = {}
        for store16 in (False, True):
            tr.set_bf16_storage(store16)
            runs = []
            for _ in range(2):
                tr.buf("grads").zero_(); tr.backward(0, n); torch.cuda.synchronize()
                runs.append(tr.buf("grads").clone())
            assert torch.isfinite(runs[0]).all()
            assert torch.equal(runs[0], runs[1]), f"bf16 storage {store16}: not reproducible"
            grads[store16] = runs[0].cpu().numpy()
        for name, sl in _segments(L):
            e = fro_err(grads[True][sl], grads[False][sl])
            assert e <= TOL_BF16, f"d{name}: bf16 vs fp32 storage, relative Frobenius error {e:.3e}"
    finally:
        tr.set_bf16_storage(False)
        pkg.policy.set_gemm_bf16(False)
    tr.close(); pol.close()


def test_update_iteration_replays_from_a_graph(pkg, cuda):
    """backward + Adam captured once (after the lazily allocated GEMM workspaces
    exist) and replayed: every replay, with eager work and synchronisations in
    between, must leave the same parameters as the same number of eager updates
    on an identical twin (the step counter and lr live in device memory)."""
    import torch
    n, T = 64, 6
    twins = [_collect(pkg, cuda, n, T, 123, 0.1) for _ in range(2)]
    (_, pol_e, tr_e, _), (_, pol_g, tr_g, _) = twins

    def update(tr):
        tr.zero_loss()
        tr.backward(0, n)
        tr.adam()

    update(tr_e)                      # warm-up: allocates the split-K / gemv workspaces
    update(tr_g)
    torch.cuda.synchronize()
    assert torch.equal(pol_e.params, pol_g.params)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        update(tr_g)
    for i in range(3):
        update(tr_e)
        graph.replay()
        torch.cuda.synchronize()
        junk = torch.randn(1 << 16, device=cuda).sum().item()   # eager work between replays
        assert np.isfinite(junk)
        assert torch.equal(pol_e.params, pol_g.params), f"replay {i}"
        assert torch.equal(tr_e.buf("adam_v"), tr_g.buf("adam_v"))
    # the forward weights follow the replayed updates (mirrors refreshed inside the graph)
    rec = _t(synth_records_host(n, 9, 0), cuda)
    term = torch.zeros(n, device=cuda)
    sa = torch.zeros(L, n, HIDDEN, device=cuda); sb = torch.zeros(L, n, HIDDEN, device=cuda)
    assert torch.equal(pol_e.forward(rec, term, sa), pol_g.forward(rec, term, sb))
    for _, pol, tr, _ in twins:
        tr.close(); pol.close()


@pytest.mark.parametrize("on_side_stream", [False, True])
def test_train_update_eager_and_graph_match_the_manual_loop(pkg, cuda, on_side_stream):
    """cfp_train_update (the reference's cu_train_update without its collect): two
    epochs of two minibatches, (a) eager and (b) captured by the library and replayed,
    against (c) the same loop written out with backward / adam calls on identical
    triplets.  Parameters, Adam moments and the last epoch's loss sums must agree bit
    for bit after every iteration; between iterations lr is annealed through its
    device scalar and eager work runs, so a replay that baked in a value or read
    stale memory would differ."""
    import torch
    n, T = 64, 6
    cfg = dict(epochs=2, minibatches=2)
    trip = [_collect(pkg, cuda, n, T, 321, 0.1, **cfg) for _ in range(3)]
    (_, pol_m, tr_m, _), (_, pol_e, tr_e, _), (_, pol_g, tr_g, _) = trip
    mb = n // 2
    assert tr_m.mb == mb
    stream = torch.cuda.Stream() if on_side_stream else torch.cuda.current_stream()
    with torch.cuda.stream(stream):
        for it in range(3):
            for tr in (tr_m, tr_e, tr_g):
                tr.buf("lr").fill_(3e-4 * (1.0 - 0.25 * it))
            for _ in range(cfg["epochs"]):
                tr_m.zero_loss()
                for m in range(cfg["minibatches"]):
                    tr_m.backward(m * mb, mb)
                    tr_m.adam()
            tr_e.update(use_graph=False)
            tr_g.update(use_graph=True)
            torch.cuda.synchronize()
            junk = torch.randn(1 << 16, device=cuda).sum().item()   # eager work between replays
            assert np.isfinite(junk)
            for name, pol, tr in (("eager", pol_e, tr_e), ("graph", pol_g, tr_g)):
                assert torch.equal(pol.params, pol_m.params), f"{name} params, iteration {it}"
                assert torch.equal(tr.buf("adam_m"), tr_m.buf("adam_m")), f"{name} adam_m {it}"
                assert torch.equal(tr.buf("adam_v"), tr_m.buf("adam_v")), f"{name} adam_v {it}"
                assert torch.equal(tr.buf("loss_acc"), tr_m.buf("loss_acc")), f"{name} loss {it}"
                assert not tr.buf("grads").any(), f"{name}: Adam leaves the grads arena zero"
        assert not torch.equal(pol_m.params, _t(trip[0][0], cuda))     # the updates moved them
        # a change of the GEMM mode makes the next graph call capture again
        pkg.policy.set_gemm_split(0)
        try:
            for _ in range(cfg["epochs"]):
                tr_m.zero_loss()
                for m in range(cfg["minibatches"]):
                    tr_m.backward(m * mb, mb)
                    tr_m.adam()
            tr_g.update(use_graph=True)
            torch.cuda.synchronize()
            assert torch.equal(pol_g.params, pol_m.params), "re-captured under the new GEMM mode"
        finally:
            pkg.policy.set_gemm_split(1)
    for _, pol, tr, _ in trip:
        tr.close(); pol.close()


def test_two_trainers_with_their_own_gemm_modes(pkg, cuda):
    """cfp_train_set_gemm_mode: two trainers in one process, one on the fp32 MFMA kernel and
    one on bf16 inputs, each with a captured update graph.  Each must equal, bit for bit, a
    twin that ran the same update eagerly under process-wide switches of the same values --
    also after the process-wide switches were flipped between the replays, which changes
    nothing for a trainer that carries its own mode (and triggers no new capture)."""
    import torch
    n, T = 64, 6
    modes = ((0, 0), (1, 1))           # (bf16, split)
    for own in modes:
        (_, pol_o, tr_o, _), (_, pol_t, tr_t, _) = [_collect(pkg, cuda, n, T, 421, 0.1) for _ in range(2)]
        tr_o.set_gemm_mode(*own)
        assert tr_o.gemm_mode() == own and tr_t.gemm_mode() == (0, 1)
        for it, ambient in enumerate(((0, 1), (1, 2), (0, 0))):
            pkg.policy.set_gemm_bf16(own[0]); pkg.policy.set_gemm_split(own[1])
            try:
                tr_t.update(use_graph=False)        # the twin follows the process-wide switches
                torch.cuda.synchronize()
                pkg.policy.set_gemm_bf16(ambient[0]); pkg.policy.set_gemm_split(ambient[1])
                tr_o.update(use_graph=True)         # its own mode, whatever the switches say
                torch.cuda.synchronize()
            finally:
                pkg.policy.set_gemm_bf16(False); pkg.policy.set_gemm_split(1)
            assert torch.equal(pol_o.params, pol_t.params), f"own mode {own}, iteration {it}, ambient {ambient}"
            assert torch.equal(tr_o.buf("loss_acc"), tr_t.buf("loss_acc"))
        tr_o.set_gemm_mode(-1, -1)
        assert tr_o.gemm_mode() == (0, 1)
        with pytest.raises(pkg._lib.CfpError):
            tr_o.set_gemm_mode(2, 0)
        for pol, tr in ((pol_o, tr_o), (pol_t, tr_t)):
            tr.close(); pol.close()


@pytest.mark.parametrize("seed,layers", [(500, 3), (501, 2), (502, 1), (503, 3)])
def test_bf16_state_slab(pkg, cuda, seed, layers):
    """cfp_train_set_bf16_rstate: the rollout's bf16-input forward writes the post-zero state
    rows as bf16 and the bf16 update reads them as bf16.  (a) the slab is, bit for bit, the
    fp32 slab of a twin trainer rounded to bf16 (nearest even), and the live state and head
    rows do not change; (b) every gradient segment of the update is within 1e-3 (relative
    Frobenius norm) of the bf16-operand fp64 update evaluated on that slab, and the update
    reproduces bit for bit; (c) the two ends that exist on the bf16 path only refuse the others
    with an error: an fp32 forward asked to write the slab, a backward outside the bf16 mode."""
    import torch
    from parity_util import TOL_BF16_OPS, bf16_round, fro_err, expand_records
    n, T = 64, 8
    for k in range(16):          # a batch off the candidate function's kink (see _collect_off_the_kink)
        params = random_params(layers, seed + 1000 * k, scale=0.3)
        pols = [pkg.Policy(n, layers, seed=1) for _ in range(2)]
        trs = []
        for i, pol in enumerate(pols):
            pol.set_params(params)
            pol.set_gemm_bf16(True)
            tr = pkg.Trainer(pol, T)
            if i == 1:
                tr.set_bf16_rstate(True)
            trs.append(tr)
        rng = np.random.default_rng(seed + 1)
        r_done = (rng.random((T, n)) < 0.1).astype(np.uint8)
        for pol, tr in zip(pols, trs):
            pol.state.zero_()
            for t in range(T):
                rec = _t(synth_records_host(n, seed, t), cuda)
                term = _t(r_done[t - 1].astype(np.float32) if t else np.zeros(n, np.float32), cuda)
                tr.record_step(t, rec, term)
        torch.cuda.synchronize()
        slab32 = trs[0].buf("r_state").cpu().numpy()
        raw = trs[1].buf("r_state").view(torch.bfloat16).flatten()[: slab32.size]
        slab16 = raw.float().cpu().numpy().reshape(slab32.shape)
        assert np.array_equal(slab16.view(np.uint32), bf16_round(slab32).astype(np.float32).view(np.uint32)), "slab rounding"
        assert torch.equal(pols[0].state, pols[1].state) and torch.equal(trs[0].buf("r_value"), trs[1].buf("r_value"))
        host = dict(r_act=rng.integers(0, ACTIONS, (T, n)).astype(np.int32),
                    adv=rng.standard_normal((T, n)).astype(np.float32),
                    ret=rng.standard_normal((T, n)).astype(np.float32), r_done=r_done)
        host["r_obs"] = trs[1].buf("r_obs").cpu().numpy()
        host["r_state"] = slab16
        host["r_logprob"] = np.zeros((T, n), np.float32)
        for t in range(T):
            ref = ob.forward_f64(params, layers, expand_records(host["r_obs"][t]), host["r_state"][t], None)
            z = ref["logits"] - ref["logits"].max(axis=1, keepdims=True)
            logp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
            host["r_logprob"][t] = (logp[np.arange(n), host["r_act"][t]] + 0.02 * rng.standard_normal(n)).astype(np.float32)
        batch, keep = ob.make_batch(T, n, 0, n, layers, T, **host)
        if min(ob.ppo_min_abs_zh(params, batch), ob.ppo_min_abs_zh(params, batch, bf16_ops=True)) >= KINK_MARGIN:
            break
        for pol, tr in zip(pols, trs):
            tr.close(); pol.close()
    else:
        raise AssertionError("no batch off the kink")
    tr, pol = trs[1], pols[1]
    for name in ("r_act", "r_logprob", "adv", "ret", "r_done"):
        tr.buf(name).copy_(_t(host[name], cuda))
    tr.adv_stats()
    g_q = ob.ppo_backward_bf16ops_f64(params, batch, bf16_storage=True)[0]
    # (c) outside the bf16 mode the backward refuses the slab
    with pytest.raises(pkg._lib.CfpError):
        tr.backward(0, n)
    pkg.policy.set_gemm_bf16(True)
    tr.set_bf16_storage(True)
    try:
        outs = []
        for _ in range(2):
            tr.buf("grads").zero_(); tr.zero_loss()
            tr.backward(0, n)
            torch.cuda.synchronize()
            outs.append(tr.buf("grads").cpu().numpy().copy())
        assert np.array_equal(outs[0], outs[1]), "bitwise reproducible"
        for name, sl in _segments(layers):
            e = fro_err(outs[0][sl], g_q[sl])
            assert e <= TOL_BF16_OPS, f"d{name} with a bf16 state slab: {e:.3e} from the bf16-operand fp64 update"
    finally:
        pkg.policy.set_gemm_bf16(False)
        tr.set_bf16_storage(False)
    # (c) the fp32 forward cannot write a bf16 slab
    pol.set_gemm_bf16(False)
    with pytest.raises(pkg._lib.CfpError):
        tr.record_step(0, _t(synth_records_host(n, seed, 0), cuda), torch.zeros(n, device=cuda))
    for pol, tr in zip(pols, trs):
        tr.close(); pol.close()


def test_checkpoint_roundtrip(pkg, cuda, tmp_path):
    """CFW1 file: header words, byte-exact params, mirrors refreshed on load, and the
    reference's rejections (wrong shape, truncated file)."""
    import torch
    n = 32
    a = pkg.Policy(n, L, seed=11)
    path = tmp_path / "w.cfw"
    a.save_weights(path)
    raw = np.fromfile(path, dtype=np.uint32)
    assert raw[0] == 0x31574643 and raw[1] == 256 and raw[2] == L and raw[3] == a.param_count
    assert np.array_equal(raw[4:].view(np.float32), a.get_params())
    b = pkg.Policy(n, L, seed=12)
    b.load_weights(path)
    assert np.array_equal(b.get_params(), a.get_params())
    rec = pkg.policy.synth_records(n, 3, 0)
    term = torch.zeros(n, device=cuda)
    sa = torch.zeros(L, n, HIDDEN, device=cuda); sb = torch.zeros(L, n, HIDDEN, device=cuda)
    assert torch.equal(a.forward(rec, term, sa), b.forward(rec, term, sb))
    c = pkg.Policy(n, 2, seed=1)
    before = c.get_params()
    with pytest.raises(pkg._lib.CfpError):
        c.load_weights(path)                       # layer count differs
    assert np.array_equal(c.get_params(), before)
    raw[: 4 + 100].tofile(tmp_path / "short.cfw")
    with pytest.raises(pkg._lib.CfpError):
        b.load_weights(tmp_path / "short.cfw")
    with pytest.raises(pkg._lib.CfpError):
        b.load_weights(tmp_path / "missing.cfw")
    for p in (a, b, c):
        p.close()


@pytest.mark.parametrize("seed,layers", [(150, 3), (151, 2), (152, 1), (153, 3), (154, 2), (155, 1),
                                         (156, 3), (157, 3)])
def test_backward_with_bf16_gemms(pkg, cuda, seed, layers):
    """The update with bf16 GEMM inputs (cfp_set_gemm_bf16) on eight consecutive seeds, one
    to three layers.  Asserted: every gradient segment within 1e-3 (relative Frobenius norm)
    of the fp64 evaluation of the same update with the same operands rounded to bf16
    (cfo_ppo_backward_bf16ops_f64) -- what is left between the two is fp32 accumulation and
    the fp32 elementwise work.  Reported, and asserted only for the whole gradient: the
    distance to the exact fp64 update, which is the batch's own sensitivity to bf16
    operands (a segment whose sum nearly cancels reads several 1e-2 on some batches).
    The clipped surrogate is
    discontinuous in the logits where the probability ratio crosses 1 +- clip, so
    the behaviour log-probabilities are set to the current policy's own (plus 0.02
    of noise): every sample then sits well inside the clip range and the loss is
    smooth under the 1e-2-sized logit perturbation bf16 inputs cause."""
    import torch
    from parity_util import TOL_BF16, TOL_BF16_OPS, fro_err, expand_records
    n, T = 64, 8
    params, pol, tr, host, seed = _collect_off_the_kink(pkg, cuda, n, T, seed, 0.1, layers=layers)
    rng = np.random.default_rng(seed + 1)
    for t in range(T):
        ref = ob.forward_f64(params, layers, expand_records(host["r_obs"][t]), host["r_state"][t], None)
        z = ref["logits"] - ref["logits"].max(axis=1, keepdims=True)
        logp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
        host["r_logprob"][t] = (logp[np.arange(n), host["r_act"][t]]
                                + 0.02 * rng.standard_normal(n)).astype(np.float32)
    tr.buf("r_logprob").copy_(_t(host["r_logprob"], cuda))
    batch, keep = ob.make_batch(T, n, 0, n, layers, T, **host)
    g_ref, l3_ref = ob.ppo_backward_f64(params, batch)
    # split kernels off: the map-byte rows of dW_enc run against an exact split of dh_enc
    g_qs = {1: ob.ppo_backward_bf16ops_f64(params, batch)[0],
            0: ob.ppo_backward_bf16ops_f64(params, batch, map_rows_exact=True)[0]}
    # (bf16 inputs, split mode): fp32 on the split kernels with nine / six partial products
    # and on the fp32 MFMA kernel; bf16 inputs on the split kernels with the fused bf16
    # window recompute, and on the generic bf16 kernel with the unfused chain
    grads = {}
    for mode in ((False, 1), (False, 2), (False, 0), (True, 1), (True, 0)):
        pkg.policy.set_gemm_bf16(mode[0])
        pkg.policy.set_gemm_split(mode[1])
        try:
            tr.buf("grads").zero_()
            tr.zero_loss()
            tr.backward(0, n)
            torch.cuda.synchronize()
        finally:
            pkg.policy.set_gemm_bf16(False)
            pkg.policy.set_gemm_split(1)
        grads[mode] = tr.buf("grads").cpu().numpy().copy()
        l3 = tr.buf("loss_acc").cpu().numpy()
        # the pg sum nearly cancels (ratios ~ 1, zero-mean advantages): absolute floor
        tol = 1e-2 if mode[0] else 1e-4
        assert np.allclose(l3, l3_ref, rtol=tol, atol=tol * np.abs(l3_ref).max()), (mode, l3, l3_ref)
    for name, sl in _segments(layers):
        for split in (1, 2, 0):
            assert_close(grads[(False, split)][sl], g_ref[sl], TOL_FP32,
                         f"fp32 d{name}, split mode {split} (same batch)")
    for split in (1, 0):
        worst = 0.0
        g_q = g_qs[split]
        for name, sl in _segments(layers):
            eq = fro_err(grads[(True, split)][sl], g_q[sl])
            e = fro_err(grads[(True, split)][sl], g_ref[sl])
            print(f"seed {seed} L{layers} split {split} d{name}: {eq:.2e} vs bf16-operand fp64, {e:.2e} vs exact fp64")
            assert eq <= TOL_BF16_OPS, f"bf16 d{name}, split mode {split}: {eq:.3e} from the bf16-operand fp64 update"
            worst = max(worst, e)
        assert worst > 1e-4, "the bf16 GEMMs did not run"
        e_all = fro_err(grads[(True, split)], g_ref)
        assert e_all <= TOL_BF16, f"whole gradient, split mode {split}: {e_all:.3e} from the exact fp64 update"
    tr.close(); pol.close()


def test_adam_writes_every_weight_mirror(pkg, cuda):
    """cfp_train_adam rewrites the forward kernels' weight mirrors (fp32 MFMA order, the
    three-term bf16 split of the encoder, the bf16 mirrors) in the pass that updates the
    parameters.  After two steps with gradients on every parameter, the fp32 and the
    bf16-input forward of the trained policy must equal, bit for bit, those of a fresh
    policy given the same parameters through cfp_policy_set_params, whose mirrors come
    from the pack kernels."""
    import torch
    n = 64
    pol = pkg.Policy(n, L, seed=21)
    tr = pkg.Trainer(pol, 4)
    rng = np.random.default_rng(22)
    before = pol.get_params()
    for _ in range(2):
        g = (rng.standard_normal(before.size) * 0.1).astype(np.float32)
        tr.buf("grads").copy_(_t(g, cuda))
        tr.adam()
    torch.cuda.synchronize()
    after = pol.get_params()
    assert np.all(after != before)                      # every parameter moved
    twin = pkg.Policy(n, L, seed=99)
    twin.set_params(after)
    rec = _t(synth_records_host(n, 23, 0), cuda)
    term = torch.zeros(n, device=cuda)
    s0 = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    for bf16 in (False, True):
        pol.set_gemm_bf16(bf16); twin.set_gemm_bf16(bf16)
        sa, sb = _t(s0, cuda), _t(s0, cuda)
        av_a = pol.forward(rec, term, sa).clone()
        av_b = twin.forward(rec, term, sb).clone()
        assert torch.equal(av_a, av_b), f"bf16={bf16}: head rows differ"
        assert torch.equal(sa, sb), f"bf16={bf16}: states differ"
    tr.close(); pol.close(); twin.close()


def test_small_tile_mirrors_current_when_switched_on_after_training(pkg, cuda):
    """Adam steps taken with 16-env tiles off, eager and as a captured update, then the
    switch is turned on: the small-tile forward must run on the updated weights (equal,
    bit for bit, to a fresh policy given the same parameters)."""
    import torch
    n = 64
    pol = pkg.Policy(n, L, seed=41)
    tr = pkg.Trainer(pol, 4)
    rng = np.random.default_rng(42)
    for _ in range(2):
        g = (rng.standard_normal(pol.param_count) * 0.1).astype(np.float32)
        tr.buf("grads").copy_(_t(g, cuda))
        tr.adam()
    torch.cuda.synchronize()
    pol.set_small_tiles(True)
    twin = pkg.Policy(n, L, seed=99)
    twin.set_params(pol.get_params())
    twin.set_small_tiles(True)
    rec = _t(synth_records_host(n, 43, 0), cuda)
    term = torch.zeros(n, device=cuda)
    s0 = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    sa, sb = _t(s0, cuda), _t(s0, cuda)
    assert torch.equal(pol.forward(rec, term, sa), twin.forward(rec, term, sb))
    assert torch.equal(sa, sb)
    tr.close(); pol.close(); twin.close()


@pytest.mark.parametrize("n,T,minibatches,bwd_win,done_p,layers,seed",
                         [(64, 8, 1, 0, 0.1, 3, 300), (128, 6, 2, 4, 0.15, 3, 301),
                          # one and two layers: the stream of every kernel of the chain changes
                          # with the parity of the layer count
                          (64, 6, 1, 4, 0.1, 1, 302), (64, 6, 1, 0, 0.1, 2, 303),
                          (64, 8, 1, 4, 0.1, 3, 304), (128, 8, 2, 0, 0.2, 2, 305),
                          (128, 4, 1, 2, 0.1, 1, 306), (64, 8, 1, 0, 0.05, 3, 307)])
def test_backward_with_bf16_storage(pkg, cuda, n, T, minibatches, bwd_win, done_p, layers, seed):
    """bf16 GEMM inputs with the window workspace stored as bf16 (cfp_train_set_bf16_storage:
    gate pre-activations, their gradients, the layer inputs and the hidden-state gradients
    between the layers; the reference's CF_GEMM_BF16 storage) on eight consecutive seeds.
    Asserted: every gradient segment, with either storage, within 1e-3 (relative Frobenius
    norm) of the fp64 evaluation of the same update with the same values rounded to bf16
    (cfo_ppo_backward_bf16ops_f64 in the matching storage mode), and the whole gradient
    within 2e-2 of the exact fp64 update.  Reported: the per-segment distance to the exact
    fp64 update (the batch's own sensitivity to bf16; a value-head gradient that nearly
    cancels reads 3e-2 to 5e-2 on some batches with either storage).  Behaviour
    log-probabilities are the current policy's own plus noise, so no sample sits on the
    clip discontinuity (see test_backward_with_bf16_gemms)."""
    import torch
    from parity_util import TOL_BF16, TOL_BF16_OPS, fro_err, expand_records
    params, pol, tr, host, seed = _collect_off_the_kink(pkg, cuda, n, T, seed, done_p, layers=layers,
                                                        minibatches=minibatches, bwd_win=bwd_win)
    rng = np.random.default_rng(seed + 1)
    for t in range(T):
        ref = ob.forward_f64(params, layers, expand_records(host["r_obs"][t]), host["r_state"][t], None)
        z = ref["logits"] - ref["logits"].max(axis=1, keepdims=True)
        logp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
        host["r_logprob"][t] = (logp[np.arange(n), host["r_act"][t]]
                                + 0.02 * rng.standard_normal(n)).astype(np.float32)
    tr.buf("r_logprob").copy_(_t(host["r_logprob"], cuda))
    mb = n // minibatches
    pkg.policy.set_gemm_bf16(True)
    try:
        for m in range(minibatches):
            batch, keep = ob.make_batch(T, n, m * mb, mb, layers, T, **host)
            g_ref, l3_ref = ob.ppo_backward_f64(params, batch)
            g_q = {st: ob.ppo_backward_bf16ops_f64(params, batch, bf16_storage=st)[0] for st in (False, True)}
            got = {}
            for store16 in (False, True):
                tr.set_bf16_storage(store16)
                outs = []
                for _ in range(2):
                    tr.buf("grads").zero_(); tr.zero_loss()
                    tr.backward(m * mb, mb)
                    torch.cuda.synchronize()
                    outs.append(tr.buf("grads").cpu().numpy().copy())
                assert np.array_equal(outs[0], outs[1]), "bitwise reproducible"
                got[store16] = outs[0]
                l3 = tr.buf("loss_acc").cpu().numpy()
                assert np.allclose(l3, l3_ref, rtol=1e-2, atol=1e-2 * np.abs(l3_ref).max()), (store16, l3, l3_ref)
            for name, sl in _segments(layers):
                for st in (False, True):
                    eq = fro_err(got[st][sl], g_q[st][sl])
                    e = fro_err(got[st][sl], g_ref[sl])
                    print(f"seed {seed} L{layers} minibatch {m} bf16 storage {st} d{name}: {eq:.2e} vs "
                          f"bf16-operand fp64, {e:.2e} vs exact fp64")
                    assert eq <= TOL_BF16_OPS, (f"minibatch {m} d{name}, bf16 storage {st}: {eq:.3e} from the "
                                                f"bf16-operand fp64 update")
            for st in (False, True):
                e_all = fro_err(got[st], g_ref)
                assert e_all <= TOL_BF16, f"minibatch {m}, bf16 storage {st}: whole gradient {e_all:.3e}"
            assert not np.array_equal(got[True], got[False]), "the storage mode did not take effect"
    finally:
        pkg.policy.set_gemm_bf16(False)
        tr.set_bf16_storage(False)
    tr.close(); pol.close()


def test_small_tile_mirrors_follow_adam(pkg, cuda):
    """With 16-env tiles on, cfp_train_adam also repacks that kernel's weight mirrors: after
    two steps the trained policy's small-tile forward equals, bit for bit, that of a fresh
    policy given the same parameters."""
    import torch
    n = 64
    pol = pkg.Policy(n, L, seed=31)
    pol.set_small_tiles(True)
    tr = pkg.Trainer(pol, 4)
    rng = np.random.default_rng(32)
    for _ in range(2):
        g = (rng.standard_normal(pol.param_count) * 0.1).astype(np.float32)
        tr.buf("grads").copy_(_t(g, cuda))
        tr.adam()
    torch.cuda.synchronize()
    twin = pkg.Policy(n, L, seed=98)
    twin.set_params(pol.get_params())
    twin.set_small_tiles(True)
    rec = _t(synth_records_host(n, 33, 0), cuda)
    term = torch.zeros(n, device=cuda)
    s0 = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    sa, sb = _t(s0, cuda), _t(s0, cuda)
    assert torch.equal(pol.forward(rec, term, sa), twin.forward(rec, term, sb))
    assert torch.equal(sa, sb)
    tr.close(); pol.close(); twin.close()
