"""Pins the CPU oracle's policy forward / PPO backward (oracle/policy_ref.c,
oracle/policy_bwd_ref.c) against an independent numpy fp64 evaluation, closed
forms, brute force and finite differences."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import (ACTIONS, GRU, HIDDEN, OBS, expand_records, numpy_forward_f64,
                         random_params, rel_err, split_params, synth_records_host)

L = 3


def _inputs(n, seed, term_p=0.3):
    rng = np.random.default_rng(seed)
    rec = synth_records_host(n, seed, 0)
    x = expand_records(rec)
    state = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    term = (rng.random(n) < term_p).astype(np.float32)
    return rec, x, state, term


def test_c_oracle_matches_numpy_fp64():
    params = random_params(L, 1)
    rec, x, state, term = _inputs(48, 2)
    a = ob.forward_f64(params, L, x, state, term)
    b = numpy_forward_f64(params, L, x, state, term)
    for k in ("h_enc", "r_state", "state", "h3", "logits", "values"):
        assert rel_err(a[k], b[k]) < 1e-12, k


def test_zero_gate_weights_closed_form():
    """W_gru = 0 => zh=zg=zp=0 => out = 0.5 st + 0.25, h' = 0.5 out + 0.5 h."""
    params = random_params(L, 3)
    sp = split_params(params, L)
    sp["W_gru"][...] = 0.0
    rec, x, state, term = _inputs(16, 4, term_p=0.0)
    r = ob.forward_f64(params, L, x, state, None)
    h = x.astype(np.float64) @ sp["W_enc"].astype(np.float64) + sp["b_enc"]
    for l in range(L):
        out = 0.5 * state[l].astype(np.float64) + 0.25
        assert np.allclose(r["state"][l], out, rtol=0, atol=1e-14)
        h = 0.5 * out + 0.5 * h
    assert np.allclose(r["h3"], h, rtol=1e-13, atol=1e-13)


def test_terminal_zeroes_state_and_zero_features_give_bias():
    params = random_params(L, 5)
    sp = split_params(params, L)
    rec, x, state, _ = _inputs(8, 6)
    term = np.array([1, 0, 1, 0, 0, 0, 0, 1], np.float32)
    r = ob.forward_f64(params, L, x, state, term)
    assert not r["r_state"][:, term != 0].any()
    assert np.array_equal(r["r_state"][:, term == 0], state[:, term == 0].astype(np.float64))
    z = ob.forward_f64(params, L, np.zeros_like(x), state, term)
    assert np.allclose(z["h_enc"], np.broadcast_to(sp["b_enc"].astype(np.float64), (8, HIDDEN)))
    # zeroed state == explicit zero state
    st0 = state.copy(); st0[:, term != 0] = 0
    r0 = ob.forward_f64(params, L, x, st0, None)
    assert np.array_equal(r0["logits"], r["logits"])


def test_gate_saturation_limits():
    """p -> 1 gives h' = out, p -> 0 gives h' = x; zg -> +inf gives out = g(zh)."""
    params = random_params(1, 7)
    sp = split_params(params, 1)
    sp["W_enc"][...] = 0.0; sp["b_enc"][...] = 1.0       # h = 1 for every unit
    W = sp["W_gru"][0]; W[...] = 0.0
    W[2 * HIDDEN:, :] = 1.0                               # zp = +256 -> p = 1
    x = np.zeros((4, OBS), np.float32)
    state = np.full((1, 4, HIDDEN), 0.3, np.float32)
    r = ob.forward_f64(params, 1, x, state, None)
    assert np.allclose(r["h3"], r["state"][0])
    W[2 * HIDDEN:, :] = -1.0                              # p = 0
    r = ob.forward_f64(params, 1, x, state, None)
    assert np.allclose(r["h3"], 1.0, atol=1e-100)
    W[HIDDEN:2 * HIDDEN, :] = 1.0; W[:HIDDEN, :] = 0.01   # sg = 1, zh = 2.56
    r = ob.forward_f64(params, 1, x, state, None)
    assert np.allclose(r["state"][0], 2.56 + 0.5, rtol=1e-6)
    W[:HIDDEN, :] = -0.01                                  # zh = -2.56 -> sigmoid
    r = ob.forward_f64(params, 1, x, state, None)
    assert np.allclose(r["state"][0], 1 / (1 + np.exp(2.56)), rtol=1e-6)


def test_fp32_port_tracks_fp64_and_carries_state():
    params = random_params(L, 8)
    n, T = 24, 6
    rng = np.random.default_rng(9)
    st32 = np.zeros((L, n, HIDDEN), np.float32)
    st64 = np.zeros((L, n, HIDDEN), np.float64)
    for t in range(T):
        rec = synth_records_host(n, 10, t)
        term = (rng.random(n) < 0.2).astype(np.float32) if t else np.zeros(n, np.float32)
        av = ob.forward_f32(params, L, rec, st32, term, threads=2)
        r = ob.forward_f64(params, L, expand_records(rec), st64, term)
        st64 = r["state"]
        assert rel_err(av[:, :ACTIONS], r["logits"]) < 1e-4
        assert rel_err(av[:, ACTIONS], r["values"]) < 1e-4
        assert rel_err(st32, st64) < 1e-4


def test_multi_step_carry_brute_force():
    """n=4, T=8 in plain numpy loops over time, random terminals."""
    params = random_params(L, 11)
    n, T = 4, 8
    rng = np.random.default_rng(12)
    st_o = np.zeros((L, n, HIDDEN)); st_n = np.zeros((L, n, HIDDEN))
    for t in range(T):
        x = expand_records(synth_records_host(n, 13, t))
        term = (rng.random(n) < 0.4).astype(np.float32)
        a = ob.forward_f64(params, L, x, st_o, term)
        b = numpy_forward_f64(params, L, x, st_n, term)
        st_o, st_n = a["state"], b["state"]
        assert rel_err(a["logits"], b["logits"]) < 1e-12
    assert rel_err(st_o, st_n) < 1e-12


# ---- PPO update ------------------------------------------------------------------
def _rollout(params, n, T, seed, done_p=0.1, layers=L):
    """Synthetic stored rollout whose r_state is what the oracle forward itself
    would have recorded (zero initial state, zeroed after a done)."""
    rng = np.random.default_rng(seed)
    r_obs = np.stack([synth_records_host(n, seed, t) for t in range(T)])
    r_done = (rng.random((T, n)) < done_p).astype(np.uint8)
    r_state = np.zeros((T, layers, n, HIDDEN), np.float32)
    st = np.zeros((layers, n, HIDDEN))
    for t in range(T):
        term = r_done[t - 1].astype(np.float32) if t else np.zeros(n, np.float32)
        r = ob.forward_f64(params, layers, expand_records(r_obs[t]), st, term)
        r_state[t] = r["r_state"]
        st = r["r_state"].astype(np.float32).astype(np.float64) * 0 + r["state"]
        # the stored record is fp32; keep the live carry consistent with it
        st = np.where(np.isfinite(st), st, 0.0)
    r_act = rng.integers(0, ACTIONS, (T, n)).astype(np.int32)
    r_logprob = np.full((T, n), -np.log(ACTIONS), np.float32) + 0.1 * rng.standard_normal((T, n)).astype(np.float32)
    adv = rng.standard_normal((T, n)).astype(np.float32)
    ret = rng.standard_normal((T, n)).astype(np.float32)
    return dict(r_obs=r_obs, r_state=r_state, r_act=r_act, r_logprob=r_logprob, adv=adv,
                ret=ret, r_done=r_done)


def _consistent_rollout(params, n, T, seed, done_p=0.1):
    """As _rollout, but the stored fp32 state is also what the live recurrence
    carries (state rounded to fp32 each step), so loss (live) == recompute (stored)."""
    rng = np.random.default_rng(seed)
    ro = _rollout(params, n, T, seed, done_p)
    st = np.zeros((L, n, HIDDEN), np.float32)
    for t in range(T):
        term = ro["r_done"][t - 1].astype(np.float32) if t else np.zeros(n, np.float32)
        r = ob.forward_f64(params, L, expand_records(ro["r_obs"][t]), st, term)
        ro["r_state"][t] = r["r_state"].astype(np.float32)
        st = r["state"].astype(np.float32)
    return ro


def test_backward_matches_finite_differences():
    """The reference's own gradcheck method (craftax_full.cu:13854-13907): central
    differences of the loss on the largest-|g| and random parameters; fail if
    diff > 2e-4 and rel > 3e-2.  In fp64 the agreement is far tighter (1e-5
    relative with a 1e-5 step; the synthetic features are large, so the loss has
    strong curvature and a 1e-3 step is already 0.25 % off)."""
    params = random_params(L, 21)
    n, T = 6, 5
    ro = _consistent_rollout(params, n, T, 22, done_p=0.15)
    batch, keep = ob.make_batch(T, n, 0, n, L, T, **ro)
    g, l3 = ob.ppo_backward_f64(params, batch)
    loss, l3b = ob.ppo_loss_f64(params, batch)
    assert np.allclose(l3, l3b, rtol=1e-6), "recompute and live replay disagree on the loss"
    rng = np.random.default_rng(23)
    o = {k: v for k, v in zip(("W_enc", "b_enc", "W_gru", "W_a", "b_a", "W_v", "b_v"),
                              np.cumsum([0, OBS * HIDDEN, HIDDEN, L * GRU * HIDDEN,
                                         ACTIONS * HIDDEN, ACTIONS, HIDDEN]))}
    probes = list(np.argsort(-np.abs(g))[:8]) + list(rng.integers(0, params.size, 24))
    probes += [o["b_enc"] + 3, o["W_gru"] + 5, o["W_gru"] + GRU * HIDDEN + 77,
               o["W_gru"] + 2 * GRU * HIDDEN + 600 * HIDDEN + 9, o["b_a"] + 2, o["W_v"] + 1,
               o["b_v"]]
    worst = 0.0
    for i in probes:
        eps = 1e-5 * max(1.0, abs(float(params[i])))   # curvature is large: see docstring
        pp = params.copy(); pp[i] += eps
        pm = params.copy(); pm[i] -= eps
        # fp32 params: use the actually representable step
        h = (float(pp[i]) - float(pm[i]))
        fd = (ob.ppo_loss_f64(pp, batch)[0] - ob.ppo_loss_f64(pm, batch)[0]) / h
        diff = abs(fd - g[i]); rel = diff / max(abs(fd), abs(g[i]), 1e-12)
        worst = max(worst, min(diff / 2e-6, rel / 1e-5))
        assert not (diff > 2e-6 and rel > 1e-5), (int(i), fd, g[i])
    assert worst < 1.0


@pytest.mark.parametrize("seg_len,layers", [(5, 3), (2, 2), (3, 1)])
def test_bf16_operand_backward_against_a_numpy_restatement(seg_len, layers):
    """The bf16-operand comparators of the update (cfo_ppo_backward_bf16ops_f64, with fp32 and
    with bf16 window storage) against a restatement with numpy matmuls over all envs at once.
    The restatement is first held, with exact operands, to the gradient that the finite
    differences above pin; with rounding switched on it then differs from that code only in
    where an operand is rounded, and the compiled comparator must round in the same places."""
    from parity_util import numpy_ppo_backward_f64, fro_err
    params = random_params(layers, 71)
    n, T = 6, 5
    ro = _rollout(params, n, T, 72, done_p=0.2, layers=layers)
    feats = np.stack([expand_records(ro["r_obs"][t]) for t in range(T)])
    batch, keep = ob.make_batch(T, n, 0, n, layers, seg_len, **ro)
    kw = dict(seg_len=seg_len)
    args = (params, layers, feats, ro["r_state"], ro["r_act"], ro["r_logprob"], ro["adv"], ro["ret"],
            ro["r_done"])
    g0, l0 = ob.ppo_backward_f64(params, batch)
    n0, m0 = numpy_ppo_backward_f64(*args, mode=0, **kw)
    assert np.allclose(m0, l0, rtol=1e-11)
    assert fro_err(n0, g0) < 1e-12
    seen = []
    for mode, exact in ((1, False), (2, False), (1, True)):
        gc, lc = ob.ppo_backward_bf16ops_f64(params, batch, bf16_storage=(mode == 2), map_rows_exact=exact)
        gn, ln = numpy_ppo_backward_f64(*args, mode=mode, map_rows_exact=exact, **kw)
        assert np.allclose(ln, lc, rtol=1e-11)
        # a sum that lands within an fp64 rounding of a bf16 tie may round the other way in
        # the two codes: the bound leaves room for a handful of such entries
        assert fro_err(gc, gn) < 1e-6, mode
        assert 1e-4 < fro_err(gc, g0) < 1e-1, "rounding took effect"
        seen.append(gc)
    assert 1e-5 < fro_err(seen[1], seen[0]), "the storage mode rounds more"
    assert 1e-5 < fro_err(seen[2], seen[0]), "the map rows of dW_enc follow the switch"


def test_backward_truncation_and_done_semantics():
    params = random_params(L, 31)
    n, T = 4, 6
    ro = _consistent_rollout(params, n, T, 32, done_p=0.0)
    full, k1 = ob.make_batch(T, n, 0, n, L, T, **ro)
    split, k2 = ob.make_batch(T, n, 0, n, L, 2, **ro)      # bptt_split = 3
    g_full, _ = ob.ppo_backward_f64(params, full)
    g_split, _ = ob.ppo_backward_f64(params, split)
    assert not np.allclose(g_full, g_split)                 # dcarry cut changes grads
    # all dones set: every step's dcarry is blocked => equals seg_len = 1
    ro1 = dict(ro); ro1["r_done"] = np.ones_like(ro["r_done"])
    a, k3 = ob.make_batch(T, n, 0, n, L, T, **ro1)
    b, k4 = ob.make_batch(T, n, 0, n, L, 1, **ro)
    ga, _ = ob.ppo_backward_f64(params, a)
    gb, _ = ob.ppo_backward_f64(params, b)
    assert np.allclose(ga, gb, rtol=1e-12, atol=1e-15)
    # heads get gradient only from their own step: unaffected by truncation
    oa = OBS * HIDDEN + HIDDEN + L * GRU * HIDDEN
    assert np.allclose(g_full[oa:], g_split[oa:], rtol=1e-12, atol=1e-15)


def test_zero_advantage_gives_entropy_and_value_gradient_only():
    params = random_params(L, 41)
    n, T = 4, 3
    ro = _consistent_rollout(params, n, T, 42)
    ro["adv"] = np.full((T, n), 0.7, np.float32)            # constant => normalised A = 0
    b, k = ob.make_batch(T, n, 0, n, L, T, **ro)
    g, l3 = ob.ppo_backward_f64(params, b)
    assert abs(l3[0]) < 1e-6                                # policy loss term vanishes
    b2, k2 = ob.make_batch(T, n, 0, n, L, T, **ro, vf=0.0, ent=0.0)
    g2, _ = ob.ppo_backward_f64(params, b2)
    assert np.abs(g2).max() < 1e-7
    assert np.abs(g).max() > 1e-6


def test_gae_and_adam_closed_forms():
    T, n = 5, 3
    rng = np.random.default_rng(51)
    values = rng.standard_normal((T, n)).astype(np.float32)
    rewards = rng.standard_normal((T, n)).astype(np.float32)
    dones = (rng.random((T, n)) < 0.3).astype(np.uint8)
    vboot = rng.standard_normal(n).astype(np.float32)
    adv = np.zeros((T, n)); ret = np.zeros((T, n))
    ob.cfo().cfo_gae_f64(values.ctypes.data, rewards.ctypes.data, dones.ctypes.data,
                         vboot.ctypes.data, adv.ctypes.data, ret.ctypes.data, n, T, 0.99, 0.95)
    # textbook: A_t = sum_k (gamma*lam)^k * prod(nonterm) * delta_{t+k}
    for e in range(n):
        for t in range(T):
            acc, w = 0.0, 1.0
            for k in range(t, T):
                vn = float(vboot[e] if k == T - 1 else values[k + 1, e])
                nt = 0.0 if dones[k, e] else 1.0
                acc += w * (float(rewards[k, e]) + 0.99 * vn * nt - float(values[k, e]))
                w *= 0.99 * 0.95 * nt
            assert abs(acc - adv[t, e]) < 1e-12
            assert abs(acc + float(values[t, e]) - ret[t, e]) < 1e-12
    # Adam, first step from zero moments: update = lr * sign(g) (up to eps)
    p = np.array([1.0, -2.0, 3.0]); g = np.array([0.5, -0.25, 0.0])
    m = np.zeros(3); v = np.zeros(3)
    ob.cfo().cfo_adam_f64(p.ctypes.data, g.ctypes.data, m.ctypes.data, v.ctypes.data, 3, 1,
                          3e-4, 0.9, 0.999, 1e-8)
    assert np.allclose(p, [1.0 - 3e-4, -2.0 + 3e-4, 3.0], atol=1e-9)


# ---- classic-game policy (config 5) ---------------------------------------------------
def test_classic_expand_and_forward_oracle():
    from parity_util import synth_classic_records_host
    n = 24
    rec = synth_classic_records_host(n, 3, 1)
    assert rec[:, :63].max() <= 16 and rec[:, 126:142].max() <= 9
    assert set(np.unique(rec[:, 142])) <= {1, 2, 3, 4} and (rec[:, 63:126] != 0).any()
    x = ob.classic_expand(rec)
    # one-hot closed form: every cell has exactly one block channel set
    cells = x[:, :63 * 21].reshape(n, 63, 21)
    assert np.array_equal(cells[:, :, :17].sum(axis=2), np.ones((n, 63), np.float32))
    assert np.array_equal(cells[:, :, :17].argmax(axis=2), rec[:, :63])
    bits = (rec[:, 63:126, None] >> np.arange(4)) & 1
    assert np.array_equal(cells[:, :, 17:], bits.astype(np.float32))
    assert np.array_equal(x[:, 1323:1339], rec[:, 126:142].astype(np.float32) / np.float32(10.0))
    assert np.array_equal(x[:, 1339:1343].argmax(axis=1) + 1, rec[:, 142])
    assert np.array_equal(x[:, 1343].view(np.uint32), np.ascontiguousarray(rec[:, 144:148]).view(np.uint32)[:, 0])
    assert np.array_equal(x[:, 1344], rec[:, 143].astype(np.float32))
    params = random_params(L, 61, obs=1345, actions=17)
    rng = np.random.default_rng(62)
    state = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    term = (rng.random(n) < 0.3).astype(np.float32)
    a = ob.classic_forward_f64(params, L, x, state, term)
    b = numpy_forward_f64(params, L, x, state, term, obs=1345, actions=17)
    for k in ("h_enc", "state", "h3", "logits", "values"):
        assert rel_err(a[k], b[k]) < 1e-12, k
    # gathered-column form of the encoder == dense form
    sp = split_params(params, L, 1345, 17)
    e = 5
    h = sp["b_enc"].astype(np.float64).copy()
    for f in np.nonzero(x[e])[0]:
        h += float(x[e, f]) * sp["W_enc"][f].astype(np.float64)
    assert np.allclose(h, a["h_enc"][e], rtol=1e-13, atol=1e-13)


# ---- cfo_sample_action (cf_nn_sample_action, craftax_full.cu:9147-9165) -----------
def test_sample_action_closed_forms():
    """Pins the sampling restatement without the reference's RNG: with equal
    logits the cumulative sum is a staircase of equal steps, so the action is
    ceil(u*A) - 1 (0 for u = 0); a dominant logit takes every u > 0; the
    log-probability is log softmax; exp(logprob) over all actions sums to one."""
    A = 43
    u = np.array([0.0, 1e-7, 0.01, 0.2, 0.5, 0.999, 0.9999999], dtype=np.float32)
    eq = np.zeros((len(u), A), dtype=np.float32)
    act, lp, _ = ob.sample_actions(eq, u)
    expect = np.maximum(np.ceil(u.astype(np.float64) * A) - 1, 0).astype(np.int32)
    assert np.array_equal(act, expect)
    assert np.allclose(lp, -np.log(A), atol=1e-6)
    dom = np.full((len(u), A), -30.0, dtype=np.float32)
    dom[:, 17] = 5.0
    act, lp, _ = ob.sample_actions(dom, u)
    # u = 0 gives target 0 <= p[0] for any positive p[0]: action 0 by construction
    assert act[0] == 0 and np.all(act[(u > 0) & (u < 0.999999)] == 17)
    assert np.allclose(lp[act == 17], 0.0, atol=1e-6)
    rng = np.random.default_rng(5)
    logits = rng.standard_normal((1, A)).astype(np.float32) * 3
    # walk u over the unit interval: every action is hit in order, and the
    # log-probabilities reported along the way form a normalised distribution
    grid = (np.arange(20000, dtype=np.float32) + 0.5) / 20000
    acts, lps, _ = ob.sample_actions(np.repeat(logits, len(grid), 0), grid)
    assert np.all(np.diff(acts) >= 0)
    ref_lp = logits[0] - logits[0].max() - np.log(np.sum(np.exp(logits[0].astype(np.float64) - logits[0].max())))
    seen = np.unique(acts)
    assert np.allclose([lps[acts == a][0] for a in seen], ref_lp[seen], atol=2e-6)
    # frequencies on the grid equal the softmax probabilities to the grid resolution
    freq = np.bincount(acts, minlength=A) / len(grid)
    assert np.max(np.abs(freq - np.exp(ref_lp))) < 2.0 / len(grid) + 1e-6


# ---- Philox4x32-10 (the reference's curandStatePhilox4_32_10_t) --------------------
def test_philox_known_answer_vectors():
    """The three known-answer vectors published with the generator (Random123
    kat_vectors, "philox4x32 10": zero counter and key, all-ones, digits of pi).
    A wrong multiplier, Weyl constant, round count or word order fails all twelve
    words."""
    kats = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for ctr, key, out in kats:
        assert [int(x) for x in ob.philox4x32_10(ctr, key)] == out


def test_philox_uniform_state_layout():
    """cfo_philox_uniform against the block function: key = seed, counter low half =
    offset / 4, high half = subsequence, word = offset % 4, uniform = x * 2^-32 +
    2^-33 in (0, 1] (cuRAND's conversion; the state layout itself is held to rocRAND's
    engine in test_philox_draw_matches_rocrand)."""
    seed, sub = 0x0123456789ABCDEF, (7 << 32) | 99
    lib = ob.cfo()
    for off in (0, 1, 2, 3, 4, 5, 11, (1 << 34) + 2):
        words = ob.philox4x32_10([(off >> 2) & 0xffffffff, (off >> 2) >> 32, sub & 0xffffffff, sub >> 32],
                                 [seed & 0xffffffff, seed >> 32])
        x = np.float32(int(words[off & 3]))
        expect = np.float32(np.float64(x) * 2.0 ** -32 + 2.0 ** -33)   # one rounding, like the fma
        got = np.float32(lib.cfo_philox_uniform(seed, sub, off))
        assert got == expect and 0.0 < got <= 1.0
    u = ob.philox_uniforms(1234, range(20000), 5)
    assert abs(u.mean() - 0.5) < 0.01 and abs(u.var() - 1.0 / 12.0) < 0.005
    assert len(np.unique(u)) > 19900


def test_philox_draw_matches_rocrand():
    """cfo_philox_draw(seed, subsequence, offset) -- the 32-bit word behind the sampler's
    uniform -- against a library routine with the same three arguments: ROCm's rocRAND
    Philox4x32-10 engine on the host (rocrand_init followed by one rocrand), built by
    oracle/Makefile.  Offsets cover every residue mod 4, values past 2^32 and the carry
    of offset / 4 into the counter's second word; subsequences and seeds use all 64
    bits.  A wrong word order, swapped counter halves or an off-by-one in the output
    word fails here.  The float conversion is cuRAND's x * 2^-32 + 2^-33 (rocRAND adds
    2^-32 instead): closed form, test_philox_uniform_state_layout."""
    import ctypes as C
    import os
    path = os.path.join(os.path.dirname(ob.CFO_PATH), "librocrand_check.so")
    if not os.path.exists(path):
        pytest.skip("oracle/librocrand_check.so not built (needs hipcc)")
    lib = C.CDLL(path)
    lib.cfo_rocrand_draws.argtypes = [C.c_uint64, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]
    mine = ob.cfo()
    mine.cfo_philox_draw.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
    mine.cfo_philox_draw.restype = C.c_uint32
    rng = np.random.default_rng(77)
    total = 0
    for seed in (0, 1234, 1234 ^ 0xA5A5A5A5A5A5A5A5, 0xFFFFFFFFFFFFFFFF, 0x0123456789ABCDEF):
        sub = np.concatenate([np.arange(8, dtype=np.uint64),
                              rng.integers(0, 1 << 63, 600, dtype=np.uint64) * np.uint64(2) + np.uint64(1),
                              np.array([(1 << 32) - 1, 1 << 32, (1 << 64) - 1], dtype=np.uint64)])
        off = np.concatenate([np.arange(16, dtype=np.uint64),
                              rng.integers(0, 1 << 40, 580, dtype=np.uint64),
                              np.array([(1 << 34) - 1, 1 << 34, (1 << 34) + 1, (1 << 34) + 2, (1 << 34) + 3,
                                        (1 << 62) + 1, (1 << 63) + 2, (1 << 64) - 1, (1 << 64) - 4],
                                       dtype=np.uint64)])[: sub.size]
        sub = sub[: off.size]
        want = np.zeros(sub.size, dtype=np.uint32)
        lib.cfo_rocrand_draws(seed, sub.ctypes.data, off.ctypes.data, sub.size, want.ctypes.data)
        got = np.array([mine.cfo_philox_draw(seed, int(s), int(o)) for s, o in zip(sub, off)],
                       dtype=np.uint32)
        assert np.array_equal(got, want), (hex(seed), np.flatnonzero(got != want)[:5])
        assert set(int(o) & 3 for o in off) == {0, 1, 2, 3}
        # and the uniform is that draw through cuRAND's conversion
        u = np.array([mine.cfo_philox_uniform(seed, int(s), int(o)) for s, o in zip(sub[:64], off[:64])],
                     dtype=np.float32)
        assert np.array_equal(u, (want[:64].astype(np.float32).astype(np.float64) * 2.0 ** -32
                                  + 2.0 ** -33).astype(np.float32))
        total += sub.size
    assert total >= 3000


def test_ppo_loss_closed_form_with_zero_head_weights():
    """cfo_ppo_loss_f64's value, not only its derivative: with W_a = 0, b_a = 0, W_v = 0
    the policy is uniform whatever the trunk computes, so per sample
        H = ln 43,  ratio = exp(-ln 43 - old_logp),  v = b_v,
        pg = -min(ratio * A, clip(ratio, 1 - eps, 1 + eps) * A),  value term = (b_v - ret)^2 / 2
    with A the advantage normalised by the whole batch's mean and 1 / (std + 1e-8)."""
    params = random_params(L, 61)
    W_enc, b_enc, W_gru, W_a, b_a, W_v, b_v = split_params(params, L)
    o_wa = OBS * HIDDEN + HIDDEN + L * GRU * HIDDEN
    p = params.copy()
    p[o_wa: o_wa + ACTIONS * HIDDEN + ACTIONS + HIDDEN] = 0.0     # W_a, b_a, W_v
    bv = float(p[-1])
    n, T = 5, 4
    ro = _consistent_rollout(p, n, T, 62, done_p=0.2)
    rng = np.random.default_rng(63)
    ro["r_logprob"] = (-np.log(ACTIONS) + 0.4 * rng.standard_normal((T, n))).astype(np.float32)
    clip, vf, ent = 0.2, 0.5, 0.01
    batch, keep = ob.make_batch(T, n, 0, n, L, T, **ro, clip=clip, vf=vf, ent=ent)
    total, l3 = ob.ppo_loss_f64(p, batch)
    adv = ro["adv"].astype(np.float64)
    mean = adv.mean()
    std = np.sqrt(max((adv * adv).mean() - mean * mean, 0.0))
    A = (adv - np.float32(mean)) * (1.0 / (np.float32(std) + np.float32(1e-8)))
    ratio = np.exp(-np.log(ACTIONS) - ro["r_logprob"].astype(np.float64))
    pg = -np.minimum(ratio * A, np.clip(ratio, 1 - clip, 1 + clip) * A)
    assert (np.abs(ratio - 1) > clip).any() and (np.abs(ratio - 1) < clip).any()   # both branches
    vterm = 0.5 * (bv - ro["ret"].astype(np.float64)) ** 2
    want = np.array([pg.sum(), vterm.sum(), n * T * np.log(ACTIONS)])
    assert np.allclose(l3, want, rtol=1e-6, atol=1e-9), (l3, want)
    # the total is that combination of the three sums (the coefficients travel as fp32)
    assert abs(total - (l3[0] + float(np.float32(vf)) * l3[1] - float(np.float32(ent)) * l3[2]) / (n * T)) < 1e-12
    assert abs(total - (want[0] + vf * want[1] - ent * want[2]) / (n * T)) < 1e-7
    # the backward pass reports the same sums
    g, l3b = ob.ppo_backward_f64(p, batch)
    assert np.allclose(l3b, want, rtol=1e-6, atol=1e-9)
