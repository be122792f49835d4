"""GPU parity of the policy forward through the C ABI against the fp64 oracle.

Tolerance: 1e-4 relative (see parity_util.rel_err) for logits, values, hidden
states; record-typed work (synthetic records, expansion) is bit-exact."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import (ACTIONS, AV, HIDDEN, TOL_FP32, assert_close, expand_records,
                         random_params, rel_err, synth_records_host)

pytestmark = pytest.mark.gpu
L = 3


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def _check_all(out, ref, state_d, what):
    av = out["av"].cpu().numpy()
    errs = {
        "logits": assert_close(av[:, :ACTIONS], ref["logits"], TOL_FP32, what + " logits"),
        "values": assert_close(av[:, ACTIONS], ref["values"], TOL_FP32, what + " values"),
        "state": assert_close(state_d.cpu().numpy(), ref["state"], TOL_FP32, what + " state"),
    }
    for k in ("h_enc", "h3", "r_state"):
        if out.get(k) is not None:
            errs[k] = assert_close(out[k].cpu().numpy(), ref[k], TOL_FP32, f"{what} {k}")
    return errs


@pytest.mark.parametrize("n,layers,term_p", [(32, 3, 0.0), (96, 3, 0.3), (256, 2, 0.5),
                                             (64, 1, 1.0), (1024, 3, 0.1)])
def test_fused_forward_matches_oracle(pkg, cuda, n, layers, term_p):
    import torch
    params = random_params(layers, 100 + n)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    rng = np.random.default_rng(n)
    rec_h = synth_records_host(n, 5, n)
    state_h = (0.5 * rng.standard_normal((layers, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < term_p).astype(np.float32)
    ref = ob.forward_f64(params, layers, expand_records(rec_h), state_h, term_h)
    state = _t(state_h, cuda)
    out = {"h_enc": torch.zeros(n, HIDDEN, device=cuda), "h3": torch.zeros(n, HIDDEN, device=cuda),
           "r_state": torch.zeros(layers, n, HIDDEN, device=cuda)}
    out["av"] = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state, r_state_t=out["r_state"],
                            h_enc=out["h_enc"], h3=out["h3"])
    torch.cuda.synchronize()
    _check_all(out, ref, state, f"fused n={n} L={layers}")
    # post-zero state record is a copy / zero: exact
    assert np.array_equal(out["r_state"].cpu().numpy(),
                          ref["r_state"].astype(np.float32))
    pol.close()


def test_encoder_weight_split_is_exact(pkg, cuda):
    """The encoder multiplies the byte-valued features on the bf16 matrix pipe
    against a three-term bf16 split of each fp32 weight.  Weights whose three
    terms are all non-zero (1 + m*2^-10 + 2^-20), one 16-feature K block of ones
    per env and nothing else make every product and every partial sum exactly
    representable in fp32, so h_enc must equal the fp64 result (rounded once, when
    the bias is added) bit for bit: a
    dropped or misplaced term, block or unit column shows as a 2^-16 (or larger)
    difference.  The 51 fp32 tail features get the same treatment on their own
    envs (values 0.5, weights with 24 significant bits)."""
    import torch
    from parity_util import OBS, split_params
    n = 128
    params = np.zeros_like(random_params(L, 1))
    o = split_params(params, L)                      # views into params
    u = np.arange(HIDDEN)
    f = np.arange(OBS)[:, None]
    o["W_enc"][:] = (1.0 + (1 + (u[None, :] + f) % 4) * 2.0 ** -10 + 2.0 ** -20).astype(np.float32)
    o["W_enc"][792:] = (1.0 + 2.0 ** -12 + 2.0 ** -23) * (1 + (u[None, :] % 3))
    o["b_enc"][:] = (u % 7).astype(np.float32)
    assert np.array_equal(o["W_enc"].astype(np.float64),
                          np.float64(o["W_enc"]))     # fp32 values, exactly
    rec = np.zeros((n, 996), np.uint8)
    tail = np.zeros((n, 51), np.float32)
    for e in range(n):
        if e < 100:                                   # map K blocks 0..49, twice (ones, then threes)
            kb = e % 50
            rec[e, 16 * kb:min(16 * kb + 16, 792)] = 1 if e < 50 else 3
        else:                                         # tail features in groups of 4
            j = min((e - 100) * 2, 47)
            tail[e, j:j + 4] = 0.5
    rec[:, 792:] = tail.view(np.uint8).reshape(n, 204)
    pol = pkg.Policy(n, L, seed=1)
    pol.set_params(params)
    h = pol.encode_step(_t(rec, cuda)).cpu().numpy()
    x64 = expand_records(rec).astype(np.float64)
    dot = x64 @ o["W_enc"].astype(np.float64)
    assert np.array_equal(dot.astype(np.float32).astype(np.float64), dot)   # sums representable
    want = (dot + o["b_enc"].astype(np.float64)).astype(np.float32)         # one rounding: + bias
    bad = np.nonzero(h != want)
    assert bad[0].size == 0, f"{bad[0].size} entries differ, first env {bad[0][:4]} unit {bad[1][:4]}"
    pol.close()


def test_split_entry_points_match_fused_and_oracle(pkg, cuda):
    """cfp_encode_step + cfp_gru_chain + cfp_head == cfp_policy_forward == oracle."""
    import torch
    n = 160
    params = random_params(L, 7)
    pol = pkg.Policy(n, L, seed=1)
    pol.set_params(params)
    rng = np.random.default_rng(8)
    rec_h = synth_records_host(n, 9, 0)
    state_h = (0.5 * rng.standard_normal((L, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < 0.25).astype(np.float32)
    ref = ob.forward_f64(params, L, expand_records(rec_h), state_h, term_h)
    rec, term = _t(rec_h, cuda), _t(term_h, cuda)
    h_enc = pol.encode_step(rec).clone()
    st_a = _t(state_h, cuda)
    h3 = pol.gru_chain(h_enc, st_a, term)
    av_a = pol.head(h3)
    st_b = _t(state_h, cuda)
    av_b = pol.forward(rec, term, st_b)
    torch.cuda.synchronize()
    assert_close(h_enc.cpu().numpy(), ref["h_enc"], TOL_FP32, "encode_step h_enc")
    assert_close(h3.cpu().numpy(), ref["h3"], TOL_FP32, "gru_chain h3")
    assert_close(av_a.cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, "head logits")
    # same kernels, same order of operations: the split path is bitwise the fused one
    assert torch.equal(av_a, av_b) and torch.equal(st_a, st_b)
    pol.close()


def test_chunked_equals_unchunked(pkg, cuda):
    """Chunking only changes the launch grid (config: 16 x 16384 vs one batch)."""
    import torch
    n = 512
    pol = pkg.Policy(n, L, seed=3)
    rec = pkg.policy.synth_records(n, 21, 0)
    term = torch.zeros(n, device=cuda)
    st_a = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    st_b = st_a.clone()
    av_a = pol.forward(rec, term, st_a, chunk=0)
    av_b = pol.forward(rec, term, st_b, chunk=128)
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_b) and torch.equal(st_a, st_b)
    pol.close()


def test_one_tile_per_workgroup_schedule_matches_pairs(pkg, cuda):
    """Batches of at most one tile per CU run one tile per workgroup (a layer's K
    phase, then its epilogue) instead of the two-tile interleave; the arithmetic per
    tile is the same, so the bits are.  16 384 envs in one launch take the pair
    schedule, the same envs in chunks of 4096 the single one; plain and recording."""
    import torch
    n = 16384
    pol = pkg.Policy(n, L, seed=4)
    rec = pkg.policy.synth_records(n, 31, 2)
    term = (torch.rand(n, device=cuda) < 0.1).float()
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    for record in (False, True):
        outs = []
        for chunk in (0, 4096):
            st = st0.clone()
            rs = torch.full_like(st0, 7.0) if record else None
            av = pol.forward(rec, term, st, r_state_t=rs, chunk=chunk).clone()
            torch.cuda.synchronize()
            outs.append((av, st, rs))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
        if record:
            assert torch.equal(outs[0][2], outs[1][2])
    pol.close()


def test_multi_step_carry_with_terminals(pkg, cuda):
    """16 consecutive steps carrying hidden state on device vs the oracle carrying
    it in fp64; state zeroed on the step after a terminal."""
    import torch
    n, T = 64, 16
    params = random_params(L, 31)
    pol = pkg.Policy(n, L, seed=1)
    pol.set_params(params)
    rng = np.random.default_rng(32)
    state = torch.zeros(L, n, HIDDEN, device=cuda)
    st64 = np.zeros((L, n, HIDDEN))
    worst = 0.0
    for t in range(T):
        rec_h = synth_records_host(n, 33, t)
        term_h = (rng.random(n) < 0.15).astype(np.float32) if t else np.zeros(n, np.float32)
        av = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state)
        ref = ob.forward_f64(params, L, expand_records(rec_h), st64, term_h)
        st64 = ref["state"]
        worst = max(worst, assert_close(av.cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32,
                                        f"step {t} logits"))
        assert_close(state.cpu().numpy(), st64, TOL_FP32, f"step {t} state")
    pol.close()


def test_reference_rollout_slice(pkg, cuda, golden):
    """Config 1 slice: real records of the reference C env (32 envs x 16 steps,
    committed fixture), weights from seed 1, zero initial state carried."""
    import torch
    recs, terms = golden["slice_records"], golden["slice_terminals"]
    T, n = terms.shape
    pol = pkg.Policy(n, L, seed=1)
    params = pol.get_params()
    state = pol.state
    st64 = np.zeros((L, n, HIDDEN))
    for t in range(T):
        av = pol.forward(_t(recs[t], cuda), _t(terms[t], cuda), state)
        ref = ob.forward_f64(params, L, expand_records(recs[t]), st64, terms[t])
        st64 = ref["state"]
        assert_close(av.cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, f"slice step {t} logits")
        assert_close(av.cpu().numpy()[:, ACTIONS], ref["values"], TOL_FP32, f"slice step {t} values")
    assert_close(state.cpu().numpy(), st64, TOL_FP32, "slice final state")
    pol.close()


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (no reference source)")
def test_config1_live_reference_env(pkg, cuda):
    """Config 1 in full on the box: the compiled reference env (1024 envs, seed 0,
    xorshift32 % 43 actions) feeds the device policy for 2000 steps, state carried and
    zeroed after terminals; during the first 200 steps every 20th step and every step
    with a terminal, afterwards every 50th step, is checked one-step against the
    oracle from the device's own state."""
    import torch
    n, T = 1024, 2000
    env = ob.RefEnv(n, 0)
    pol = pkg.Policy(n, L, seed=1)
    params = pol.get_params()
    state = pol.state
    n_term = 0
    try:
        for t in range(T):
            rec_h = env.records()
            term_h = env.terminals() if t else np.zeros(n, np.float32)
            n_term += int((term_h != 0).sum())
            check = (t % 20 == 0 or (term_h != 0).any()) if t < 200 else t % 50 == 0
            if check:
                st_in = state.cpu().numpy().copy()
            av = pol.forward(_t(rec_h, cuda), _t(term_h, cuda), state)
            if check:
                ref = ob.forward_f64(params, L, expand_records(rec_h), st_in, term_h)
                assert_close(av.cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, f"t={t} logits")
                assert_close(av.cpu().numpy()[:, ACTIONS], ref["values"], TOL_FP32, f"t={t} values")
                assert_close(state.cpu().numpy(), ref["state"], TOL_FP32, f"t={t} state")
            env.step()
        assert n_term > 0, "no episode ended: the terminal path was not exercised"
    finally:
        env.close()
        pol.close()


def test_full_size_properties(pkg, cuda):
    """At the benchmark's full size (262 144 envs) the oracle is too slow; use
    size-independent properties: (i) envs are independent, so a sampled subset
    run alone reproduces its rows bit for bit; (ii) a checksum of the sampled
    rows matches the oracle; (iii) chunked == unchunked."""
    import torch
    n = 262144
    pol = pkg.Policy(n, L, seed=1)
    params = pol.get_params()
    rec = pkg.policy.synth_records(n, 77, 3)
    term = (torch.rand(n, device=cuda) < 0.05).float()
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    st_a = st0.clone()
    av_a = pol.forward(rec, term, st_a, chunk=0).clone()
    st_b = st0.clone()
    av_b = pol.forward(rec, term, st_b, chunk=16384)
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_b) and torch.equal(st_a, st_b)
    assert torch.isfinite(av_a).all()
    # sampled tiles (whole 32-env tiles, spread over the batch, incl. first/last)
    tiles = [0, 1, 4095, 4096, 8191, 5000, 2731]
    idx = torch.cat([torch.arange(t * 32, t * 32 + 32) for t in tiles]).to(cuda)
    sub_rec = rec[idx].contiguous(); sub_term = term[idx].contiguous()
    sub_st = st0[:, idx].contiguous()
    small = pkg.Policy(len(idx), L, seed=1)
    av_s = small.forward(sub_rec, sub_term, sub_st)
    torch.cuda.synchronize()
    assert torch.equal(av_s, av_a[idx]) and torch.equal(sub_st, st_a[:, idx])
    ref = ob.forward_f64(params, L, expand_records(sub_rec.cpu().numpy()),
                         st0[:, idx].cpu().numpy(), sub_term.cpu().numpy())
    assert_close(av_s.cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, "full-size sample logits")
    assert_close(sub_st.cpu().numpy(), ref["state"], TOL_FP32, "full-size sample state")
    small.close(); pol.close()


def _config2_features(n, cuda, seed):
    """The second baseline configuration's feature matrix: each entry an integer U{0..40}
    cast to float with probability 0.6, else U[0, 1)."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    ints = torch.randint(0, 41, (n, 843), generator=g).float()
    cont = torch.rand(n, 843, generator=g)
    pick = torch.rand(n, 843, generator=g) < 0.6
    return torch.where(pick, ints, cont).to(cuda)


def test_config2_feature_matrix_at_65536(pkg, cuda):
    """The second baseline configuration as stated: 65 536 envs, an fp32 feature matrix
    [65536][843] (60 % small integers, 40 % U[0,1) in every column), prior hidden state
    N(0, 0.5), one step, through cfp_policy_forward_features.  Sampled 32-env tiles
    (first, last, spread) against the fp64 oracle on the same rows; the whole batch is
    finite and reproduces, rows of the sampled tiles run alone give the same bits."""
    import torch
    n = 65536
    pol = pkg.Policy(n, L, seed=1)
    params = pol.get_params()
    x = _config2_features(n, cuda, 21)
    assert 0.35 < float((x != x.floor()).float().mean()) < 0.45
    term = torch.zeros(n, device=cuda)
    st0 = torch.randn(L, n, HIDDEN, device=cuda, generator=torch.Generator(device=cuda).manual_seed(22)) * 0.5
    st_a = st0.clone()
    h_enc = torch.empty(n, HIDDEN, device=cuda); h3 = torch.empty(n, HIDDEN, device=cuda)
    av_a = pol.forward_features(x, term, st_a, h_enc=h_enc, h3=h3).clone()
    st_b = st0.clone()
    av_b = pol.forward_features(x, term, st_b)
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_b) and torch.equal(st_a, st_b) and torch.isfinite(av_a).all()
    tiles = [0, 1, 2047, 1024, 777, 1500]
    idx = torch.cat([torch.arange(t * 32, t * 32 + 32) for t in tiles]).to(cuda)
    ref = ob.forward_f64(params, L, x[idx].cpu().numpy(), st0[:, idx].cpu().numpy(), None)
    assert_close(h_enc[idx].cpu().numpy(), ref["h_enc"], TOL_FP32, "config 2 h_enc")
    assert_close(av_a[idx].cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, "config 2 logits")
    assert_close(av_a[idx].cpu().numpy()[:, ACTIONS], ref["values"], TOL_FP32, "config 2 values")
    assert_close(st_a[:, idx].cpu().numpy(), ref["state"], TOL_FP32, "config 2 state")
    assert_close(h3[idx].cpu().numpy(), ref["h3"], TOL_FP32, "config 2 h3")
    # the sampled rows alone, as a batch of their own: the same bits
    st_c = st0[:, idx].contiguous().clone()
    h_c = torch.empty(idx.numel(), HIDDEN, device=cuda)
    av_c = torch.empty(idx.numel(), av_a.shape[1], device=cuda)
    pol.forward_features(x[idx].contiguous(), term[idx].contiguous(), st_c, h_enc=h_c, av=av_c)
    torch.cuda.synchronize()
    assert torch.equal(av_c, av_a[idx]) and torch.equal(st_c, st_a[:, idx]) and torch.equal(h_c, h_enc[idx])
    pol.close()


def test_config2_records_at_65536(pkg, cuda):
    """The record-typed equivalent of the second configuration on the fused kernel:
    65 536 envs of synthetic records, prior state N(0, 0.5), sampled tiles against the
    fp64 oracle; rows of a sampled tile run alone reproduce bit for bit."""
    import torch
    n = 65536
    pol = pkg.Policy(n, L, seed=1)
    params = pol.get_params()
    rec = pkg.policy.synth_records(n, 31, 0)
    term = torch.zeros(n, device=cuda)
    st0 = torch.randn(L, n, HIDDEN, device=cuda, generator=torch.Generator(device=cuda).manual_seed(32)) * 0.5
    st = st0.clone()
    av = pol.forward(rec, term, st).clone()
    torch.cuda.synchronize()
    tiles = [0, 2047, 1023, 311, 1999]
    idx = torch.cat([torch.arange(t * 32, t * 32 + 32) for t in tiles]).to(cuda)
    ref = ob.forward_f64(params, L, expand_records(rec[idx].cpu().numpy()), st0[:, idx].cpu().numpy(), None)
    assert_close(av[idx].cpu().numpy()[:, :ACTIONS], ref["logits"], TOL_FP32, "config 2 (records) logits")
    assert_close(av[idx].cpu().numpy()[:, ACTIONS], ref["values"], TOL_FP32, "config 2 (records) values")
    assert_close(st[:, idx].cpu().numpy(), ref["state"], TOL_FP32, "config 2 (records) state")
    small = pkg.Policy(len(idx), L, seed=1)
    sub_st = st0[:, idx].contiguous()
    av_s = small.forward(rec[idx].contiguous(), term[idx].contiguous(), sub_st)
    torch.cuda.synchronize()
    assert torch.equal(av_s, av[idx]) and torch.equal(sub_st, st[:, idx])
    small.close(); pol.close()


def test_forward_is_bitwise_reproducible_under_memory_pressure(pkg, cuda):
    """The kernel waits for its LDS-direct weight loads by counting its own vector
    memory operations; a miscount would read a ring slot before it has landed, and
    what it reads then depends on timing.  Same inputs, three runs -- one alone, two
    racing a large device copy on another stream -- must agree bit for bit, for the
    plain, the r_state-recording and the classic kernels."""
    import torch
    n = 65536
    side = torch.cuda.Stream()
    big = torch.empty(1 << 28, dtype=torch.uint8, device=cuda)
    for variant in ("full", "classic"):
        pol = pkg.Policy(n, L, seed=5, variant=variant)
        rec = (pkg.policy.synth_classic_records(n, 3, 1) if variant == "classic"
               else pkg.policy.synth_records(n, 3, 1))
        term = (torch.rand(n, device=cuda) < 0.1).float()
        st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
        outs = []
        for run in range(3):
            st = st0.clone()
            rs = torch.zeros_like(st0) if run != 1 else None
            torch.cuda.synchronize()
            if run:
                with torch.cuda.stream(side):
                    for _ in range(4):
                        big[: 1 << 27].copy_(big[1 << 27:])
            av = pol.forward(rec, term, st, r_state_t=rs).clone()
            torch.cuda.synchronize()
            outs.append((av, st))
        for av, st in outs[1:]:
            assert torch.equal(av, outs[0][0]) and torch.equal(st, outs[0][1]), variant
        pol.close()


def test_small_tiles_are_bitwise_reproducible_under_memory_pressure(pkg, cuda):
    """The same guard for the 16-env-tile kernel, whose weight ring is waited for with
    counted s_waitcnt as well: plain and r_state-recording forms at 4096 envs (all 256
    CUs), one run alone and two racing a large device copy."""
    import torch
    n = 4096
    side = torch.cuda.Stream()
    big = torch.empty(1 << 28, dtype=torch.uint8, device=cuda)
    pol = pkg.Policy(n, L, seed=5)
    pol.set_small_tiles(True)
    rec = pkg.policy.synth_records(n, 3, 1)
    term = (torch.rand(n, device=cuda) < 0.1).float()
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    for record in (False, True):
        outs = []
        for run in range(3):
            st = st0.clone()
            rs = torch.zeros_like(st0) if record else None
            h_enc = torch.zeros(n, HIDDEN, device=cuda)
            torch.cuda.synchronize()
            if run:
                with torch.cuda.stream(side):
                    for _ in range(2):
                        big[: 1 << 27].copy_(big[1 << 27:])
            av = pol.forward(rec, term, st, r_state_t=rs, h_enc=h_enc if run != 1 else None).clone()
            torch.cuda.synchronize()
            outs.append((av, st, rs))
        for av, st, rs in outs[1:]:
            assert torch.equal(av, outs[0][0]) and torch.equal(st, outs[0][1]), record
            if record:
                assert torch.equal(rs, outs[0][2])
    pol.close()


def test_error_paths_on_device(pkg, cuda):
    import torch
    pol = pkg.Policy(64, L, seed=1)
    rec = torch.zeros(48, 996, dtype=torch.uint8, device=cuda)     # 48 is not a multiple of 32
    with pytest.raises(pkg._lib.CfpError, match="multiple of 32"):
        pol.forward(rec, torch.zeros(48, device=cuda), torch.zeros(L, 48, HIDDEN, device=cuda))
    rec = torch.zeros(64 * 996 + 4, dtype=torch.uint8, device=cuda)[4:].view(64, 996)
    with pytest.raises(pkg._lib.CfpError, match="16-byte"):
        pol.forward(rec, torch.zeros(64, device=cuda), torch.zeros(L, 64, HIDDEN, device=cuda))
    with pytest.raises(pkg._lib.CfpError, match="param count"):
        pol.set_params(np.zeros(10, np.float32))
    pol.close()


@pytest.mark.parametrize("n,layers,term_p", [(32, 3, 0.0), (96, 3, 0.3), (1024, 3, 0.1), (64, 1, 1.0),
                                             (4096, 2, 0.05)])
def test_small_tiles_match_oracle(pkg, cuda, n, layers, term_p):
    """cfp_policy_set_small_tiles: the 16-env-tile kernel (16 x 16 matrix instructions, own
    weight mirrors) against the fp64 oracle, plain and recording; its r_state record is a
    copy / zero (exact); against the 32-env kernel it agrees to rounding but not in bits."""
    import torch
    params = random_params(layers, 300 + n)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    pol.set_small_tiles(True)
    rng = np.random.default_rng(n + 1)
    rec_h = synth_records_host(n, 6, n)
    state_h = (0.5 * rng.standard_normal((layers, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < term_p).astype(np.float32)
    k = min(n, 512)     # the oracle takes the first rows
    ref = ob.forward_f64(params, layers, expand_records(rec_h[:k]), state_h[:, :k], term_h[:k])
    rec, term = _t(rec_h, cuda), _t(term_h, cuda)
    for record in (False, True):
        state = _t(state_h, cuda)
        out = {"h_enc": torch.zeros(n, HIDDEN, device=cuda), "h3": torch.zeros(n, HIDDEN, device=cuda),
               "r_state": torch.zeros(layers, n, HIDDEN, device=cuda) if record else None}
        out["av"] = pol.forward(rec, term, state, r_state_t=out["r_state"], h_enc=out["h_enc"],
                                h3=out["h3"])
        torch.cuda.synchronize()
        sub = {key: (v[:k] if v.dim() == 2 else v[:, :k]) if v is not None else None for key, v in out.items()}
        _check_all(sub, ref, state[:, :k], f"small tiles n={n} L={layers} record={record}")
        if record:
            assert np.array_equal(out["r_state"].cpu().numpy()[:, :k], ref["r_state"].astype(np.float32))
        assert torch.isfinite(out["av"]).all()
    # the 32-env kernel on the same inputs: same result to rounding
    pol.set_small_tiles(False)
    state_b = _t(state_h, cuda)
    av_b = pol.forward(rec, term, state_b)
    torch.cuda.synchronize()
    assert rel_err(out["av"].cpu().numpy(), av_b.cpu().numpy().astype(np.float64)) < 1e-4
    assert rel_err(state.cpu().numpy(), state_b.cpu().numpy().astype(np.float64)) < 1e-4
    pol.close()


def test_small_tiles_leave_large_batches_alone(pkg, cuda):
    """Above 4096 envs the flag changes nothing: the 32-env kernels run and the bits are
    those of a policy without the flag."""
    import torch
    n = 16384
    pol = pkg.Policy(n, L, seed=2)
    rec = pkg.policy.synth_records(n, 41, 0)
    term = torch.zeros(n, device=cuda)
    st0 = torch.randn(L, n, HIDDEN, device=cuda) * 0.5
    sa = st0.clone(); av_a = pol.forward(rec, term, sa).clone()
    pol.set_small_tiles(True)
    sb = st0.clone(); av_b = pol.forward(rec, term, sb)
    torch.cuda.synchronize()
    assert torch.equal(av_a, av_b) and torch.equal(sa, sb)
    pol.close()
