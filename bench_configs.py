"""Timings of the secondary workloads on one MI355X, one JSON line each:

  forward_65536   policy forward, 65 536 envs, h256x3, one step from records
                  (fp32 and bf16-input kernels)
  ppo_update      PPO update, 4096 envs x 64 steps = 262 144 samples, one
                  minibatch = all envs: windowed recompute backward + Adam
  ppo_update_shapes    the update iteration (cfp_train_update, eager and graph) at
                  other horizons, env counts, minibatch and epoch settings
  rollout_policy_side  forward in recording mode + sampling + reward/done rows per
                  step at 4096 .. 262 144 envs (the policy half of cu_rollout_step)
  classic_1m      classic-game policy forward, 1 048 576 envs, 148-byte records
  record_kernels  the HBM-bound byte kernels at 65 536 envs: state -> 996-byte
                  records (fuzzed reference states of tests/golden, tiled) and
                  records -> fp32 features, and the unfused MinGRU gate/blend
                  epilogue of one layer
  stream_ceilings what plain library copies, fills and reads stream on the GPU
  env_step        the env on the device at 8192 / 65 536 / 262 144 envs: game step with the
                  envs' own random actions + world generation for finished envs (the
                  reference's "env only" figure, which also writes the observation
                  records), and the kernels one by one
  train_iteration  collect + update with everything on the device, samples/s
  rollout_in_the_loop  policy in the loop: record -> forward + sample -> env step ->
                  reward/done rows -> reset (cfp_env_rollout_step), steps per second

Usage:  python bench_configs.py [--reps 10] [--only NAME]
The headline workload (262 144 envs) is bench.py at the repository root."""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

PEAK_FP32 = 157.3                    # TFLOP/s, fp32 MFMA
FWD_FLOP = 1633792                   # per env-step: encoder + 3 gate GEMMs + head
UPD_FLOP = 4469248                   # per sample: recompute forward + backward
CLASSIC_FLOP = 1179648 + 9216        # gate GEMMs + 18-row head (gather encoder not counted)
# what the fp32 classic kernel issues per env: the above plus 3 K blocks of scalar features on the
# fp32 pipe, and 83 K blocks of 16 cell features x 256 units x 3 bf16 terms on the bf16 pipe
CLASSIC_ISSUE_FP32 = CLASSIC_FLOP + 24 * 256 * 2
CLASSIC_ISSUE_BF16 = 83 * 16 * 256 * 2 * 3
PEAK_BF16 = 2500.0


def _time(torch, fn, reps, warm=2, warm_ms=80.0):
    """Mean milliseconds of fn over reps calls (HIP events), after at least `warm` calls
    and `warm_ms` of untimed work: the shader clock needs some tens of milliseconds of
    load to rise from idle to its steady value, and a few short launches timed before
    that read 10-25 % slow."""
    import time
    t0, calls = time.perf_counter(), 0
    while calls < warm or (time.perf_counter() - t0) * 1e3 < warm_ms:
        fn()
        calls += 1
        if calls % 4 == 0:
            torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def forward_65536(pkg, torch, reps):
    """Second baseline configuration: 65 536 envs, one step, prior state N(0, 0.5); from
    records (fused kernel, fp32 and bf16-input) and from the fp32 feature matrix as the
    configuration states it (encoder GEMM of the seam + fused layers and heads)."""
    n = 65536
    pol = pkg.Policy(n, 3, seed=1)
    rec = pkg.policy.synth_records(n, 1234, 0)
    term = torch.zeros(n, device="cuda")
    av = torch.empty(n, 44, device="cuda")
    st0 = torch.randn(3, n, 256, device="cuda") * 0.5
    state = st0.clone()
    out = {"workload": "forward_65536", "envs": n}

    def rate(ms):
        return {"ms_per_step": ms, "env_steps_per_s": n / ms * 1e3, "tflops": FWD_FLOP * n / ms / 1e9,
                "frac_fp32_mfma_peak": FWD_FLOP * n / ms / 1e9 / PEAK_FP32}
    for name, on in (("fp32", False), ("bf16_in", True)):
        pol.set_gemm_bf16(on)
        state.copy_(st0)
        out[name] = rate(_time(torch, lambda: pol.forward(rec, term, state, av=av), reps))
    pol.set_gemm_bf16(False)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.where(torch.rand(n, 843, device="cuda", generator=g) < 0.6,
                    torch.randint(0, 41, (n, 843), device="cuda", generator=g).float(),
                    torch.rand(n, 843, device="cuda", generator=g))
    state.copy_(st0)
    out["fp32_from_feature_matrix"] = rate(_time(torch, lambda: pol.forward_features(x, term, state, av=av), reps))
    h = torch.empty(n, 256, device="cuda")
    W = pol.params[: 843 * 256].view(843, 256)
    out["fp32_from_feature_matrix"]["encoder_gemm_ms"] = _time(
        torch, lambda: pkg.policy.gemm_enc_fwd(W, x, h), reps)
    pol.close()
    return out


def ppo_update(pkg, torch, reps):
    n, T = 4096, 64
    pol = pkg.Policy(n, 3, seed=1)
    tr = pkg.Trainer(pol, T)
    pol.state.zero_()
    term = torch.zeros(n, device="cuda")
    for t in range(T):
        tr.record_step(t, pkg.policy.synth_records(n, 1234, t), term)
    g = torch.Generator(device="cuda").manual_seed(7)
    tr.buf("r_act").copy_(torch.randint(0, 43, (T, n), device="cuda", generator=g, dtype=torch.int32))
    tr.buf("r_logprob").fill_(-3.7612)          # -log 43: a uniform behaviour policy
    tr.buf("adv").copy_(torch.randn(T, n, device="cuda", generator=g))
    tr.buf("ret").copy_(torch.randn(T, n, device="cuda", generator=g))
    tr.buf("r_done").zero_()
    tr.adv_stats()

    def step():
        tr.backward(0, n)
        tr.adam()
    ms = _time(torch, step, reps, warm=1)
    ms_bwd = _time(torch, lambda: tr.backward(0, n), reps, warm=1)
    tr.adam()
    samples = n * T
    out = {"workload": "ppo_update", "envs": n, "T": T, "samples": samples,
           "window": tr.window, "ms_per_update": ms, "ms_backward": ms_bwd,
           "samples_per_s": samples / ms * 1e3,
           "tflops": UPD_FLOP * samples / ms / 1e9,
           "frac_fp32_mfma_peak": UPD_FLOP * samples / ms / 1e9 / PEAK_FP32}
    # same update with the GEMMs as fp32 MFMA (mode 0) and as six partial products (mode 2)
    for mode, key in ((0, "fp32_mfma_gemms"), (2, "split6_gemms"), (3, "split8_gemms")):
        pkg.policy.set_gemm_split(mode)
        try:
            ms_m = _time(torch, step, reps, warm=1)
        finally:
            pkg.policy.set_gemm_split(1)
        out[key] = {"ms_per_update": ms_m, "samples_per_s": samples / ms_m * 1e3,
                    "tflops": UPD_FLOP * samples / ms_m / 1e9}
    pkg.policy.set_gemm_bf16(True)       # same update with bf16 GEMM inputs
    try:
        ms16 = _time(torch, step, reps, warm=1)
        tr.set_bf16_storage(True)        # ... and the window workspace stored as bf16
        ms16s = _time(torch, step, reps, warm=1)
    finally:
        tr.set_bf16_storage(False)
        pkg.policy.set_gemm_bf16(False)
    out["bf16_in"] = {"ms_per_update": ms16, "samples_per_s": samples / ms16 * 1e3,
                      "tflops": UPD_FLOP * samples / ms16 / 1e9}
    out["bf16_in_bf16_storage"] = {"ms_per_update": ms16s, "samples_per_s": samples / ms16s * 1e3,
                                   "tflops": UPD_FLOP * samples / ms16s / 1e9}
    assert torch.isfinite(pol.params).all()
    tr.close()
    # ... and the r_state slab as bf16 too (cfp_train_set_bf16_rstate): written by the bf16-input
    # forward of the rollout, so the slab is recorded again in that mode
    pol.set_gemm_bf16(True)
    tr = pkg.Trainer(pol, T)
    tr.set_bf16_rstate(True)
    pol.state.zero_()
    for t in range(T):
        tr.record_step(t, pkg.policy.synth_records(n, 1234, t), term)
    tr.buf("r_act").copy_(torch.randint(0, 43, (T, n), device="cuda", generator=g, dtype=torch.int32))
    tr.buf("r_logprob").fill_(-3.7612)
    tr.buf("adv").copy_(torch.randn(T, n, device="cuda", generator=g))
    tr.buf("ret").copy_(torch.randn(T, n, device="cuda", generator=g))
    tr.buf("r_done").zero_()
    tr.adv_stats()
    pkg.policy.set_gemm_bf16(True)
    tr.set_bf16_storage(True)
    try:
        def step16():
            tr.backward(0, n)
            tr.adam()
        ms16r = _time(torch, step16, reps, warm=1)
    finally:
        pkg.policy.set_gemm_bf16(False)
        pol.set_gemm_bf16(False)
    out["bf16_in_bf16_storage_bf16_rstate"] = {"ms_per_update": ms16r, "samples_per_s": samples / ms16r * 1e3,
                                               "tflops": UPD_FLOP * samples / ms16r / 1e9}
    tr.close()
    pol.close()
    return out


def ppo_update_shapes(pkg, torch, reps):
    """cfp_train_update (epochs x minibatches x (backward, Adam)) at other shapes than
    config 4, eager and as the library's captured graph."""
    out = {"workload": "ppo_update_shapes", "shapes": []}
    for n, T, cfg in ((4096, 128, {}), (8192, 64, {}), (4096, 64, {"minibatches": 4}),
                      (1024, 128, {"epochs": 2}), (4096, 64, {"bptt_split": 4})):
        pol = pkg.Policy(n, 3, seed=1)
        tr = pkg.Trainer(pol, T, **cfg)
        pol.state.zero_()
        term = torch.zeros(n, device="cuda")
        for t in range(T):
            tr.record_step(t, pkg.policy.synth_records(n, 1234, t), term)
        g = torch.Generator(device="cuda").manual_seed(7)
        tr.buf("r_act").copy_(torch.randint(0, 43, (T, n), device="cuda", generator=g, dtype=torch.int32))
        tr.buf("r_logprob").fill_(-3.7612)
        tr.buf("adv").copy_(torch.randn(T, n, device="cuda", generator=g))
        tr.buf("ret").copy_(torch.randn(T, n, device="cuda", generator=g))
        tr.buf("r_done").zero_()
        tr.adv_stats()
        row = {"envs": n, "T": T, **cfg, "window": tr.window, "minibatch": tr.mb}
        for key, use_graph in (("eager", False), ("graph", True)):
            ms = _time(torch, lambda: tr.update(use_graph=use_graph), max(2, reps // 3), warm=1)
            row[key] = {"ms_per_iteration": ms,
                        "samples_per_s": n * T * cfg.get("epochs", 1) / ms * 1e3}
        assert torch.isfinite(pol.params).all()
        out["shapes"].append(row)
        tr.close()
        pol.close()
    return out


def rollout_policy_side(pkg, torch, reps):
    """The policy half of the reference's rollout step (cu_rollout_step + k_record_rd):
    record -> fused forward on the live state with the r_obs / r_state rows written ->
    categorical sampling (Philox) into r_act / r_logprob / r_value and the env's action
    slots -> reward/done rows; T = 8 steps per round of slabs, state carried.  The env
    step itself is not part of this library."""
    out = {"workload": "rollout_policy_side", "steps_per_round": 8, "sizes": {}}
    T = 8
    for n in (4096, 8192, 65536, 262144):
        pol = pkg.Policy(n, 3, seed=1)
        tr = pkg.Trainer(pol, T)
        # as in the reference, the records of step t are produced straight into the slab
        # row r_obs[t] (k_record_obs writes there), so the step makes no copy of them
        r_obs = tr.buf("r_obs")
        recs = [pkg.policy.synth_records(n, 99, t, rec=r_obs[t]) for t in range(T)]
        term = (torch.rand(n, device="cuda") < 0.0025).float()
        rew = torch.rand(n, device="cuda")
        acts = torch.empty(n, device="cuda")
        r_rew, r_done = tr.buf("r_reward"), tr.buf("r_done")

        def round_():
            for t in range(T):
                tr.rollout_step(t, recs[t], term, 1234, env_actions=acts)
                pkg.policy.record_rd(rew, term, r_rew[t], r_done[t])
        ms = _time(torch, round_, max(2, reps // 2), warm=1) / T
        out["sizes"][str(n)] = {"ms_per_step": ms, "env_steps_per_s": n / ms * 1e3,
                                "frac_fp32_mfma_peak": FWD_FLOP * n / ms / 1e9 / PEAK_FP32}
        # the same round with the bf16-input forward kernel (cfp_policy_set_gemm_bf16)
        pol.set_gemm_bf16(True)
        ms_b = _time(torch, round_, max(2, reps // 2), warm=1) / T
        pol.set_gemm_bf16(False)
        out["sizes"][str(n)]["bf16_in"] = {"ms_per_step": ms_b, "env_steps_per_s": n / ms_b * 1e3}
        if n <= 8192:
            # 16-env tiles (opt-in): twice the CUs at work at these sizes
            pol.set_small_tiles(True)
            ms_t = _time(torch, round_, max(2, reps // 2), warm=1) / T
            st = pol.state.clone()
            av = torch.empty(n, 44, device="cuda")
            ms_f = _time(torch, lambda: pol.forward(recs[0], term, st, av=av), reps)
            pol.set_small_tiles(False)
            ms_f32 = _time(torch, lambda: pol.forward(recs[0], term, st, av=av), reps)
            out["sizes"][str(n)]["small_tiles"] = {
                "ms_per_step": ms_t, "env_steps_per_s": n / ms_t * 1e3,
                "frac_fp32_mfma_peak": FWD_FLOP * n / ms_t / 1e9 / PEAK_FP32,
                "forward_only_ms": ms_f, "forward_only_ms_32_env_tiles": ms_f32}
            # the same round captured once into a graph and replayed, as the reference does
            # with its rollout (the device step counter keeps the draws fresh)
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    round_()
                ms_g = _time(torch, graph.replay, max(2, reps // 2), warm=1) / T
            out["sizes"][str(n)]["graph_replay_ms_per_step"] = ms_g
            del graph
        tr.close()
        pol.close()
    return out


def classic_1m(pkg, torch, reps):
    n = 1 << 20
    pol = pkg.Policy(n, 3, seed=1, variant="classic")
    rec = pkg.policy.synth_classic_records(n, 1234, 0)
    term = torch.zeros(n, device="cuda")
    av = torch.empty(n, 18, device="cuda")
    out = {"workload": "classic_1m", "envs": n}
    for name, on in (("fp32", False), ("bf16_in", True)):
        pol.set_gemm_bf16(on)
        ms = _time(torch, lambda: pol.forward(rec, term, pol.state, av=av), reps)
        out[name] = {"ms_per_step": ms, "env_steps_per_s": n / ms * 1e3,
                     "mfma_tflops": CLASSIC_FLOP * n / ms / 1e9,
                     "frac_fp32_mfma_peak": CLASSIC_FLOP * n / ms / 1e9 / PEAK_FP32}
    bound_ms = (CLASSIC_ISSUE_FP32 / PEAK_FP32 + CLASSIC_ISSUE_BF16 / PEAK_BF16) * n / 1e9
    out["fp32"]["mixed_pipe_bound_ms"] = bound_ms
    out["fp32"]["frac_of_mixed_pipe_bound"] = bound_ms / out["fp32"]["ms_per_step"]
    pol.close()
    return out


def record_kernels(pkg, torch, reps):
    import numpy as np
    n = 65536
    root = os.path.dirname(os.path.abspath(__file__))
    g = np.load(os.path.join(root, "tests", "golden", "record_fixtures.npz"))
    sc, pl = g["fuzz_scalars"], g["fuzz_planes"]          # [384][S], [384][3][2304]
    idx = np.arange(n) % sc.shape[0]
    scalars = torch.from_numpy(np.ascontiguousarray(sc[idx])).cuda()
    planes = torch.from_numpy(np.ascontiguousarray(pl[idx])).cuda().view(-1)
    plane = pl.shape[2]
    rec = torch.empty(n, 996, dtype=torch.uint8, device="cuda")
    xobs = torch.empty(n, 843, device="cuda")
    P = pkg.policy
    ms_r = _time(torch, lambda: P.record_obs(scalars, planes, planes[plane:], planes[2 * plane:],
                                             n, 3 * plane, 0, rec=rec), reps)
    ms_x = _time(torch, lambda: P.expand_obs(rec, n, xobs=xobs), reps)
    # the same records from the reference's per-field device arrays (cfp_record_obs_soa): the
    # fixture states scattered into [sub_index][env] arrays, mobs at the player's level
    s32 = torch.from_numpy(np.ascontiguousarray(sc[idx]).view(np.int32).copy()).cuda()
    names = ["player_position", "player_level", "player_direction", "player_health", "player_food",
             "player_drink", "player_energy", "player_mana", "player_xp", "player_dexterity",
             "player_strength", "player_intelligence", "is_sleeping", "is_resting", "inv_wood",
             "inv_stone", "inv_coal", "inv_iron", "inv_diamond", "inv_sapphire", "inv_ruby",
             "inv_sapling", "inv_torches", "inv_arrows", "inv_books", "inv_pickaxe", "inv_sword",
             "inv_bow", "inv_potions", "inv_armour", "sword_enchantment", "bow_enchantment",
             "armour_enchantments", "light_level", "learned_spells"]
    arrays, w = {}, 0
    kinds = dict(P.ENV_SOA_FIELDS)
    for name in names:
        k = kinds[name]
        cols = s32[:, w:w + k].t().contiguous()
        if name in ("player_health", "light_level"):
            cols = cols.view(torch.float32)
        elif name in ("is_sleeping", "is_resting", "learned_spells"):
            cols = (cols != 0).to(torch.uint8)
        arrays[name] = cols
        w += k
    level = s32[:, 2].clamp(0, 8).long()
    env = torch.arange(n, device="cuda")
    mk = torch.zeros(9, n, dtype=torch.int32, device="cuda")
    mk[level, env] = s32[:, w]
    arrays["monsters_killed"] = mk
    arrays["boss_timesteps_to_spawn_this_round"] = s32[:, w + 1].contiguous()
    w += 2
    mt = torch.zeros(135, n, dtype=torch.int32, device="cuda")
    mm = torch.zeros(135, n, dtype=torch.uint8, device="cuda")
    mp = torch.zeros(270, n, dtype=torch.int32, device="cuda")
    first, cls = (0, 3, 6, 8, 11), (0, 0, 0, 1, 1, 1, 2, 2, 3, 3, 3, 4, 4, 4)
    for m in range(14):
        cfm = (cls[m] * 9 + level) * 3 + (m - first[cls[m]])
        mt[cfm, env] = s32[:, w + m]
        mm[cfm, env] = (s32[:, w + 14 + m] != 0).to(torch.uint8)
        mp[2 * cfm, env] = s32[:, w + 28 + 2 * m]
        mp[2 * cfm + 1, env] = s32[:, w + 28 + 2 * m + 1]
    arrays.update(mob_type_id=mt, mob_mask=mm, mob_position=mp)
    rec2 = torch.empty_like(rec)
    ms_s = _time(torch, lambda: P.record_obs_soa(arrays, n, planes, planes[plane:], planes[2 * plane:],
                                                 n, 3 * plane, 0, rec=rec2), reps)
    assert torch.equal(rec, rec2), "records from the field arrays differ from the staged form"
    # the unfused gate/blend epilogue of one MinGRU layer (k_mingru_epi_fwd), recording form
    pre = torch.randn(n, 768, device="cuda")
    xin = torch.randn(n, 256, device="cuda")
    state = torch.randn(n, 256, device="cuda") * 0.5
    rs = torch.empty(n, 256, device="cuda")
    hout = torch.empty(n, 256, device="cuda")
    term = torch.zeros(n, device="cuda")
    ms_e = _time(torch, lambda: P.mingru_epi_fwd(pre, xin, state, term, r_state_store=rs,
                                                 h_out=hout), reps)
    b_e = 4 + 256 * 4 * (3 + 1 + 1 + 3)     # terminal; pre(3), x, state in; h, state, r_state out
    # algorithmic bytes per env: scalars + 99 cells x 3 plane bytes gathered + 996 written;
    # 996 read + 843 x 4 written
    b_r, b_x = sc.shape[1] + 99 * 3 + 996, 996 + 843 * 4
    return {"workload": "record_kernels", "envs": n,
            "record_obs": {"ms": ms_r, "envs_per_s": n / ms_r * 1e3, "bytes_per_env": b_r,
                           "gb_per_s": b_r * n / ms_r / 1e6, "frac_hbm_peak": b_r * n / ms_r / 1e6 / 8000},
            "record_obs_soa": {"ms": ms_s, "envs_per_s": n / ms_s * 1e3},
            "expand_obs": {"ms": ms_x, "envs_per_s": n / ms_x * 1e3, "bytes_per_env": b_x,
                           "gb_per_s": b_x * n / ms_x / 1e6, "frac_hbm_peak": b_x * n / ms_x / 1e6 / 8000},
            "mingru_epi_fwd": {"ms": ms_e, "envs_per_s": n / ms_e * 1e3, "bytes_per_env": b_e,
                               "gb_per_s": b_e * n / ms_e / 1e6,
                               "frac_hbm_peak": b_e * n / ms_e / 1e6 / 8000}}


def stream_ceilings(pkg, torch, reps):
    """What plain library kernels stream on this GPU (1 GiB operands, far beyond every
    cache): the yardstick for the HBM-bound kernels of the update next to the
    published 8 TB/s.  Rates count bytes read plus bytes written."""
    n = 1 << 28                                           # floats: 1 GiB
    a = torch.randn(n, device="cuda")
    b = torch.randn(n, device="cuda")
    c = torch.empty(n, device="cuda")
    gib = n * 4
    out = {"workload": "stream_ceilings", "bytes_per_operand": gib}
    for name, fn, moved in (("copy_1r_1w", lambda: c.copy_(a), 2 * gib),
                            ("fill_1w", lambda: c.fill_(1.0), gib),
                            ("sum_1r", lambda: a.sum(), gib),
                            ("add_2r_1w", lambda: torch.add(a, b, out=c), 3 * gib)):
        ms = _time(torch, fn, reps)
        out[name] = {"ms": ms, "tb_per_s": moved / ms / 1e9}
    del a, b, c
    # one of this library's own streaming kernels at a size far beyond the last-level cache:
    # the unfused MinGRU epilogue (5 rows read, 3 written per env and layer) at 262 144 envs
    n_env = 262144
    pre = torch.randn(n_env, 768, device="cuda")
    xin = torch.randn(n_env, 256, device="cuda")
    state = torch.randn(n_env, 256, device="cuda") * 0.5
    rs = torch.empty(n_env, 256, device="cuda")
    hout = torch.empty(n_env, 256, device="cuda")
    term = torch.zeros(n_env, device="cuda")
    ms = _time(torch, lambda: pkg.policy.mingru_epi_fwd(pre, xin, state, term, r_state_store=rs,
                                                        h_out=hout), reps)
    out["mingru_epi_fwd_5r_3w_262144_envs"] = {"ms": ms, "tb_per_s": 8196 * n_env / ms / 1e9}
    return out


def env_step(pkg, torch, reps):
    """Env-only steps per second, as the reference's `bench` mode counts them (random
    actions, auto-reset and observation encode included; README.md:27-52)."""
    out = {"workload": "env_step", "envs": {}}
    iters = max(20, 10 * reps)
    for n in (8192, 65536, 262144):
        env = pkg.Env(n)
        env.init(0)
        rec = torch.empty(n, 996, dtype=torch.uint8, device="cuda")

        def full():
            env.step(None)
            env.reset()
            env.record_obs(rec)

        def play():
            env.step(None)
            env.reset()

        for _ in range(300):          # spread the episodes' phases before timing
            full()
        torch.cuda.synchronize()
        ms_full = _time(torch, full, iters)
        ms_play = _time(torch, play, iters)
        cnt, _ = env.reset_list()
        out["envs"][str(n)] = {
            "us_per_step_all": round(ms_full * 1e3, 1), "M_env_steps_per_s": round(n / ms_full / 1e3, 1),
            "us_step_and_reset": round(ms_play * 1e3, 1), "M_env_steps_per_s_without_records": round(n / ms_play / 1e3, 1),
            "finished_envs_last_step": cnt,
        }
        env.close()
    return out


def rollout_in_the_loop(pkg, torch, reps):
    """cu_rollout_step with everything on the device (the reference's `run` mode,
    craftax_full.cu:12127-12176): h256x3 policy in the loop.  Steady state: 300 random-action
    steps first, so that the episodes' phases are spread and a step regenerates its share of
    finished envs (about 0.3 % of them); `fresh_worlds` regenerates those from their reset keys
    (k_reset_list), `reset_pool` copies them from a pool of 4096 worlds (the reference's pooled
    reset, craftax_full.c:3738-3741)."""
    out = {"workload": "rollout_in_the_loop", "policy": "h256x3 fp32", "envs": {}}
    T = 8
    for n in (1024, 4096, 8192, 65536, 262144):
        res = {}
        for mode, pool in (("fresh_worlds", 0), ("reset_pool", 4096)):
            env = pkg.Env(n, pool=pool)
            env.init(0)
            if pool:
                env.pool_fill(99)
            for _ in range(300):
                env.step(None)
                env.reset_from_pool() if pool else env.reset()
            pol = pkg.Policy(n, layers=3, seed=1)
            if n <= 4096:
                pol.set_small_tiles(True)
            tr = pkg.Trainer(pol, T)
            state = {"t": 0}

            def step():
                env.rollout_step(tr, state["t"] % T, 1234)
                state["t"] += 1

            ms = _time(torch, step, 64)
            cnt, _ = env.reset_list()
            res[mode] = {"us_per_step": round(ms * 1e3, 1), "M_env_steps_per_s": round(n / ms / 1e3, 2),
                         "frac_fp32_peak_of_forward_flops": round(FWD_FLOP * n / (ms * 1e-3) / 1e12 / PEAK_FP32, 3),
                         "finished_envs_last_step": cnt}
            # the same step without the trainer's slabs: cu_rollout_step_plain, what the reference's
            # `run` mode times (craftax_full.cu:12089-12092, 12127-12176)
            ms_run = _time(torch, lambda: env.run_step(pol, 1234), 64)
            res[mode]["run_mode"] = {"us_per_step": round(ms_run * 1e3, 1), "M_env_steps_per_s": round(n / ms_run / 1e3, 2),
                                     "frac_fp32_peak_of_forward_flops": round(FWD_FLOP * n / (ms_run * 1e-3) / 1e12 / PEAK_FP32, 3)}
            if n <= 8192:   # ... and replayed from a graph of one step (the reference's graph = 1)
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        env.run_step(pol, 1234)
                    ms_g = _time(torch, graph.replay, 64)
                torch.cuda.synchronize()
                res[mode]["run_mode"]["graph_replay_us_per_step"] = round(ms_g * 1e3, 1)
            tr.close()
            pol.close()
            env.close()
        out["envs"][str(n)] = res
    return out


def train_iteration(pkg, torch, reps):
    """One PPO iteration with everything on the device, as the reference's `train` mode counts
    it (README.md:348-356, horizon 128): cfp_train_collect (T rollout steps with the env, the
    bootstrap value, GAE) followed by cfp_train_update (backward + Adam, captured graph)."""
    out = {"workload": "train_iteration", "policy": "h256x3", "cases": {}}
    for n, T in ((1024, 128), (4096, 128), (8192, 128), (16384, 128), (65536, 128)):
        env = pkg.Env(n)
        env.init(0)
        for _ in range(300):          # spread the episodes' phases (random actions) before timing
            env.step(None)
            env.reset()
        pol = pkg.Policy(n, layers=3, seed=1)
        if n <= 4096:
            pol.set_small_tiles(True)
        tr = pkg.Trainer(pol, T)
        case = {}
        for mode in ("fp32", "bf16_in_bf16_storage", "bf16_in_bf16_storage_bf16_rstate"):
            bf = mode != "fp32"
            pol.set_gemm_bf16(bf)
            tr.set_gemm_mode(1 if bf else 0, 1)
            tr.set_bf16_storage(bf)
            tr.set_bf16_rstate(mode.endswith("rstate"))

            def it():
                env.collect(tr, 1234)
                tr.update(use_graph=True)
            ms = _time(torch, it, 3, warm=2)
            ms_c = _time(torch, lambda: env.collect(tr, 1234), 3, warm=1)
            case[mode] = {"ms_per_iteration": round(ms, 3), "ms_collect": round(ms_c, 3),
                          "ms_update": round(ms - ms_c, 3), "M_samples_per_s": round(n * T / ms / 1e3, 2)}
        tr.set_bf16_rstate(False)
        pol.set_gemm_bf16(False)
        assert torch.isfinite(pol.params).all()
        out["cases"][f"{n}x{T}"] = case
        tr.close()
        pol.close()
        env.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--only", default=None)
    args = ap.parse_args()
    import torch
    import __graft_entry__ as ge
    pkg = ge.load_package()
    assert torch.cuda.is_available(), "bench_configs.py needs a GPU"
    for fn in (forward_65536, ppo_update, ppo_update_shapes, rollout_policy_side, classic_1m,
               record_kernels, stream_ceilings, env_step, rollout_in_the_loop, train_iteration):
        if args.only and fn.__name__ != args.only:
            continue
        print(json.dumps(fn(pkg, torch, args.reps)), flush=True)


if __name__ == "__main__":
    main()
