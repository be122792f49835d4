"""The env step on the GPU (cfp_env_step) against the compiled reference env
(oracle/_ref: the reference's craftax_full.c, stepped env by env with the same actions):
every state field, reward, terminal flag and reset key after every step, bit for bit
(floats by bit pattern).  Resets are supplied: when an env finishes, the reference's
freshly generated state is uploaded, so world generation is not on this test's path.
Reference functions: craftax_gameplay_step_native and what it calls
(craftax_full.c:3798-3878, 4210-8225), c_step_gameplay (:3981-4011), k_step
(craftax_full.cu:8760-8779)."""
import numpy as np
import pytest
import torch

import env_bind as eb

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ref():
    try:
        return eb.Ref()
    except FileNotFoundError:
        pytest.skip("oracle/_ref/libcfref.so is not built")


def _compare(tag, final, mine, rew, rew_gpu, term, term_gpu):
    d = eb.diff_fields(final, mine)
    msg = []
    for f in d[:8]:
        idx = np.argwhere(final[f] != mine[f])
        msg.append(f"{f}{idx[0].tolist()}: ref {final[f][tuple(idx[0])]} gpu {mine[f][tuple(idx[0])]}")
    assert not d, f"{tag}: state fields differ: " + "; ".join(msg)
    assert np.array_equal(rew.view(np.uint32), rew_gpu.view(np.uint32)), f"{tag}: rewards differ"
    assert np.array_equal(term, term_gpu), f"{tag}: terminals differ"


def _rollout(pkg, ref, n, steps, seed, own_actions):
    ref.init(n, seed)
    env = pkg.Env(n)
    env.import_states(ref.export())
    assert not eb.diff_fields(ref.export(), env.export_states(eb.STATE_DTYPE)), "import/export round trip"
    if own_actions:
        env.seed_actions(seed)
    terminals_seen = 0
    for t in range(steps):
        act = ref.next_actions()
        final, rew, term, keys = ref.step(act)
        env.step(None if own_actions else torch.from_numpy(act).cuda())
        mine = env.export_states(eb.STATE_DTYPE)
        _compare(f"step {t}", final, mine, rew, env.rewards.cpu().numpy(), term, env.terminals.cpu().numpy())
        cnt, recs = env.reset_list()
        done = np.nonzero(term)[0]
        assert cnt == len(done)
        if cnt:
            order = np.argsort(recs[:, 0])
            assert np.array_equal(recs[order, 0], done)
            assert np.array_equal(recs[order, 1:].view(np.uint32), keys[done])
            fresh = ref.export(list(done))
            for k, e in enumerate(done):   # resets supplied by the reference
                env.import_states(fresh[k:k + 1], first=int(e))
            terminals_seen += cnt
    return terminals_seen


def test_env_step_matches_reference_256x600(pkg, cuda, ref):
    """256 envs x 600 steps with the reference's xorshift32 % 43 actions, seed 0."""
    seen = _rollout(pkg, ref, 256, 600, 0, own_actions=False)
    assert seen > 0   # the run went through episode ends


def test_env_step_with_a_half_empty_wavefront(pkg, cuda, ref):
    """Env counts are multiples of 32 like the reference's --envs (craftax_full.cu:11820): 96 envs
    are one full wavefront of the step kernel and one with 32 lanes, whose votes, shuffles and
    spawn passes run over the lanes that exist."""
    seen = _rollout(pkg, ref, 96, 300, 11, own_actions=False)
    assert seen > 0


def test_env_calls_reject_bad_arguments(pkg, cuda):
    """The reference exits on a bad --envs (craftax_full.cu:11820-11825); a library returns an
    error and says why.  No kernel is launched by any of these calls."""
    err = pkg._lib.CfpError
    for n in (0, -32, 33, 48):
        with pytest.raises(err, match="multiple of 32"):
            pkg.Env(n)
    with pytest.raises(err, match="negative"):
        pkg.Env(64, pool=-1)
    env = pkg.Env(64)
    states = np.zeros(4, eb.STATE_DTYPE)
    with pytest.raises(err, match="outside"):
        env.import_states(states, first=62)
    with pytest.raises(err, match="outside"):
        env.export_states(eb.STATE_DTYPE, first=60, count=8)
    with pytest.raises(err, match="without a reset pool"):
        env.reset_from_pool()
    with pytest.raises(err, match="without a reset pool"):
        env.pool_fill(0)
    pol = pkg.Policy(96, layers=1, seed=1)
    tr = pkg.Trainer(pol, 4)
    with pytest.raises(err, match="holds 64 envs"):
        env.rollout_step(tr, 0, 1)
    tr.close(); pol.close(); env.close()


def test_env_step_own_action_stream(pkg, cuda, ref):
    """The kernel's own xorshift32 % 43 stream (d_actions = NULL) is the reference's."""
    _rollout(pkg, ref, 64, 200, 7, own_actions=True)


def test_records_from_stepped_state(pkg, cuda, ref):
    """cfp_env_record_obs on the stepped device state equals the reference's own encoder
    on its state (craftax_encode_compact_observation, craftax_full.c:2830)."""
    import ctypes as C
    n = 128
    ref.init(n, 3)
    env = pkg.Env(n)
    env.import_states(ref.export())
    ref.lib.cfref_observations.restype = C.POINTER(C.c_uint8)
    for t in range(120):
        act = ref.next_actions()
        final, rew, term, keys = ref.step(act)
        env.step(torch.from_numpy(act).cuda())
        done = np.nonzero(term)[0]
        if len(done):
            fresh = ref.export(list(done))
            for k, e in enumerate(done):
                env.import_states(fresh[k:k + 1], first=int(e))
        if t % 10 == 9:
            rec = env.record_obs().cpu().numpy()
            want = np.ctypeslib.as_array(ref.lib.cfref_observations(), shape=(n, 996))
            assert np.array_equal(rec, want), f"records differ at step {t}"


def test_reset_from_pool(pkg, cuda, ref):
    """Envs on the reset list become copies of pool entry key0 % pool; the env key and
    the action stream survive (craftax_full.c:3738-3741)."""
    n, pool = 64, 8
    ref.init(n, 11)
    states = ref.export()
    env = pkg.Env(n, pool=pool)
    dying = states.copy()
    dying["player_health"][::3] = 0.05   # these die at the next damage or starve tick
    dying["player_food"][::3] = 0
    dying["player_drink"][::3] = 0
    dying["player_recover"][::3] = -15.0
    env.import_states(dying)
    env.import_pool(states[:pool])
    env.step(torch.zeros(n, dtype=torch.float32, device="cuda"))
    before = env.export_states(eb.STATE_DTYPE)
    cnt, recs = env.reset_list()
    assert cnt == len(range(0, n, 3))
    env.reset_from_pool()
    after = env.export_states(eb.STATE_DTYPE)
    hit = np.zeros(n, bool)
    for e, k0, _ in recs:
        hit[e] = True
        want = states[(int(k0) & 0xFFFFFFFF) % pool].copy()
        want["rng_key"] = before["rng_key"][e]
        assert not eb.diff_fields(want.reshape(1), after[e:e + 1]), f"env {e}"
    assert not eb.diff_fields(before[~hit], after[~hit])


def test_collect_with_the_env_on_the_device(pkg, cuda, ref):
    """cfp_train_collect (cu_train_collect, craftax_full.cu:12980-13016): policy and envs
    both on the device for T steps.  The stored actions are replayed through the reference
    env on the CPU; observations, rewards and done flags of every step must be the slabs',
    bit for bit, including envs that finish and are refilled from the reset pool."""
    import ctypes as C
    n, T, pool, seed = 64, 40, 4, 5
    ref.init(n, seed)
    states = ref.export()
    pool_states = states[8:8 + pool].copy()
    weak = states.copy()
    for e in range(0, n, 4):            # a quarter of the envs starve within the horizon
        weak["player_health"][e] = 1.0 + (e % 3)
        weak["player_food"][e] = 0
        weak["player_recover"][e] = -14.0 + (e % 5)
        ref.import_(e, weak[e])
    env = pkg.Env(n, pool=pool)
    env.import_states(weak)
    env.import_pool(pool_states)
    pol = pkg.Policy(n, layers=3, seed=1)
    tr = pkg.Trainer(pol, T)
    env.collect(tr, seed=1234)
    torch.cuda.synchronize()
    r_obs = tr.buf("r_obs").cpu().numpy()
    r_act = tr.buf("r_act").cpu().numpy()
    r_rew = tr.buf("r_reward").cpu().numpy()
    r_done = tr.buf("r_done").cpu().numpy()
    ref.lib.cfref_observations.restype = C.POINTER(C.c_uint8)
    ref.lib.cfref_encode.argtypes = [C.c_int, C.c_void_p]
    rec = np.zeros((n, 996), np.uint8)
    finished = 0
    for t in range(T):
        for e in range(n):
            ref.lib.cfref_encode(e, C.c_void_p(rec[e].ctypes.data))
        assert np.array_equal(rec, r_obs[t]), f"observations of step {t}"
        final, rew, term, keys = ref.step(r_act[t].astype(np.float32))
        assert np.array_equal(rew.view(np.uint32), r_rew[t].view(np.uint32)), f"rewards of step {t}"
        assert np.array_equal(term.astype(np.uint8), r_done[t]), f"done flags of step {t}"
        for e in np.nonzero(term)[0]:   # the device refilled these from the pool
            fresh = pool_states[int(keys[e, 0]) % pool].copy()
            fresh["rng_key"] = final["rng_key"][e]
            ref.import_(int(e), fresh)
            finished += 1
    assert finished >= 4
    mine = env.export_states(eb.STATE_DTYPE)
    assert not eb.diff_fields(ref.export(), mine), "states after the rollout"
    adv = tr.buf("adv").cpu().numpy()
    assert np.isfinite(adv).all() and np.abs(adv).max() > 0


def test_collect_regenerating_worlds(pkg, cuda, ref):
    """cfp_train_collect without a reset pool: finished envs are regenerated from their reset
    keys on the device.  Replayed through the reference env, which regenerates the same worlds
    from the same keys: every step's observations, rewards and done flags are the slabs', and
    the final states agree."""
    import ctypes as C
    n, T, seed = 96, 48, 9      # one and a half wavefronts of the step kernel, three tiles of the policy
    ref.init(n, seed)
    states = ref.export()
    weak = states.copy()
    for e in range(0, n, 3):            # a third of the envs starve within the horizon
        weak["player_health"][e] = 1.0 + (e % 4)
        weak["player_food"][e] = 0
        weak["player_drink"][e] = 0
        weak["player_recover"][e] = -14.0 + (e % 7)
        ref.import_(e, weak[e])
    env = pkg.Env(n)
    env.import_states(weak)
    pol = pkg.Policy(n, layers=3, seed=1)
    tr = pkg.Trainer(pol, T)
    env.collect(tr, seed=77)
    torch.cuda.synchronize()
    r_obs = tr.buf("r_obs").cpu().numpy()
    r_act = tr.buf("r_act").cpu().numpy()
    r_rew = tr.buf("r_reward").cpu().numpy()
    r_done = tr.buf("r_done").cpu().numpy()
    ref.lib.cfref_encode.argtypes = [C.c_int, C.c_void_p]
    rec = np.zeros((n, 996), np.uint8)
    finished = 0
    for t in range(T):
        for e in range(n):
            ref.lib.cfref_encode(e, C.c_void_p(rec[e].ctypes.data))
        assert np.array_equal(rec, r_obs[t]), f"observations of step {t}"
        final, rew, term, keys = ref.step(r_act[t].astype(np.float32))
        assert np.array_equal(rew.view(np.uint32), r_rew[t].view(np.uint32)), f"rewards of step {t}"
        assert np.array_equal(term.astype(np.uint8), r_done[t]), f"done flags of step {t}"
        finished += int(term.sum())
    assert finished >= 20
    assert not eb.diff_fields(ref.export(), env.export_states(eb.STATE_DTYPE)), "states after the rollout"
    tr.close(); pol.close()


def test_phase_timers_change_nothing_but_the_clock(pkg, cuda):
    """cfp_train_set_profile (the reference's CRAFTAX_CU_TRAIN_PROF, craftax_full.cu:12925):
    two trainers on equal envs and policies run the same iteration, one with the phase timers
    on (eager update with waits between the phases), one through the captured graph: slabs and
    parameters agree bit for bit, the four sums are positive and add up to no more than the
    wall time of the two calls, and a reset clears them."""
    import time
    n, T = 256, 8
    outs = []
    for timed in (False, True):
        env = pkg.Env(n)
        env.init(5)
        pol = pkg.Policy(n, layers=2, seed=3)
        tr = pkg.Trainer(pol, T)
        tr.set_profile(timed)
        assert tr.profile() == {"rollout": 0.0, "gae": 0.0, "backward": 0.0, "adam": 0.0}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        env.collect(tr, seed=11)
        tr.update(use_graph=True)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        ms = tr.profile(reset=True)
        if timed:
            assert all(v > 0.0 for v in ms.values()), ms
            assert sum(ms.values()) <= wall_ms, (ms, wall_ms)
            assert ms["rollout"] > ms["gae"], ms
        else:
            assert all(v == 0.0 for v in ms.values()), ms
        assert all(v == 0.0 for v in tr.profile().values())
        outs.append((tr.buf("r_obs").clone(), tr.buf("adv").clone(), pol.params.clone()))
        tr.close(); pol.close(); env.close()
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_env_step_on_every_floor_against_the_host_build(pkg, cuda, ref):
    """States on all nine floors with full inventories, armour, spells, enchantments and a boss
    fight under way (env_bind.deep_states): the GPU step against the host build of the same
    game-logic text (oracle/libcfenvhost.so), every field after every step, 288 envs x 400
    steps, resets supplied by the host generator.  The host build is held to the reference
    (strict per-operation fp32 build) on these states by the CPU suite; together: the kernel
    computes on deep floors what the reference's source defines."""
    n, steps = 288 - 288 % 64, 400
    states = eb.deep_states(ref, n, 23)
    host = eb.HostStep()
    env = pkg.Env(n)
    env.import_states(states)
    mine = states.copy()
    levels_seen, terminals = set(), 0
    script = eb.deep_script(n)
    for t in range(steps):
        act = ref.next_actions()          # any action stream will do: the reference's own
        if t < 2:
            act = np.where(script >= 0, script, act).astype(np.float32)
        rew, term, keys = host.step(mine, act)
        env.step(torch.from_numpy(act).cuda())
        got = env.export_states(eb.STATE_DTYPE)
        _compare(f"step {t}", mine, got, rew, env.rewards.cpu().numpy(), term, env.terminals.cpu().numpy())
        levels_seen |= set(mine["player_level"].tolist())
        for e in np.nonzero(term)[0]:
            st = mine[e:e + 1].copy()
            host.lib.cfhost_reset(eb.ptr(st), eb.ptr(np.ascontiguousarray(keys[e])))
            mine[e] = st[0]
            env.import_states(st, first=int(e))
            terminals += 1
    assert levels_seen >= set(range(9)) and terminals > 0, (levels_seen, terminals)


def _cell_agreement(a, b):
    """(differing cells, cells, worlds with any difference) over the three byte maps."""
    diff = np.zeros(len(a), bool)
    cells = bad = 0
    for f in ("map", "item_map", "light_map"):
        neq = a[f] != b[f]
        bad += int(neq.sum())
        cells += neq.size
        diff |= neq.reshape(len(a), -1).any(axis=1)
    return bad, cells, int(diff.sum())


def test_device_worldgen_against_host_and_reference(pkg, cuda, ref):
    """cfp_env_init (k_env_init; craftax_generate_world_from_key, craftax_full.c:2050-2142):
    worlds generated on the GPU against the same generator run on the host and against the
    compiled reference's c_init.  The three dungeon floors and every scalar are integer work
    and must be identical; the six noise floors may differ where a Perlin value lies within
    a rounding of a threshold (the GPU's cos / sin are not the C library's): at most one
    world in a hundred may show any difference, and at most one cell in a million."""
    n, seed = 512, 2024
    env = pkg.Env(n)
    env.init(seed)
    gpu = env.export_states(eb.STATE_DTYPE)
    host = pkg.env.generate_host(eb.STATE_DTYPE, seed, n)
    ref.init(n, seed)
    want = ref.export()
    for other, name in ((host, "host generator"), (want, "compiled reference")):
        bad, cells, worlds = _cell_agreement(gpu, other)
        print(f"GPU worldgen vs {name}: {bad} of {cells} cells differ, {worlds} of {n} worlds")
        assert worlds <= n // 100 and bad <= max(cells // 1000000, 200), name
        same = ~np.array([bool(eb.diff_fields(gpu[i:i + 1], other[i:i + 1])) for i in range(n)])
        assert same.sum() >= n - n // 100
        for f in eb.STATE_DTYPE.names:     # everything that is not a map or derived from one
            if f in ("map", "item_map", "light_map", "spawn_all_bits", "spawn_grave_bits", "spawn_water_bits",
                     "down_ladders", "up_ladders", "pad_"):
                continue
            x, y = gpu[f], other[f]
            if x.dtype == np.float32:
                x, y = x.view(np.uint32), y.view(np.uint32)
            assert np.array_equal(x, y), f"{f} vs {name}"
        for lvl in (1, 3, 4):              # dungeons
            for f in ("map", "item_map", "light_map", "down_ladders", "up_ladders"):
                assert np.array_equal(gpu[f][:, lvl], other[f][:, lvl]), f"{f}[{lvl}] vs {name}"


def test_closed_loop_with_device_resets(pkg, cuda, ref):
    """256 envs x 500 steps with nothing supplied by the host: envs created by cfp_env_init,
    stepped with their own action streams, finished envs regenerated by cfp_env_reset.  Every
    state field, reward and terminal is the compiled reference's after every step.  A reset
    whose world differs from the reference's in a noise cell (see the worldgen test) is
    counted and re-synchronised; at most one such reset is tolerated here."""
    n, steps, seed = 256, 500, 0
    ref.init(n, seed)
    env = pkg.Env(n)
    env.init(seed)
    start = env.export_states(eb.STATE_DTYPE)
    assert not eb.diff_fields(ref.export(), start), "initial worlds"
    resets = resynced = 0
    for t in range(steps):
        act = ref.next_actions()
        final, rew, term, keys = ref.step(act)
        env.step(None)
        mine = env.export_states(eb.STATE_DTYPE)
        _compare(f"step {t}", final, mine, rew, env.rewards.cpu().numpy(), term, env.terminals.cpu().numpy())
        done = np.nonzero(term)[0]
        if len(done):
            env.reset()
            fresh = ref.export(list(done))
            got = env.export_states(eb.STATE_DTYPE)[done]
            for k, e in enumerate(done):
                resets += 1
                if eb.diff_fields(fresh[k:k + 1], got[k:k + 1]):
                    resynced += 1
                    env.import_states(fresh[k:k + 1], first=int(e))
    assert resets > 100 and resynced <= 1, (resets, resynced)


def test_list_reset_in_a_large_env_vector(pkg, cuda):
    """Above 16 384 envs cfp_env_reset runs the world generator with 256 threads a floor (below,
    with 512): 16 448 envs made by cfp_env_init, a few hundred of them weakened so that they
    starve within sixty steps, every regenerated env against the host build of the same
    generator from the same reset key, and a sample of the initial worlds likewise."""
    n, seed = 16384 + 64, 5
    host = eb.HostStep()
    env = pkg.Env(n)
    env.init(seed)
    for e in (0, 1, 4097, n - 1):
        want = host.generate(seed + e, 1)
        assert not eb.diff_fields(want, env.export_states(eb.STATE_DTYPE, first=e, count=1)), f"initial world {e}"
    weak_envs = list(range(3, n, 53))
    for k, e in enumerate(weak_envs):
        st = env.export_states(eb.STATE_DTYPE, first=e, count=1)
        st["player_health"] = 1.0 + (k % 4)
        st["player_food"] = 0
        st["player_drink"] = 0
        st["player_recover"] = -14.0 + (k % 7)
        env.import_states(st, first=e)
    noop = torch.zeros(n, device=cuda)
    compared = 0
    for t in range(60):
        env.step(noop)
        cnt, recs = env.reset_list()
        if not cnt:
            continue
        before = {int(r[0]): env.export_states(eb.STATE_DTYPE, first=int(r[0]), count=1) for r in recs}
        env.reset()
        for r in recs:
            e = int(r[0])
            st = before[e]
            host.lib.cfhost_reset(eb.ptr(st), eb.ptr(np.ascontiguousarray(r[1:3]).view(np.uint32)))
            got = env.export_states(eb.STATE_DTYPE, first=e, count=1)
            assert not eb.diff_fields(st, got), f"step {t}: regenerated env {e}: {eb.diff_fields(st, got)}"
            compared += 1
    assert compared >= 100, compared
    env.close()


@pytest.mark.parametrize("n,small,pool", [(256, False, 0), (512, True, 0), (20480, False, 64)])
def test_run_step_is_the_rollout_step_without_slabs(pkg, cuda, n, small, pool):
    """cfp_env_run_step (cu_rollout_step_plain, the reference's `run` mode) against
    cfp_env_rollout_step on a twin: same worlds, same weights, same seed -- the sampled actions,
    log-probabilities and values of every step are the slabs' rows, rewards and terminals agree,
    the device step counter counts the steps, and the env states agree at the end (sampler
    fused into the 16-env-tile kernel, behind the 32-env-tile forward, and one thread per env
    above 16 384 envs; regenerated worlds and the pool)."""
    T = 12
    twins = []
    for _ in range(2):
        env = pkg.Env(n, pool=pool)
        env.init(3)
        if pool:
            env.pool_fill(9)
        pol = pkg.Policy(n, layers=2, seed=4)
        if small:
            pol.set_small_tiles(True)
        twins.append((env, pol))
    (env_a, pol_a), (env_b, pol_b) = twins
    tr = pkg.Trainer(pol_a, T)
    act, logp, val, ctr = env_b.run_outputs()
    for t in range(T):
        env_a.rollout_step(tr, t, 77)
        env_b.run_step(pol_b, 77)
        torch.cuda.synchronize()
        assert torch.equal(tr.buf("r_act")[t], act), f"step {t}: actions"
        assert torch.equal(tr.buf("r_logprob")[t], logp) and torch.equal(tr.buf("r_value")[t], val), f"step {t}"
        assert torch.equal(env_a.rewards, env_b.rewards) and torch.equal(env_a.terminals, env_b.terminals), f"step {t}"
        assert int(ctr[0]) == t + 1
    assert torch.equal(pol_a.state, pol_b.state)
    for first in range(0, n, 4096):
        cnt = min(64, n - first)
        a = env_a.export_states(eb.STATE_DTYPE, first=first, count=cnt)
        b = env_b.export_states(eb.STATE_DTYPE, first=first, count=cnt)
        assert not eb.diff_fields(a, b), f"final states from env {first}"
    tr.close()
    for env, pol in twins:
        pol.close(); env.close()


@pytest.mark.parametrize("n,small", [(256, False), (512, True)])
def test_run_step_replays_from_a_graph(pkg, cuda, n, small):
    """The reference captures one `run` step into a graph and replays it (cu_run_rollout_bench
    with graph = 1, craftax_full.cu:12142-12160; "replays are bitwise identical to eager
    launches").  Same here: one captured cfp_env_run_step replayed twelve times on a side
    stream, with eager work and synchronisations in between, against an eager twin -- draws,
    rewards, terminals, the step counter and the policy state after every replay, the env
    states at the end.  Weakened envs finish inside the run, so replays also regenerate worlds
    (the finished-env counter is cleared by a kernel of the step, not by a memset node)."""
    twins = []
    for _ in range(2):
        env = pkg.Env(n)
        env.init(21)
        weak = env.export_states(eb.STATE_DTYPE)
        for k, e in enumerate(range(0, n, 5)):
            weak["player_health"][e] = 1.0 + (k % 3)
            weak["player_food"][e] = 0
            weak["player_drink"][e] = 0
            weak["player_recover"][e] = -14.0 + (k % 5)
        env.import_states(weak)
        pol = pkg.Policy(n, layers=2, seed=8)
        if small:
            pol.set_small_tiles(True)
        twins.append((env, pol))
    (env_e, pol_e), (env_g, pol_g) = twins
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            env_g.run_step(pol_g, 5)
    torch.cuda.synchronize()
    out_e, out_g = env_e.run_outputs(), env_g.run_outputs()
    finished = 0
    for i in range(12):
        env_e.run_step(pol_e, 5)
        with torch.cuda.stream(side):
            graph.replay()
        torch.cuda.synchronize()
        junk = torch.randn(1 << 16, device=cuda).sum().item()   # eager work between replays
        assert np.isfinite(junk)
        for a, b, name in zip(out_e, out_g, ("actions", "logprobs", "values", "counter")):
            assert torch.equal(a, b), f"replay {i}: {name}"
        assert int(out_g[3][0]) == i + 1       # a capture runs nothing: replay i is step i
        assert torch.equal(env_e.rewards, env_g.rewards) and torch.equal(env_e.terminals, env_g.terminals)
        assert torch.equal(pol_e.state, pol_g.state)
        finished += int(env_g.terminals.sum().item())
    assert finished > 0
    assert not eb.diff_fields(env_e.export_states(eb.STATE_DTYPE), env_g.export_states(eb.STATE_DTYPE))
    for env, pol in twins:
        pol.close(); env.close()
