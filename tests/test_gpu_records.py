"""GPU parity of the byte/integer kernels: bit-exact against golden records of
the compiled reference and against the oracle."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import expand_records, synth_records_host

pytestmark = pytest.mark.gpu
P = ob.PLANE


def _t(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


@pytest.mark.parametrize("key", ["traj", "fuzz"])
def test_record_obs_matches_reference_vectors(pkg, cuda, golden, key):
    import torch
    sc, pl, want = golden[f"{key}_scalars"], golden[f"{key}_planes"], golden[f"{key}_records"]
    n = sc.shape[0]
    planes = _t(pl, cuda)                      # [n][3][2304]: env stride 6912
    base = planes.view(-1)
    rec = pkg.policy.record_obs(_t(sc, cuda), base, base[P:], base[2 * P:], n, 3 * P, 0)
    torch.cuda.synchronize()
    got = rec.cpu().numpy()
    bad = np.nonzero((got != want).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} of {n} records differ, first {bad[:5]}"


def test_record_tail_brute_force(pkg, cuda, golden):
    """Every inventory value 0..99 through the device tail (IEEE sqrtf * 0.1f)."""
    import torch
    sc = np.zeros((100, ob.SCALARS_BYTES), np.uint8)
    s32, f32 = sc.view(np.int32), sc.view(np.float32)
    off = {f[0]: getattr(ob.EnvScalars, f[0]).offset // 4 for f in ob.EnvScalars._fields_}
    for v in range(100):
        for nme in ("wood", "stone", "coal", "iron", "diamond", "sapphire", "ruby", "sapling",
                    "torches", "arrows", "player_food", "player_drink", "player_energy",
                    "player_mana", "player_xp", "player_dexterity", "player_strength",
                    "player_intelligence"):
            s32[v, off[nme]] = v
        s32[v, off["potions"]:off["potions"] + 6] = v
        f32[v, off["player_health"]] = np.float32(v * 0.09)
        s32[v, off["player_direction"]] = 1
    planes = torch.zeros(100 * 3 * P, dtype=torch.uint8, device=cuda)
    rec = pkg.policy.record_obs(_t(sc, cuda), planes, planes[P:], planes[2 * P:], 100, 3 * P, 0)
    torch.cuda.synchronize()
    got = np.ascontiguousarray(rec.cpu().numpy()[:, 792:]).view(np.uint32)
    assert np.array_equal(got, golden["tail_probe"].view(np.uint32))


def test_record_obs_full_level_planes(pkg, cuda, golden):
    """Same vectors laid out as the real env holds them: [env][9 levels][48][48],
    level_stride = 2304, so raw-level and clamped-level indexing are exercised."""
    import torch
    sc, pl, want = golden["fuzz_scalars"][:96], golden["fuzz_planes"][:96], golden["fuzz_records"][:96]
    n = sc.shape[0]
    level = sc.view(np.int32)[:, 2]
    full = np.random.default_rng(1).integers(0, 255, (3, n, 9, P), dtype=np.uint8)
    for e in range(n):
        for k in range(3):
            full[k, e, level[e]] = pl[e, k]
    d = _t(full, cuda)
    rec = pkg.policy.record_obs(_t(sc, cuda), d[0].reshape(-1), d[1].reshape(-1), d[2].reshape(-1),
                                n, 9 * P, P)
    torch.cuda.synchronize()
    assert np.array_equal(rec.cpu().numpy(), want)


def test_record_obs_ragged_count_and_oracle(pkg, cuda, golden):
    """n not a multiple of the 4-env workgroup; compared with the oracle."""
    import torch
    sc, pl = golden["fuzz_scalars"][:37], golden["fuzz_planes"][:37]
    want = ob.encode_compact(sc, pl[:, 0], pl[:, 1], pl[:, 2])
    planes = _t(pl, cuda).view(-1)
    rec = torch.full((40, 996), 0xEE, dtype=torch.uint8, device=cuda)
    pkg.policy.record_obs(_t(sc, cuda), planes, planes[P:], planes[2 * P:], 37, 3 * P, 0, rec=rec)
    torch.cuda.synchronize()
    got = rec.cpu().numpy()
    assert np.array_equal(got[:37], want)
    assert (got[37:] == 0xEE).all()            # nothing written past n


def test_record_obs_mob_collisions_last_slot_wins(pkg, cuda, golden):
    """Several live mobs of one class on one lit cell: the highest slot's type is the
    one recorded (craftax_encode_mobs3_compact writes in ascending slot order).  Built
    from a fuzzed reference state; compared with the oracle and checked directly."""
    import torch
    sc = golden["fuzz_scalars"][:64].copy()
    pl = golden["fuzz_planes"][:64].copy()
    pl[:, 2] = 255                                     # every cell lit
    s32 = sc.view(np.int32)
    off = {f[0]: getattr(ob.EnvScalars, f[0]).offset // 4 for f in ob.EnvScalars._fields_}
    groups = ((0, 3), (3, 3), (6, 2), (8, 3), (11, 3))  # first slot, slots of each class
    for e in range(64):
        s32[e, off["player_position"]:off["player_position"] + 2] = (20, 20)
        s32[e, off["mob_mask"]:off["mob_mask"] + 14] = 0
        first, cnt = groups[e % 5]
        for j in range(cnt):
            m = first + j
            if (e // 5) % 2 == 1 and j == 1:
                continue                               # a gap: slots first and first+2 collide
            s32[e, off["mob_mask"] + m] = 1
            s32[e, off["mob_type_id"] + m] = (e + 3 * j) % 8
            s32[e, off["mob_position"] + 2 * m:off["mob_position"] + 2 * m + 2] = (21, 19)
    want = ob.encode_compact(sc, pl[:, 0], pl[:, 1], pl[:, 2])
    planes = _t(pl, cuda).view(-1)
    rec = pkg.policy.record_obs(_t(sc, cuda), planes, planes[P:], planes[2 * P:], 64, 3 * P, 0)
    torch.cuda.synchronize()
    got = rec.cpu().numpy()
    assert np.array_equal(got, want)
    cell = (21 - 20 + 4) * 11 + (19 - 20 + 5)          # view cell of map (21, 19)
    for e in range(64):
        first, cnt = groups[e % 5]
        gap = (e // 5) % 2 == 1
        last_j = 0 if (gap and cnt == 2) else cnt - 1
        last_type = (e + 3 * last_j) % 8
        ch = 3 + e % 5
        assert got[e, cell * 8 + ch] == last_type + 1, (e, got[e, cell * 8:cell * 8 + 8])


def test_expand_obs_bit_exact(pkg, cuda):
    import torch
    rec = np.zeros((320, 996), np.uint8)
    rec[:256, :792] = np.arange(256, dtype=np.uint8)[:, None]
    rng = np.random.default_rng(5)
    rec[256:, :792] = rng.integers(0, 256, (64, 792), dtype=np.uint8)
    tail = rng.integers(0, 2 ** 32, (320, 51), dtype=np.uint64).astype(np.uint32)  # NaN payloads, -0, denormals
    rec[:, 792:] = tail.view(np.uint8).reshape(320, 204)
    x = pkg.policy.expand_obs(_t(rec, cuda), 320)
    torch.cuda.synchronize()
    assert np.array_equal(x.cpu().numpy().view(np.uint32), expand_records(rec).view(np.uint32))
    # output base not 16-byte aligned (element-wise kernel) and a ragged float count
    big = torch.zeros(321 * 843 + 1, device=cuda)
    rec321 = np.concatenate([rec, rec[:1]])
    pkg.policy.expand_obs(_t(rec321, cuda), 321, xobs=big[1:].view(321, 843))
    x2 = pkg.policy.expand_obs(_t(rec321, cuda), 321)
    torch.cuda.synchronize()
    want321 = expand_records(rec321).view(np.uint32)
    assert np.array_equal(big[1:].view(321, 843).cpu().numpy().view(np.uint32), want321)
    assert np.array_equal(x2.cpu().numpy().view(np.uint32), want321)
    # trainer window addressing: t0, mb, n, env_start
    slab = rng.integers(0, 256, (4, 8, 996), dtype=np.uint8)
    x = pkg.policy.expand_obs(_t(slab, cuda), count=2 * 3, t0=1, mb=3, n=8, env_start=2)
    torch.cuda.synchronize()
    want = expand_records(slab[1:3, 2:5].reshape(-1, 996))
    assert np.array_equal(x.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_synth_records_device_equals_host(pkg, cuda):
    import torch
    for n, seed, step in ((32, 1, 0), (1000, 7, 5), (4096, 2 ** 40 + 3, 127)):
        d = pkg.policy.synth_records(n, seed, step)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy(), synth_records_host(n, seed, step))


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (no reference source)")
def test_record_obs_live_reference_env(pkg, cuda):
    """State -> record on the device against the compiled reference env itself: 256 envs
    (seed 7, the harness's xorshift32 % 43 actions) stepped 600 times; every 40th step
    the encoder-input state of every env goes through k_record_obs and must equal the
    996-byte record the reference wrote for that env, bit for bit.  Fresh states on
    every run of the box, beyond the committed fixtures (mobs, darkness, deeper levels
    and post-reset states all occur within these steps)."""
    import torch
    n = 256
    env = ob.RefEnv(n, 7)
    try:
        checked = 0
        for t in range(601):
            if t % 40 == 0:
                want = env.records()
                views = [env.view(e) for e in range(n)]
                sc = np.stack([v[0] for v in views])
                pl = np.stack([v[1] for v in views]).reshape(n, 3, P)
                base = _t(pl, cuda).view(-1)
                rec = pkg.policy.record_obs(_t(sc, cuda), base, base[P:], base[2 * P:], n, 3 * P, 0)
                torch.cuda.synchronize()
                got = rec.cpu().numpy()
                bad = np.nonzero((got != want).any(axis=1))[0]
                assert bad.size == 0, f"step {t}: {bad.size} of {n} records differ, first {bad[:5]}"
                checked += n
            env.step()
        assert checked == 16 * n
    finally:
        env.close()


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (no reference source)")
def test_record_obs_live_fuzzed_states(pkg, cuda):
    """2048 freshly fuzzed states of the compiled reference (edge positions, every level,
    random mobs of every class on lit and dark cells, full inventories; seeds other than
    the committed fixtures') through k_record_obs in batches of 256, against the
    reference's own encoder on the same state, bit for bit."""
    import torch
    n = 256
    env = ob.RefEnv(n, 3)
    try:
        for rnd in range(8):
            want = np.empty((n, 996), dtype=np.uint8)
            scs, pls = [], []
            for e in range(n):
                env.fuzz(e, 500000 + rnd * n + e)
                sc, pl = env.view(e)
                scs.append(sc); pls.append(pl)
                want[e] = env.encode(e)
            base = _t(np.stack(pls).reshape(n, 3, P), cuda).view(-1)
            rec = pkg.policy.record_obs(_t(np.stack(scs), cuda), base, base[P:], base[2 * P:], n, 3 * P, 0)
            torch.cuda.synchronize()
            got = rec.cpu().numpy()
            bad = np.nonzero((got != want).any(axis=1))[0]
            assert bad.size == 0, f"round {rnd}: {bad.size} records differ, first seeds {500000 + rnd * n + bad[:5]}"
            mobs = (want[:, :792].reshape(n, 99, 8)[:, :, 3:] != 0).sum()
            assert mobs > 0, "the fuzzed states put no mob into view"
    finally:
        env.close()


# ---- records straight from the reference's per-field device arrays ----------------------
_SOA_DTYPES = {"player_health": np.float32, "light_level": np.float32, "is_sleeping": np.uint8,
               "is_resting": np.uint8, "learned_spells": np.uint8, "mob_mask": np.uint8}
_SLOT_CLASS = (0, 0, 0, 1, 1, 1, 2, 2, 3, 3, 3, 4, 4, 4)
_CLASS_FIRST = (0, 3, 6, 8, 11)


def _soa_from_scalars(pkg, sc, n_stride, seed):
    """cfp_env_scalars rows -> the reference's layout (craftax_full.cu:620-712): one array
    per field, [sub_index][env] with stride n_stride; the env's 14 mob slots go to level
    jax_index(player_level, 9) of the 9-level mob arrays and its monsters_killed entry to
    index player_level; every other entry holds random values the encoder must not read."""
    n = sc.shape[0]
    s32, f32 = sc.view(np.int32), sc.view(np.float32)
    off = {f[0]: getattr(ob.EnvScalars, f[0]).offset // 4 for f in ob.EnvScalars._fields_}
    rng = np.random.default_rng(seed)
    out = {}
    for name, k in pkg.policy.ENV_SOA_FIELDS:
        dt = _SOA_DTYPES.get(name, np.int32)
        if dt is np.float32:
            out[name] = rng.random((k, n_stride)).astype(np.float32)
        elif dt is np.uint8:
            out[name] = rng.integers(0, 2, (k, n_stride)).astype(np.uint8)
        else:
            out[name] = rng.integers(-3, 60, (k, n_stride)).astype(np.int32)
    level = s32[:, off["player_level"]]
    mlevel = np.where(level < 0, level + 9, level).clip(0, 8)          # jax_index(level, 9)
    env = np.arange(n)
    rename = {"wood": "inv_wood", "stone": "inv_stone", "coal": "inv_coal", "iron": "inv_iron",
              "diamond": "inv_diamond", "sapphire": "inv_sapphire", "ruby": "inv_ruby",
              "sapling": "inv_sapling", "torches": "inv_torches", "arrows": "inv_arrows",
              "books": "inv_books", "pickaxe": "inv_pickaxe", "sword": "inv_sword", "bow": "inv_bow",
              "potions": "inv_potions", "armour": "inv_armour"}
    for fname, ftype in ob.EnvScalars._fields_:
        o = off[fname]
        if fname in ("mob_type_id", "mob_mask", "mob_position", "monsters_killed_level"):
            continue
        name = rename.get(fname, fname)
        k = dict(pkg.policy.ENV_SOA_FIELDS)[name]
        src = f32 if _SOA_DTYPES.get(name) is np.float32 else s32
        for i in range(k):
            v = src[:, o + i]
            out[name][i, :n] = (v != 0) if _SOA_DTYPES.get(name) is np.uint8 else v
    out["monsters_killed"][level.clip(0, 8), env] = s32[:, off["monsters_killed_level"]]
    for m in range(14):
        c = _SLOT_CLASS[m]
        cfm = (c * 9 + mlevel) * 3 + (m - _CLASS_FIRST[c])
        out["mob_type_id"][cfm, env] = s32[:, off["mob_type_id"] + m]
        out["mob_mask"][cfm, env] = s32[:, off["mob_mask"] + m] != 0
        for a in range(2):
            out["mob_position"][cfm * 2 + a, env] = s32[:, off["mob_position"] + 2 * m + a]
    return out


def test_record_obs_from_reference_soa_layout(pkg, cuda, golden):
    """cfp_record_obs_soa on the fuzzed reference states scattered into the reference's
    own device layout (field arrays [sub_index][env], 9-level mob arrays, stride > n):
    the golden records bit for bit, the skip mask honoured, and the list form writing
    exactly the listed rows."""
    import torch
    sc, pl, want = golden["fuzz_scalars"], golden["fuzz_planes"], golden["fuzz_records"]
    n = sc.shape[0]
    n_stride = n + 7
    host = _soa_from_scalars(pkg, sc, n_stride, 11)
    arrays = {k: _t(v, cuda) for k, v in host.items()}
    planes = _t(pl, cuda).view(-1)
    P3 = 3 * P
    rec = pkg.policy.record_obs_soa(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, P3, 0)
    torch.cuda.synchronize()
    got = rec.cpu().numpy()
    bad = np.nonzero((got != want).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} of {n} records differ, first {bad[:5]}"
    # skip mask: flagged rows stay as they were
    skip = (np.arange(n) % 3 == 1).astype(np.uint8)
    rec2 = torch.full((n, 996), 0xEE, dtype=torch.uint8, device=cuda)
    pkg.policy.record_obs_soa(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, P3, 0,
                              skip=_t(skip, cuda), rec=rec2)
    torch.cuda.synchronize()
    got2 = rec2.cpu().numpy()
    assert np.array_equal(got2[skip == 0], want[skip == 0])
    assert np.all(got2[skip == 1] == 0xEE)
    # list form: entries are the .env members of 12-byte structs; count < max_count
    listed = np.nonzero(skip)[0][::-1].copy()
    recs = np.full((n, 3), -1, np.int32)
    recs[: listed.size, 1] = listed
    d_list = _t(recs, cuda)
    count = torch.tensor([listed.size], dtype=torch.int32, device=cuda)
    pkg.policy.record_obs_soa_list(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, P3, 0,
                                   d_list.view(-1)[1:], 12, count, n, rec2)
    torch.cuda.synchronize()
    assert np.array_equal(rec2.cpu().numpy(), want)
    # a one-env list and a launch far larger than the count
    rec3 = torch.full((n, 996), 0xEE, dtype=torch.uint8, device=cuda)
    one = torch.tensor([5], dtype=torch.int32, device=cuda)
    pkg.policy.record_obs_soa_list(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, P3, 0,
                                   one, 4, torch.tensor([1], dtype=torch.int32, device=cuda), n, rec3)
    torch.cuda.synchronize()
    got3 = rec3.cpu().numpy()
    assert np.array_equal(got3[5], want[5]) and np.all(np.delete(got3, 5, axis=0) == 0xEE)
    # a device count above max_count and entries outside the env range: the list is read up
    # to max_count only, out-of-range entries are skipped, every other row stays untouched
    rec4 = torch.full((n, 996), 0xEE, dtype=torch.uint8, device=cuda)
    bad = torch.tensor([3, -7, n + 100, 9, 11, 12], dtype=torch.int32, device=cuda)
    pkg.policy.record_obs_soa_list(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, P3, 0,
                                   bad, 4, torch.tensor([1000000], dtype=torch.int32, device=cuda), 4, rec4)
    torch.cuda.synchronize()
    got4 = rec4.cpu().numpy()
    assert np.array_equal(got4[[3, 9]], want[[3, 9]])
    assert np.all(np.delete(got4, [3, 9], axis=0) == 0xEE)


def test_record_obs_soa_above_the_small_batch_threshold(pkg, cuda, golden):
    """Up to 16 384 envs the SoA kernel gathers 16 envs a round, above that 32 (a 128-byte line
    of every field array): the fuzzed reference states tiled to 18 432 envs, every record
    against the golden bytes, dense and through a list of all envs in reverse order."""
    import torch
    reps = 48
    sc = np.tile(golden["fuzz_scalars"], (reps, 1))
    pl = np.tile(golden["fuzz_planes"], (reps, 1, 1))
    want = np.tile(golden["fuzz_records"], (reps, 1))
    n = sc.shape[0]
    assert n > 16384
    n_stride = n + 32
    arrays = {k: _t(v, cuda) for k, v in _soa_from_scalars(pkg, sc, n_stride, 12).items()}
    planes = _t(pl, cuda).view(-1)
    rec = pkg.policy.record_obs_soa(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, 3 * P, 0)
    torch.cuda.synchronize()
    bad = np.nonzero((rec.cpu().numpy() != want).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} of {n} records differ, first {bad[:5]}"
    rec2 = torch.full((n, 996), 0xEE, dtype=torch.uint8, device=cuda)
    order = torch.arange(n - 1, -1, -1, dtype=torch.int32, device=cuda)
    pkg.policy.record_obs_soa_list(arrays, n_stride, planes, planes[P:], planes[2 * P:], n, 3 * P, 0,
                                   order, 4, torch.tensor([n], dtype=torch.int32, device=cuda), n, rec2)
    torch.cuda.synchronize()
    assert np.array_equal(rec2.cpu().numpy(), want)
