"""Pins the CPU oracle's record encoder/expander (oracle/record_encode.c)
against vectors dumped from the compiled reference and against closed forms."""
import numpy as np
import pytest

import oracle_bind as ob
from parity_util import expand_records

P = ob.PLANE


def _encode(scalars, planes):
    return ob.encode_compact(scalars, planes[:, 0], planes[:, 1], planes[:, 2])


def test_encoder_matches_reference_on_trajectory_states(golden):
    rec = _encode(golden["traj_scalars"], golden["traj_planes"])
    assert np.array_equal(rec, golden["traj_records"])


def test_encoder_matches_reference_on_fuzzed_states(golden):
    rec = _encode(golden["fuzz_scalars"], golden["fuzz_planes"])
    want = golden["fuzz_records"]
    bad = np.nonzero((rec != want).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} fuzzed states differ, first {bad[:5]}"


def test_fixtures_cover_the_edge_cases(golden):
    """The vectors must exercise what a plausible mistake would break."""
    cells = golden["fuzz_records"][:, :792].reshape(-1, 99, 8)
    assert (cells[:, :, 2] == 0).any() and (cells[:, :, 2] == 1).any()
    for ch in range(3, 8):                      # every mob class shows up
        assert (cells[:, :, ch] > 0).any(), ch
    assert cells[:, :, 3:].max() == 8           # type id 7 -> byte 8
    sc = golden["fuzz_scalars"].view(np.int32)
    pos = sc[:, 0:2]
    assert (pos.min(axis=0) <= 3).all() and (pos.max(axis=0) >= 44).all()
    traj = golden["traj_records"][:, :792].reshape(-1, 99, 8)
    assert (traj[:, :, 3:] > 0).any()   # live mobs; darkness comes from the fuzz set


def test_record_invariants(golden):
    for key in ("traj_records", "fuzz_records"):
        rec = golden[key]
        cells = rec[:, :792].reshape(-1, 99, 8)
        vis = cells[:, :, 2]
        assert set(np.unique(vis)) <= {0, 1}
        # invisible cell: block, item and visible bytes are zero
        assert not cells[:, :, :2][vis == 0].any()
        assert (cells[:, :, 0][vis == 1] <= 36).all()
        assert ((cells[:, :, 1][vis == 1] >= 1) & (cells[:, :, 1][vis == 1] <= 5)).all()
        assert cells[:, :, 3:].max() <= 8
        tail = np.ascontiguousarray(rec[:, 792:]).view(np.float32)
        assert np.allclose(tail[:, 31:35].sum(axis=1), 1.0)   # direction one-hot


def test_tail_arithmetic_brute_force(golden):
    """sqrtf(i) * (1/10f) etc. for every inventory value 0..99, against the
    reference's own tail function (a true division would differ for 24 values)."""
    want = golden["tail_probe"]
    sc = np.zeros((100, ob.SCALARS_BYTES), np.uint8)
    s32 = sc.view(np.int32)
    f32 = sc.view(np.float32)
    names = [f[0] for f in ob.EnvScalars._fields_]
    off = {n: getattr(ob.EnvScalars, n).offset // 4 for n in names}
    for v in range(100):
        for n in ("wood", "stone", "coal", "iron", "diamond", "sapphire", "ruby",
                  "sapling", "torches", "arrows", "player_food", "player_drink",
                  "player_energy", "player_mana", "player_xp", "player_dexterity",
                  "player_strength", "player_intelligence"):
            s32[v, off[n]] = v
        s32[v, off["potions"]:off["potions"] + 6] = v
        f32[v, off["player_health"]] = np.float32(v * 0.09)
        s32[v, off["player_direction"]] = 1
    planes = np.zeros((100, 3, P), np.uint8)
    got = np.ascontiguousarray(_encode(sc, planes)[:, 792:]).view(np.float32)
    # the probe state has no mobs and spawn timer 0 -> boss flag 1 in both
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    x = np.arange(100, dtype=np.float32)
    assert np.array_equal(got[:, 0], np.sqrt(x) * np.float32(0.1))
    assert (got[:, 0] != np.sqrt(x) / np.float32(10.0)).sum() >= 20


def test_expand_closed_form():
    rec = np.zeros((300, ob.REC_BYTES), np.uint8)
    rec[:256, :792] = np.arange(256, dtype=np.uint8)[:, None]
    bits = np.array([0x00000000, 0x80000000, 0x3f800000, 0x7fc00001, 0xffc12345,
                     0x7f800000, 0x00000001, 0x3dcccccd], dtype=np.uint32)
    tail = np.resize(bits, (300, 51)).copy()
    rec[:, 792:] = tail.view(np.uint8).reshape(300, 204)
    x = ob.expand_record(rec)
    assert np.array_equal(x[:256, :792], np.repeat(np.arange(256, dtype=np.float32)[:, None], 792, 1))
    assert np.array_equal(x[:, 792:].view(np.uint32), tail)
    assert np.array_equal(expand_records(rec).view(np.uint32), x.view(np.uint32))


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (no reference source here)")
def test_encoder_matches_reference_live():
    """Same-binary comparison on a live rollout plus fresh fuzz seeds."""
    env = ob.RefEnv(64, 42)
    try:
        for step in range(120):
            env.step()
            if step % 10:
                continue
            recs = env.records()
            views = [env.view(e) for e in range(64)]
            sc = np.stack([v[0] for v in views])
            pl = np.stack([v[1].reshape(3, P) for v in views])
            assert np.array_equal(_encode(sc, pl), recs), f"step {step}"
        for i in range(256):
            env.fuzz(i % 64, 99000 + i)
            sc, pl = env.view(i % 64)
            got = _encode(sc[None], pl.reshape(1, 3, P))[0]
            assert np.array_equal(got, env.encode(i % 64)), f"fuzz seed {99000 + i}"
    finally:
        env.close()


def test_stock_flag_build_differs_only_in_tail_floats_by_one_ulp():
    """oracle/Makefile builds the compiled-reference checker with -mno-recip added to the
    reference's own flags and says what that changes: nothing in the map bytes, rewards and
    terminals; tail floats by at most one ulp.  Held here against a build with the stock
    flags over config 1's first 200 steps (1024 envs, seed 0, the xorshift32 % 43 actions)."""
    import ctypes as C
    import hashlib
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    stock_path = os.path.join(root, "oracle", "_ref", "libcfref_stock.so")
    stamp = os.path.join(root, "oracle", "_ref", "stock_build_cpu.txt")
    if not (os.path.exists(stock_path) and os.path.exists(stamp)):
        pytest.skip("stock-flag build of the reference not present")
    flags = next(l for l in open("/proc/cpuinfo") if l.startswith("flags"))
    if hashlib.md5(flags.encode()).hexdigest() != open(stamp).read().split()[0]:
        pytest.skip("the stock-flag build (-march=native) was made on another CPU")
    libs = []
    for name in ("libcfref.so", "libcfref_stock.so"):
        lib = C.CDLL(os.path.join(root, "oracle", "_ref", name))
        lib.cfref_init.argtypes = [C.c_int, C.c_uint64]
        lib.cfref_observations.restype = C.POINTER(C.c_uint8)
        lib.cfref_rewards.restype = C.POINTER(C.c_float)
        lib.cfref_terminals.restype = C.POINTER(C.c_float)
        lib.cfref_init(1024, 0)
        libs.append(lib)
    worst_ulp, moved = 0, set()
    for t in range(200):
        out = []
        for lib in libs:
            lib.cfref_step()
            obs = np.ctypeslib.as_array(lib.cfref_observations(), shape=(1024, 996)).copy()
            rew = np.ctypeslib.as_array(lib.cfref_rewards(), shape=(1024,)).copy()
            term = np.ctypeslib.as_array(lib.cfref_terminals(), shape=(1024,)).copy()
            out.append((obs, rew, term))
        (o0, r0, t0), (o1, r1, t1) = out
        assert np.array_equal(o0[:, :792], o1[:, :792]), f"map bytes differ at step {t}"
        assert np.array_equal(r0.view(np.uint32), r1.view(np.uint32)), f"rewards differ at step {t}"
        assert np.array_equal(t0, t1), f"terminals differ at step {t}"
        a = o0[:, 792:].copy().view(np.uint32).astype(np.int64)
        b = o1[:, 792:].copy().view(np.uint32).astype(np.int64)
        d = np.abs(a - b)
        worst_ulp = max(worst_ulp, int(d.max()))
        moved |= set(np.nonzero(d.any(axis=0))[0].tolist())
    # the square roots of the tail: ten inventory counts (0..9) and six potion counts (16..21)
    assert worst_ulp <= 1, worst_ulp
    assert moved <= set(range(0, 10)) | set(range(16, 22)), sorted(moved)
