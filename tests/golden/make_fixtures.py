"""Regenerates tests/golden/record_fixtures.npz from the compiled reference
(oracle/_ref/libcfref.so, built by `make -C oracle ref` where /root/reference
exists).  Run from the repo root:  python tests/golden/make_fixtures.py

Contents (inputs and expected outputs only):
  traj_*   encoder inputs + records sampled from config 1 of the baseline
           (compact-obs C env, 1024 envs, seed 0, xorshift32 % 43 actions)
  fuzz_*   seeded adversarial states pushed through the reference's own
           craftax_encode_compact_observation
  tail_*   the reference's scalar tail for inventory values 0..99
  slice_*  records/terminals of envs 0..31 for steps 0..15 of config 1
           (the rollout slice the GPU box replays through the policy)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_bind as ob  # noqa: E402

N_ENVS, SEED, STEPS = 1024, 0, 2000
CHECKPOINTS = sorted(set([0, 1, 2, 3, 5, 8, 13, 21, 34, 55, 89, 144, 233, 377, 610, 987,
                          1597, 1999] + list(range(100, 2000, 100))))
PER_CHECKPOINT = 8
SLICE_ENVS, SLICE_STEPS = 32, 16


def crop(planes):
    return planes.reshape(3, ob.PLANE)


def main():
    assert ob.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    rng = np.random.default_rng(12345)
    env = ob.RefEnv(N_ENVS, SEED)
    sc_l, pl_l, rec_l, meta_l = [], [], [], []
    slice_rec = np.zeros((SLICE_STEPS, SLICE_ENVS, ob.REC_BYTES), np.uint8)
    slice_term = np.zeros((SLICE_STEPS, SLICE_ENVS), np.float32)
    for step in range(STEPS + 1):
        if step > 0:
            env.step()
        if step < SLICE_STEPS:
            # the policy at step t consumes the records after t env steps and
            # the terminals the env wrote during the step before
            slice_rec[step] = env.records()[:SLICE_ENVS]
            slice_term[step] = env.terminals()[:SLICE_ENVS] if step > 0 else 0.0
        if step in CHECKPOINTS:
            recs = env.records()
            mobs = recs[:, :792].reshape(N_ENVS, 99, 8)[:, :, 3:].any(axis=(1, 2))
            dark = (recs[:, :792].reshape(N_ENVS, 99, 8)[:, :, 2] == 0).any(axis=1)
            cand = np.nonzero(dark)[0] if dark.any() else np.nonzero(mobs)[0]
            pick = list(rng.choice(cand, size=min(len(cand), PER_CHECKPOINT // 2),
                                   replace=False)) if len(cand) else []
            pick += list(rng.choice(N_ENVS, size=PER_CHECKPOINT - len(pick), replace=False))
            for e in pick:
                sc, planes = env.view(int(e))
                sc_l.append(sc); pl_l.append(crop(planes)); rec_l.append(recs[e].copy())
                meta_l.append((int(e), step))
    out = {
        "traj_scalars": np.stack(sc_l), "traj_planes": np.stack(pl_l),
        "traj_records": np.stack(rec_l), "traj_env_step": np.array(meta_l, np.int32),
        "slice_records": slice_rec, "slice_terminals": slice_term,
    }
    sc_l, pl_l, rec_l = [], [], []
    for i in range(384):
        e = i % N_ENVS
        env.fuzz(e, 7000 + i)
        sc, planes = env.view(e)
        sc_l.append(sc); pl_l.append(crop(planes)); rec_l.append(env.encode(e))
    out.update(fuzz_scalars=np.stack(sc_l), fuzz_planes=np.stack(pl_l),
               fuzz_records=np.stack(rec_l))
    tails = np.zeros((100, 51), np.float32)
    for v in range(100):
        ob.ref().cfref_tail_probe(v, np.float32(v * 0.09), tails[v].ctypes.data)
    out["tail_probe"] = tails
    env.close()
    path = os.path.join(HERE, "record_fixtures.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes;",
          {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
