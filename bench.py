#!/usr/bin/env python3
"""Benchmark of the batched policy forward on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--envs N] [--no-cpu]

One step = one pass of the fused policy forward (996-byte records -> encoder
-> MinGRU x3 -> actor/value heads) over one batch of synthetic records that is
already resident in HBM, hidden state carried from step to step.  The default
workload is the baseline's third config: 262 144 envs, h256x3, one unchunked
launch per step; the 16 x 16 384 chunked schedule is timed beside it.

Prints ONE JSON line (metric = env-steps/s) with two extra objects:
  roofline     algorithmic FLOPs per launch / measured launch time (HIP events on
               the launch stream) against the fp32 MFMA peak (157.3 TFLOP/s).
               Beside it, as extra keys, the bound of the kernel's actual
               instruction mix: all FLOPs issue on the fp32 MFMA except the
               encoder's byte-valued features, which issue as three bf16 MFMAs
               per product (2.5 PFLOP/s).  `traffic` is read from the tracked
               counter summary under profiles/ and is null when that summary
               was taken from other kernel sources than the ones present
  cpu_baseline the CPU oracle's scalar fp32 forward timed on this host's cores
               on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

FLOP_PER_ENV_STEP = 2 * 843 * 256 + 3 * 2 * 768 * 256 + 2 * 44 * 256   # 1 633 792
BYTES_PER_ENV_STEP = 996 + 4 + 3 * 256 * 4 * 2 + 44 * 4                # 7 320
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
# Which matrix pipe the FLOPs issue on.  The encoder's 792 byte-valued features
# are exact in bf16 and each fp32 weight is exactly three bf16 terms, so their
# products run as three bf16 MFMAs (fp32 accumulate); everything else (51 fp32
# tail features, gate GEMMs, heads) is fp32 MFMA.
FLOP_BF16_PIPE_ALGO = 2 * 792 * 256                 # per env-step, algorithmic
FLOP_BF16_PIPE_ISSUED = 3 * FLOP_BF16_PIPE_ALGO     # three terms per weight
FLOP_FP32_PIPE = FLOP_PER_ENV_STEP - FLOP_BF16_PIPE_ALGO
# matrix-pipe time bound per env-step and the effective peak of this mix
T_BOUND_PER_ENV_STEP = (FLOP_FP32_PIPE / (PEAK_FP32_MFMA_TFLOPS * 1e12) +
                        FLOP_BF16_PIPE_ISSUED / (PEAK_BF16_MFMA_TFLOPS * 1e12))
PEAK_MIX_TFLOPS = FLOP_PER_ENV_STEP / T_BOUND_PER_ENV_STEP / 1e12   # 196.9
LAYERS = 3
KERNEL_SOURCES = ("policy_forward.hip", "policy_tile.h", "cfp_common.h", "cfp_internal.h", "sample_row.h")
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "policy_forward_262144_pmc.txt")


def kernel_source_id():
    """sha1 over the sources of k_policy_forward: ties a counter summary to a build."""
    import hashlib
    h = hashlib.sha1()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "craftax.cu_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(n):
    """HBM bytes per launch from the tracked rocprofv3 FETCH_SIZE / WRITE_SIZE summary
    (already scaled by what the counters read for a plain copy), or None when the
    summary is missing, was taken at another batch size or from other kernel sources."""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    def field(key):
        m = re.search(r"^" + key + r"\s*=\s*(\S+)", text, flags=re.M)
        return m.group(1) if m else None
    if field("envs") != str(n) or field("kernel_source_sha1") != kernel_source_id():
        return None
    t = field("traffic_bytes_per_launch")
    return int(t) if t and t.isdigit() else None


def policy_in_the_loop(pkg, torch, n, steps):
    """The whole rollout step with the env on the device (record -> forward + sample -> game
    step -> reward / done rows -> regeneration of finished worlds), reported beside `value`:
    env-steps/s and the forward's FLOPs over the whole step's time against the fp32 peak."""
    env = pkg.Env(n)
    env.init(0)
    for _ in range(300):           # random-action steps: the episodes' phases spread out
        env.step(None)
        env.reset()
    pol = pkg.Policy(n, LAYERS, seed=1)
    T = 8
    tr = pkg.Trainer(pol, T)
    for t in range(16):            # settles the clock
        env.rollout_step(tr, t % T, 1234)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for t in range(steps):
        env.rollout_step(tr, t % T, 1234)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    out = {"ms_per_step": ms, "env_steps_per_s": n / ms * 1e3, "steps": steps,
           "finished_envs_last_step": env.reset_list()[0],
           "frac_fp32_peak_of_forward_flops": FLOP_PER_ENV_STEP * n / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
           "what": "cfp_env_rollout_step: env, records, h256x3 policy, sampling and resets on the device, "
                   "observations / states / actions / rewards recorded into a trainer's slabs"}
    # the same step without the slabs (cfp_env_run_step = the reference's `run` mode)
    e0.record()
    for t in range(steps):
        env.run_step(pol, 1234)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    out["run_mode"] = {"ms_per_step": ms, "env_steps_per_s": n / ms * 1e3,
                       "frac_fp32_peak_of_forward_flops":
                           FLOP_PER_ENV_STEP * n / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                       "what": "cfp_env_run_step: the same step with no slabs"}
    tr.close(); pol.close(); env.close()
    return out


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--envs", type=int, default=262144)
    ap.add_argument("--ring", type=int, default=16,
                    help="distinct pre-generated record batches cycled through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--schedule", choices=("both", "unchunked", "chunked"), default="both",
                    help="which launch schedule(s) to time; profiles use one at a time")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MiB",
                    help="only run a plain device copy of this many MiB four times "
                         "(calibrates the FETCH_SIZE / WRITE_SIZE counters) and exit")
    return ap.parse_args()


def time_steps(pol, recs, term, state, av, steps, chunk, torch):
    """Time `steps` forwards with HIP events on the launch stream; returns
    (wall seconds for all steps, mean per-step device milliseconds)."""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i][0].record()
        pol.forward(recs[i % len(recs)], term, state, av=av, chunk=chunk)
        ev[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = sum(a.elapsed_time(b) for a, b in ev) / steps
    return wall, dev_ms


def cpu_baseline(params, seed):
    """CPU oracle (scalar fp32 port of the reference's k_policy_ref_l3) on a
    bounded sample: 32 768 envs x 12 steps, state carried, all host threads the
    box grants (at most 16)."""
    import numpy as np
    import oracle_bind as ob
    from parity_util import HIDDEN, synth_records_host
    threads = max(1, min(16, ob.cfo().cfo_max_threads(), os.cpu_count() or 1))
    n, steps = 32768, 12
    state = np.zeros((LAYERS, n, HIDDEN), np.float32)
    term = np.zeros(n, np.float32)
    recs = [synth_records_host(n, seed, s) for s in range(2)]
    ob.forward_f32(params, LAYERS, recs[0][:1024], state[:, :1024].copy(), term[:1024], threads)
    t0 = time.perf_counter()
    for s in range(steps):
        ob.forward_f32(params, LAYERS, recs[s % 2], state, term, threads)
    dt = time.perf_counter() - t0
    out = {"value": n * steps / dt, "unit": "env-steps/s", "cores": threads, "kind": "port",
           "sample": f"{n} envs x {steps} steps of the same forward (oracle/policy_ref.c "
                     f"cfo_forward_f32, OpenMP, {dt:.1f} s)",
           "gflops": FLOP_PER_ENV_STEP * n * steps / dt / 1e9}
    # the record encoder's CPU restatement (state -> 996-byte record, one thread), on the
    # fuzzed reference states of tests/golden tiled to 65 536 envs
    try:
        g = np.load(os.path.join(ROOT, "tests", "golden", "record_fixtures.npz"))
        idx = np.arange(65536) % g["fuzz_scalars"].shape[0]
        sc, pl = g["fuzz_scalars"][idx], g["fuzz_planes"][idx]
        m, it, li = (np.ascontiguousarray(pl[:, k]) for k in range(3))
        ob.encode_compact(sc[:256], m[:256], it[:256], li[:256])
        t0 = time.perf_counter()
        ob.encode_compact(sc, m, it, li)
        out["record_encode_envs_per_s_1_thread"] = 65536 / (time.perf_counter() - t0)
    except OSError:
        pass
    if ob.have_ref():
        # the reference's own CPU env (random actions), for orientation only: a
        # different path (env step, not policy forward)
        sps1 = ob.ref().cfref_bench(1024, 300, 1, 0)
        spsN = ob.ref().cfref_bench(8192, 60, threads, 0)
        out["reference_env_sps"] = {"1024_envs_1_thread": sps1,
                                    f"8192_envs_{threads}_threads": spsN}
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (--gpus {args.gpus} was asked "
              "for); envs are independent, so N GPUs would each run this same kernel on "
              "n/N envs with no exchange", file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as ge
    pkg = ge.load_package()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.copy_probe:
        src = torch.full((args.copy_probe << 20,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes": src.numel(), "copies": 4}))
        return
    n, steps, warmup = args.envs, args.steps, args.warmup
    seed = 1234
    pol = pkg.Policy(n, LAYERS, seed=1)          # weights: Xavier-uniform from seed 1
    params = pol.get_params()
    ring = max(1, min(args.ring, steps))
    recs = [pkg.policy.synth_records(n, seed, s) for s in range(ring)]
    term = (torch.rand(n, device="cuda") < 0.0034).float()   # the real env's terminal rate
    av = torch.empty(n, 44, device="cuda")
    state = pol.state
    torch.cuda.synchronize()

    results = {}
    schedules = [("unchunked", 0), ("chunked_16x16384", 16384 if n > 16384 else 0)]
    if args.schedule == "unchunked":
        schedules = schedules[:1]
    elif args.schedule == "chunked":
        schedules = schedules[1:]
    for name, chunk in schedules:
        state.zero_()
        for i in range(warmup):
            pol.forward(recs[i % ring], term, state, av=av, chunk=chunk)
        wall, dev_ms = time_steps(pol, recs, term, state, av, steps, chunk, torch)
        results[name] = {"ms_per_step": wall / steps * 1e3, "device_ms_per_step": dev_ms,
                         "env_steps_per_s": n * steps / wall}
    assert torch.isfinite(av).all(), "non-finite policy outputs"

    # bf16-input / fp32-accumulate variant of the same step (reported beside the fp32
    # figure, never as `value`): bound by vector work and HBM, so it carries an HBM
    # fraction instead of an MFMA one
    bf16 = None
    if args.schedule == "both":
        pol.set_gemm_bf16(True)
        state.zero_()
        for i in range(warmup):
            pol.forward(recs[i % ring], term, state, av=av)
        wall, dev_ms = time_steps(pol, recs, term, state, av, steps, 0, torch)
        pol.set_gemm_bf16(False)
        assert torch.isfinite(av).all(), "non-finite bf16 policy outputs"
        bf16 = {"ms_per_step": wall / steps * 1e3, "device_ms_per_step": dev_ms,
                "env_steps_per_s": n * steps / wall, "kernel": "k_policy_forward_bf16",
                "hbm_frac": BYTES_PER_ENV_STEP * n / (dev_ms * 1e-3) / 8e12,
                "tflops": FLOP_PER_ENV_STEP * n / (dev_ms * 1e-3) / 1e12}

    best = results.get("unchunked") or results["chunked_16x16384"]
    launches = 1 if "unchunked" in results else max(1, n // 16384)
    launch_s = best["device_ms_per_step"] * 1e-3 / launches
    achieved = FLOP_PER_ENV_STEP * (n // launches) / launch_s / 1e12
    line = {
        "metric": "policy-forward env-steps/sec @262k envs h256x3; % fp32 MFMA peak",
        "value": best["env_steps_per_s"], "unit": "env-steps/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": best["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"policy forward h256x3, {n} envs, one unchunked launch per "
                               f"step, {steps} consecutive steps carrying hidden state, "
                               "synthetic 996-byte records resident in HBM",
                   "envs": n, "layers": LAYERS, "hidden": 256, "chunk": 0,
                   "record_batches_in_hbm": ring},
        "pct_fp32_mfma_peak": 100.0 * achieved / PEAK_FP32_MFMA_TFLOPS,
        "chunked_16x16384": results.get("chunked_16x16384"),
        "bf16_in_fp32_acc_unchunked": bf16,
        "kernel_source_sha1": kernel_source_id(),
        # algorithmic FLOPs per launch / launch time against the fp32 MFMA peak; the
        # mixed-pipe keys price the same launch against the bound of its instruction mix
        # (fp32 pipe at 157.3, the encoder's byte features on the bf16 pipe at 2500)
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                     "mixed_pipe_peak": PEAK_MIX_TFLOPS,
                     "frac_of_mixed_pipe_bound": achieved / PEAK_MIX_TFLOPS,
                     "fp32_pipe_flops_per_launch": FLOP_FP32_PIPE * n // launches,
                     "bf16_pipe_issued_flops_per_launch": FLOP_BF16_PIPE_ISSUED * n // launches,
                     "traffic": measured_traffic(n) if launches == 1 else None,
                     "kernel": "k_policy_forward",
                     "flops_per_launch": FLOP_PER_ENV_STEP * n // launches,
                     "algorithmic_hbm_bytes_per_launch": BYTES_PER_ENV_STEP * n // launches,
                     "launch_ms": launch_s * 1e3},
    }
    pol.close()
    if args.schedule == "both":
        line["policy_in_the_loop"] = policy_in_the_loop(pkg, torch, n, min(steps, 64))
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(params, seed)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
