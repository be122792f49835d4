"""In-tree build of libcfpolicy.so for gfx950 (hipcc cross-compiles without a GPU)."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libcfpolicy.so")
SOURCES = ["policy_forward.hip", "policy_forward_bf16.hip", "policy_forward_t16.hip", "cfp_api.hip", "gemm.hip", "record.hip", "train.hip", "ppo_kernels.hip", "rollout.hip", "enc_grad.hip", "gemm_x9.hip", "env_step.hip"]
ARCH = "gfx950"


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH, /opt/rocm/bin)")


# Kernels that wait for loads they issue from inline assembly with explicit
# `s_waitcnt vmcnt(N)`, N = the number of younger vector-memory operations the
# source issues: the fused fp32 forward (both tile sizes) and the reverse MinGRU sweep.
COUNTED_WAIT_KERNELS = ("k_policy_forwardI", "k_policy_forward_t16I", "k_gru_reverseI")


def check_no_scratch(remarks):
    """A register spill is a vector-memory operation the source cannot count, so a
    build in which one of the kernels above uses scratch memory is rejected."""
    name, bad = None, []
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line and name and any(k in name for k in COUNTED_WAIT_KERNELS):
            if int(line.split("ScratchSize [bytes/lane]:")[1].split()[0]) != 0:
                bad.append(name)
    if bad:
        raise RuntimeError("kernels with counted waits spill registers to scratch memory: " + ", ".join(bad))


# Register budget and occupancy each of those kernels is scheduled for.  Their waits count
# the operations the source issues between a load and its use; how many wavefronts share a
# SIMD decides how far ahead those loads have to be issued (the forward kernels are written
# for one, respectively two, wavefronts per SIMD; the sweep for at least four, its
# __launch_bounds__), and a jump in registers is how a compiler change that re-orders or
# duplicates those loads shows first.  (kernel name part, VGPRs allowed, AGPRs allowed,
# occupancy [waves/SIMD] lowest, highest)
COUNTED_WAIT_BUDGET = (
    ("k_policy_forwardI", 256, 160, 1, 1),
    ("k_policy_forward_t16I", 192, 0, 2, 2),
    ("k_gru_reverseI", 128, 0, 4, 8),
)


def resource_usage(remarks):
    """{mangled kernel name: {"VGPRs", "AGPRs", "Occupancy", "ScratchSize"}} from the
    -Rpass-analysis=kernel-resource-usage remarks."""
    import re
    out, name = {}, None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
            out[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z][\w ]*?)(?: \[[^\]]*\])?:\s+(\d+)", line)
        if m and name:
            out[name][m.group(1)] = int(m.group(2))
    return out


def check_counted_wait_budget(remarks):
    """Refuse a build in which a kernel with counted waits left the register budget or the
    occupancy it is scheduled for."""
    bad = []
    for name, use in resource_usage(remarks).items():
        for part, vgprs, agprs, occ_lo, occ_hi in COUNTED_WAIT_BUDGET:
            if part not in name or "VGPRs" not in use:
                continue
            occ = use.get("Occupancy", occ_lo)
            if use["VGPRs"] > vgprs or use.get("AGPRs", 0) > agprs or not occ_lo <= occ <= occ_hi:
                bad.append(f"{name}: {use['VGPRs']} VGPRs, {use.get('AGPRs', 0)} AGPRs, occupancy {occ} "
                           f"(allowed: {vgprs}, {agprs}, {occ_lo}..{occ_hi})")
    if bad:
        raise RuntimeError("kernels with counted waits outside their register / occupancy budget:\n  " + "\n  ".join(bad))


def build(verbose=False):
    """Compile every HIP source into one shared library; always recompiles."""
    cmd = [
        hipcc_path(), f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
        "-shared", "-Wall", "-Wno-unused-function",
        # packed fp32 VALU ops are kept off for gfx950 device code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Rpass-analysis=kernel-resource-usage",
        "-o", OUT,
    ] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", "[-Rpass-analysis=kernel-resource-usage]")
    err = "\n".join(l for l in res.stderr.splitlines() if not any(n in l for n in noise))
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    check_no_scratch(res.stderr)
    check_counted_wait_budget(res.stderr)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
