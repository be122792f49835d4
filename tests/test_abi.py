"""The C-ABI library loads and exports exactly what include/cfp.h declares; no
compute is launched here (runs without a GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for header in ("cfp.h", "cfp_env.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(cfp_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_symbols_are_exported(pkg):
    lib = C.CDLL(pkg._lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} declared in cfp.h but not exported"


def test_binding_covers_every_declaration(pkg):
    assert sorted(pkg._lib.PROTOTYPES) == _declared()


def test_env_scalars_layout_matches_binding():
    import oracle_bind as ob
    text = open(os.path.join(ROOT, "include", "cfp.h")).read()
    body = text[text.index("typedef struct cfp_env_scalars {"):text.index("} cfp_env_scalars;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    n_i32 = 0
    for stmt in body.split("{", 1)[1].split(";"):
        m = re.match(r"\s*(int32_t|float)\s+(.*)", stmt.strip(), flags=re.S)
        if not m:
            continue
        for decl in m.group(2).split(","):
            cnt = 1
            for d in re.findall(r"\[(\w+)\]", decl):
                cnt *= int(d) if d.isdigit() else {"CFP_MOB_SLOTS": 14}[d]
            n_i32 += cnt
    assert n_i32 * 4 == ob.SCALARS_BYTES == 424


def test_argument_validation_needs_no_gpu(pkg):
    """Bad arguments are rejected with a message before any HIP call, like the
    reference's exit(1) paths (craftax_full.cu:11820-11825)."""
    lib = pkg.lib()
    h = C.c_void_p()
    assert lib.cfp_policy_create(C.byref(h), 100, 3, 1) != 0          # not a multiple of 32
    assert b"multiple of 32" in lib.cfp_last_error()
    assert lib.cfp_policy_create(C.byref(h), 64, 4, 1) != 0           # layers out of range
    assert b"layers" in lib.cfp_last_error()
    assert lib.cfp_policy_create(None, 64, 3, 1) != 0
    assert lib.cfp_gemm_fwd(0, 1, 1, None, None, None, None) != 0
    assert lib.cfp_encode_step(None, None, 32, None) != 0
    assert lib.cfp_abi_version() >= 1


def test_build_rejects_a_spilling_forward_kernel():
    """The forward kernel counts its own vector-memory operations for explicit
    s_waitcnt; the build refuses a compile whose k_policy_forward uses scratch."""
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "craftax.cu_amd", "build.py")
    spec = importlib.util.spec_from_file_location("cfp_build", path)
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    fn = "remark: f.hip:1:1: Function Name: _ZN3cfp16k_policy_forwardILi0ELi0EEEvNS_7FwdArgsE [-R]\n"
    other = "remark: f.hip:1:1: Function Name: _ZN3cfp6k_gemmILb0EEEvNS_8GemmArgsE [-R]\n"
    b.check_no_scratch(fn + "remark:     ScratchSize [bytes/lane]: 0 [-R]\n" +
                       other + "remark:     ScratchSize [bytes/lane]: 64 [-R]\n")
    with pytest.raises(RuntimeError, match="scratch"):
        b.check_no_scratch(fn + "remark:     ScratchSize [bytes/lane]: 24 [-R]\n")


def test_build_rejects_a_counted_wait_kernel_outside_its_register_budget():
    """The kernels with counted waits are scheduled for a fixed number of wavefronts per
    SIMD; the build refuses one whose registers or occupancy left the committed range."""
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "craftax.cu_amd", "build.py")
    spec = importlib.util.spec_from_file_location("cfp_build", path)
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)

    def remarks(fn, vgprs, agprs, occ):
        return (f"f.hip:1:1: remark: Function Name: {fn} [-Rpass-analysis=kernel-resource-usage]\n"
                f"f.hip:1:1: remark:     VGPRs: {vgprs} [-Rpass-analysis=kernel-resource-usage]\n"
                f"f.hip:1:1: remark:     AGPRs: {agprs} [-Rpass-analysis=kernel-resource-usage]\n"
                f"f.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
                f"f.hip:1:1: remark:     Occupancy [waves/SIMD]: {occ} [-Rpass-analysis=kernel-resource-usage]\n")
    fwd = "_ZN3cfp16k_policy_forwardILi0ELi0ELb0EEEvNS_7FwdArgsE"
    t16 = "_ZN3cfp12_GLOBAL__N_120k_policy_forward_t16ILi0EEEvNS_7FwdArgsE"
    rev = "_ZN3cfp12_GLOBAL__N_113k_gru_reverseILb1ELb1ELb0EEEvNS_11ReverseArgsE"
    other = "_ZN3cfp6k_gemmILb0EEEvNS_8GemmArgsE"
    use = b.resource_usage(remarks(fwd, 256, 126, 1))
    assert use[fwd] == {"VGPRs": 256, "AGPRs": 126, "ScratchSize": 0, "Occupancy": 1}
    # today's figures pass; a kernel without counted waits may use what it likes
    b.check_counted_wait_budget(remarks(fwd, 256, 126, 1) + remarks(t16, 162, 0, 2) + remarks(rev, 96, 0, 5) +
                                remarks(other, 512, 0, 1))
    for bad in (remarks(fwd, 256, 200, 1), remarks(fwd, 128, 0, 2), remarks(t16, 230, 0, 2), remarks(t16, 120, 0, 3),
                remarks(rev, 140, 0, 3), remarks(rev, 128, 0, 3)):
        with pytest.raises(RuntimeError, match="budget"):
            b.check_counted_wait_budget(bad)
