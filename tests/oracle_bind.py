"""ctypes bindings of the CPU oracle (oracle/libcfo.so) and, when it was built,
the compiled reference checker (oracle/_ref/libcfref.so).  Test infrastructure:
imported only by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CFO_PATH = os.path.join(ROOT, "oracle", "libcfo.so")
REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libcfref.so")

HIDDEN, GRU, OBS, REC_BYTES, ACTIONS, AV = 256, 768, 843, 996, 43, 44
MOB_SLOTS = 14
PLANE = 48 * 48

vp = C.c_void_p


class EnvScalars(C.Structure):
    """cfp_env_scalars of include/cfp.h."""
    _fields_ = [
        ("player_position", C.c_int32 * 2), ("player_level", C.c_int32),
        ("player_direction", C.c_int32), ("player_health", C.c_float),
        ("player_food", C.c_int32), ("player_drink", C.c_int32),
        ("player_energy", C.c_int32), ("player_mana", C.c_int32),
        ("player_xp", C.c_int32), ("player_dexterity", C.c_int32),
        ("player_strength", C.c_int32), ("player_intelligence", C.c_int32),
        ("is_sleeping", C.c_int32), ("is_resting", C.c_int32),
        ("wood", C.c_int32), ("stone", C.c_int32), ("coal", C.c_int32),
        ("iron", C.c_int32), ("diamond", C.c_int32), ("sapphire", C.c_int32),
        ("ruby", C.c_int32), ("sapling", C.c_int32), ("torches", C.c_int32),
        ("arrows", C.c_int32), ("books", C.c_int32), ("pickaxe", C.c_int32),
        ("sword", C.c_int32), ("bow", C.c_int32), ("potions", C.c_int32 * 6),
        ("armour", C.c_int32 * 4), ("sword_enchantment", C.c_int32),
        ("bow_enchantment", C.c_int32), ("armour_enchantments", C.c_int32 * 4),
        ("light_level", C.c_float), ("learned_spells", C.c_int32 * 2),
        ("monsters_killed_level", C.c_int32),
        ("boss_timesteps_to_spawn_this_round", C.c_int32),
        ("mob_type_id", C.c_int32 * MOB_SLOTS), ("mob_mask", C.c_int32 * MOB_SLOTS),
        ("mob_position", (C.c_int32 * 2) * MOB_SLOTS),
    ]


SCALARS_BYTES = C.sizeof(EnvScalars)   # 424


class PpoBatch(C.Structure):
    """cfo_ppo_batch of oracle/cfo_train.h."""
    _fields_ = [
        ("T", C.c_int), ("n", C.c_int), ("env_start", C.c_int), ("mb", C.c_int),
        ("layers", C.c_int), ("seg_len", C.c_int),
        ("r_obs", vp), ("r_state", vp), ("r_act", vp), ("r_logprob", vp),
        ("adv", vp), ("ret", vp), ("r_done", vp),
        ("adv_sum", C.c_double), ("adv_sumsq", C.c_double),
        ("clip", C.c_float), ("vf", C.c_float), ("ent", C.c_float),
    ]


_cfo = None
_ref = None


def cfo():
    global _cfo
    if _cfo is None:
        if not os.path.exists(CFO_PATH):
            raise ImportError(f"{CFO_PATH} missing: run `make -C oracle all`")
        lib = C.CDLL(CFO_PATH)
        lib.cfo_encode_compact_batch.argtypes = [C.c_int, vp, vp, vp, vp, C.c_size_t,
                                                 C.c_size_t, vp]
        lib.cfo_expand_record.argtypes = [vp, vp]
        lib.cfo_forward_f64.argtypes = [vp, C.c_int, C.c_int] + [vp] * 9
        lib.cfo_classic_expand.argtypes = [vp, vp]
        lib.cfo_sample_action.argtypes = [vp, C.c_int, C.c_float, vp]
        lib.cfo_sample_action.restype = C.c_int
        lib.cfo_sample_margin.argtypes = [vp, C.c_int, C.c_float]
        lib.cfo_sample_margin.restype = C.c_float
        lib.cfo_philox4x32_10.argtypes = [vp, vp, vp]
        lib.cfo_philox4x32_10.restype = None
        lib.cfo_philox_uniform.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
        lib.cfo_philox_uniform.restype = C.c_float
        lib.cfo_classic_forward_f64.argtypes = [vp, C.c_int, C.c_int] + [vp] * 9
        lib.cfo_forward_f32.argtypes = [vp, C.c_int, C.c_int, vp, vp, vp, vp, C.c_int]
        lib.cfo_max_threads.restype = C.c_int
        lib.cfo_ppo_loss_f64.restype = C.c_double
        lib.cfo_ppo_loss_f64.argtypes = [vp, C.POINTER(PpoBatch), vp]
        lib.cfo_ppo_backward_f64.argtypes = [vp, C.POINTER(PpoBatch), vp, vp]
        lib.cfo_ppo_min_abs_zh.argtypes = [vp, C.POINTER(PpoBatch), C.c_int]
        lib.cfo_ppo_min_abs_zh.restype = C.c_double
        lib.cfo_ppo_backward_bf16ops_f64.argtypes = [vp, C.POINTER(PpoBatch), vp, vp, C.c_int]
        lib.cfo_gae_f64.argtypes = [vp, vp, vp, vp, vp, vp, C.c_int, C.c_int,
                                    C.c_double, C.c_double]
        lib.cfo_adam_f64.argtypes = [vp, vp, vp, vp, C.c_size_t, C.c_int, C.c_double,
                                     C.c_double, C.c_double, C.c_double]
        _cfo = lib
    return _cfo


def have_ref():
    return os.path.exists(REF_PATH)


def ref():
    global _ref
    if _ref is None:
        lib = C.CDLL(REF_PATH)
        lib.cfref_init.argtypes = [C.c_int, C.c_uint64]
        lib.cfref_observations.restype = vp
        lib.cfref_terminals.restype = vp
        lib.cfref_rewards.restype = vp
        lib.cfref_view.argtypes = [C.c_int, vp, vp]
        lib.cfref_encode.argtypes = [C.c_int, vp]
        lib.cfref_fuzz_state.argtypes = [C.c_int, C.c_uint64]
        lib.cfref_tail_probe.argtypes = [C.c_int, C.c_float, vp]
        lib.cfref_bench.restype = C.c_double
        lib.cfref_bench.argtypes = [C.c_int, C.c_int, C.c_int, C.c_uint64]
        _ref = lib
    return _ref


def _p(a):
    return None if a is None else a.ctypes.data_as(vp)


# ---- oracle wrappers ---------------------------------------------------------
def encode_compact(scalars_u8, maps, items, lights, level_stride=0):
    """scalars_u8 [n][424] uint8 (EnvScalars bytes); maps/items/lights [n][...] u8
    with one env per row.  Returns records [n][996]."""
    n = scalars_u8.shape[0]
    maps = np.ascontiguousarray(maps); items = np.ascontiguousarray(items)
    lights = np.ascontiguousarray(lights)
    env_stride = maps.strides[0]
    assert items.strides[0] == env_stride and lights.strides[0] == env_stride
    rec = np.empty((n, REC_BYTES), dtype=np.uint8)
    cfo().cfo_encode_compact_batch(n, _p(np.ascontiguousarray(scalars_u8)), _p(maps),
                                   _p(items), _p(lights), env_stride, level_stride,
                                   _p(rec))
    return rec


def expand_record(rec):
    rec = np.ascontiguousarray(rec).reshape(-1, REC_BYTES)
    x = np.empty((rec.shape[0], OBS), dtype=np.float32)
    for i in range(rec.shape[0]):
        cfo().cfo_expand_record(_p(rec[i]), _p(x[i]))
    return x


def forward_f64(params, layers, x, state, terminals):
    """fp64 oracle forward.  x [n][843] f32, state [L][n][256] (any float dtype,
    not modified), terminals [n] or None.  Returns dict of fp64 arrays."""
    params = np.ascontiguousarray(params, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.shape[0]
    st_in = np.ascontiguousarray(state, dtype=np.float64)
    term = None if terminals is None else np.ascontiguousarray(terminals, dtype=np.float32)
    out = {
        "h_enc": np.empty((n, HIDDEN)), "r_state": np.empty((layers, n, HIDDEN)),
        "state": np.empty((layers, n, HIDDEN)), "h3": np.empty((n, HIDDEN)),
        "logits": np.empty((n, ACTIONS)), "values": np.empty(n),
    }
    cfo().cfo_forward_f64(_p(params), layers, n, _p(x), _p(st_in), _p(term),
                          _p(out["h_enc"]), _p(out["r_state"]), _p(out["state"]),
                          _p(out["h3"]), _p(out["logits"]), _p(out["values"]))
    return out


def classic_expand(rec):
    rec = np.ascontiguousarray(rec, dtype=np.uint8).reshape(-1, 148)
    x = np.empty((rec.shape[0], 1345), dtype=np.float32)
    for i in range(rec.shape[0]):
        cfo().cfo_classic_expand(_p(rec[i]), _p(x[i]))
    return x


def classic_forward_f64(params, layers, x, state, terminals):
    """fp64 oracle forward of the classic-game policy; x [n][1345]."""
    params = np.ascontiguousarray(params, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.shape[0]
    st_in = np.ascontiguousarray(state, dtype=np.float64)
    term = None if terminals is None else np.ascontiguousarray(terminals, dtype=np.float32)
    out = {
        "h_enc": np.empty((n, HIDDEN)), "r_state": np.empty((layers, n, HIDDEN)),
        "state": np.empty((layers, n, HIDDEN)), "h3": np.empty((n, HIDDEN)),
        "logits": np.empty((n, 17)), "values": np.empty(n),
    }
    cfo().cfo_classic_forward_f64(_p(params), layers, n, _p(x), _p(st_in), _p(term),
                                  _p(out["h_enc"]), _p(out["r_state"]), _p(out["state"]),
                                  _p(out["h3"]), _p(out["logits"]), _p(out["values"]))
    return out


def forward_f32(params, layers, rec, state, terminals, threads=0):
    """Scalar fp32 CPU forward (the timed CPU baseline); state updated in place."""
    params = np.ascontiguousarray(params, dtype=np.float32)
    rec = np.ascontiguousarray(rec, dtype=np.uint8)
    n = rec.shape[0]
    assert state.dtype == np.float32 and state.flags.c_contiguous
    term = None if terminals is None else np.ascontiguousarray(terminals, dtype=np.float32)
    av = np.empty((n, AV), dtype=np.float32)
    cfo().cfo_forward_f32(_p(params), layers, n, _p(rec), _p(state), _p(term), _p(av),
                          threads)
    return av


def make_batch(T, n, env_start, mb, layers, seg_len, r_obs, r_state, r_act, r_logprob,
               adv, ret, r_done, clip=0.2, vf=0.5, ent=0.01):
    """Build a PpoBatch; returns (batch, keepalive list)."""
    arrs = [np.ascontiguousarray(r_obs, dtype=np.uint8),
            np.ascontiguousarray(r_state, dtype=np.float32),
            np.ascontiguousarray(r_act, dtype=np.int32),
            np.ascontiguousarray(r_logprob, dtype=np.float32),
            np.ascontiguousarray(adv, dtype=np.float32),
            np.ascontiguousarray(ret, dtype=np.float32),
            np.ascontiguousarray(r_done, dtype=np.uint8)]
    a64 = arrs[4].astype(np.float64)
    b = PpoBatch(T, n, env_start, mb, layers, seg_len, *[_p(a) for a in arrs],
                 float(a64.sum()), float((a64 * a64).sum()), clip, vf, ent)
    return b, arrs


def ppo_loss_f64(params, batch):
    params = np.ascontiguousarray(params, dtype=np.float32)
    l3 = np.zeros(3)
    v = cfo().cfo_ppo_loss_f64(_p(params), C.byref(batch), _p(l3))
    return v, l3


def ppo_backward_f64(params, batch):
    params = np.ascontiguousarray(params, dtype=np.float32)
    g = np.zeros(params.size)
    l3 = np.zeros(3)
    cfo().cfo_ppo_backward_f64(_p(params), C.byref(batch), _p(g), _p(l3))
    return g, l3


def ppo_min_abs_zh(params, batch, bf16_ops=False):
    """Distance of the batch from the kink of the candidate function (see cfo_train.h)."""
    params = np.ascontiguousarray(params, dtype=np.float32)
    return float(cfo().cfo_ppo_min_abs_zh(_p(params), C.byref(batch), int(bool(bf16_ops))))


def ppo_backward_bf16ops_f64(params, batch, bf16_storage=False, map_rows_exact=False):
    """The update's gradients with every matrix-product operand rounded to bf16 (and, with
    bf16_storage, what the bf16 window storage rounds), sums in fp64.  map_rows_exact: the
    map-byte rows of dW_enc multiply the unrounded encoder gradient (split kernels off)."""
    params = np.ascontiguousarray(params, dtype=np.float32)
    g = np.zeros(params.size)
    l3 = np.zeros(3)
    cfo().cfo_ppo_backward_bf16ops_f64(_p(params), C.byref(batch), _p(g), _p(l3),
                                       int(bool(bf16_storage)) | 2 * int(bool(map_rows_exact)))
    return g, l3


# ---- compiled-reference wrappers ------------------------------------------------
class RefEnv:
    """The reference's CPU env (compact-obs build) stepping with its own
    deterministic random-action stream."""

    def __init__(self, num_envs, seed):
        self.n = num_envs
        ref().cfref_init(num_envs, seed)
        assert ref().cfref_obs_bytes() == REC_BYTES

    def step(self):
        ref().cfref_step()

    def records(self):
        buf = (C.c_uint8 * (self.n * REC_BYTES)).from_address(ref().cfref_observations())
        return np.frombuffer(buf, dtype=np.uint8).reshape(self.n, REC_BYTES).copy()

    def terminals(self):
        buf = (C.c_float * self.n).from_address(ref().cfref_terminals())
        return np.frombuffer(buf, dtype=np.float32).copy()

    def view(self, env):
        sc = np.zeros(SCALARS_BYTES, dtype=np.uint8)
        planes = np.zeros(3 * PLANE, dtype=np.uint8)
        ref().cfref_view(env, _p(sc), _p(planes))
        return sc, planes

    def encode(self, env):
        rec = np.zeros(REC_BYTES, dtype=np.uint8)
        ref().cfref_encode(env, _p(rec))
        return rec

    def fuzz(self, env, seed):
        ref().cfref_fuzz_state(env, seed)

    def close(self):
        ref().cfref_free()


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32); k = np.asarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    cfo().cfo_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def philox_uniforms(seed, subsequences, offset):
    """cfo_philox_uniform for one seed/offset over an array of subsequences."""
    lib = cfo()
    return np.array([lib.cfo_philox_uniform(int(seed), int(s), int(offset)) for s in subsequences],
                    dtype=np.float32)


def sample_actions(logits, u):
    """cfo_sample_action row by row: logits [n][A] f32, u [n] f32 ->
    (actions i32[n], logprobs f32[n], margins f32[n])."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    n, A = logits.shape
    act = np.empty(n, dtype=np.int32)
    lp = np.empty(n, dtype=np.float32)
    mg = np.empty(n, dtype=np.float32)
    one = C.c_float()
    lib = cfo()
    for i in range(n):
        act[i] = lib.cfo_sample_action(_p(logits[i]), A, float(u[i]), C.byref(one))
        lp[i] = one.value
        mg[i] = lib.cfo_sample_margin(_p(logits[i]), A, float(u[i]))
    return act, lp, mg
