"""Host-side mirror of the reference's CuPolicy call surface over the C ABI.

Names follow craftax_full.cu: encode_step (:11931), gru_chain (:11978), the
policy half of rollout_step (:12022) and the GEMM wrappers (:11604-11666).
PyTorch is used only to own device memory and streams; every computation is a
call into libcfpolicy.so.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib

HIDDEN, GRU, OBS, OBS_MAP, OBS_TAIL = 256, 768, 843, 792, 51
REC_BYTES, ACTIONS, AV = 996, 43, 44
CLASSIC_OBS, CLASSIC_REC_BYTES, CLASSIC_ACTIONS, CLASSIC_AV = 1345, 148, 17, 18

_cfp = None


def lib():
    global _cfp
    if _cfp is None:
        _cfp = _lib.load()
    return _cfp


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc):
    _lib.check(lib(), rc)


def param_offsets(layers):
    """Flat arena layout, craftax_full.cu:9094-9102."""
    o = {"W_enc": 0, "b_enc": OBS * HIDDEN}
    o["W_gru"] = o["b_enc"] + HIDDEN
    o["W_a"] = o["W_gru"] + layers * GRU * HIDDEN
    o["b_a"] = o["W_a"] + ACTIONS * HIDDEN
    o["W_v"] = o["b_a"] + ACTIONS
    o["b_v"] = o["W_v"] + HIDDEN
    o["count"] = o["b_v"] + 1
    return o


def split_params(params, layers):
    """Views of a flat host params array, shaped as the reference documents them."""
    o = param_offsets(layers)
    p = np.asarray(params)
    return {
        "W_enc": p[o["W_enc"]:o["b_enc"]].reshape(OBS, HIDDEN),
        "b_enc": p[o["b_enc"]:o["W_gru"]],
        "W_gru": p[o["W_gru"]:o["W_a"]].reshape(layers, GRU, HIDDEN),
        "W_a": p[o["W_a"]:o["b_a"]].reshape(ACTIONS, HIDDEN),
        "b_a": p[o["b_a"]:o["W_v"]],
        "W_v": p[o["W_v"]:o["b_v"]],
        "b_v": p[o["b_v"]:o["count"]],
    }


class Policy:
    """cfp_policy handle (CuPolicy, craftax_full.cu:11758)."""

    def __init__(self, num_envs, layers=3, seed=1, variant="full"):
        """variant "full": 996-byte records, 43 actions; "classic": 148-byte records,
        17 actions, gathered-column encoder (Rollout, main_classic.cu:326)."""
        self._h = C.c_void_p()
        assert variant in ("full", "classic")
        create = lib().cfp_policy_create if variant == "full" else lib().cfp_policy_create_classic
        _check(create(C.byref(self._h), num_envs, layers, seed))
        self.n = num_envs
        self.layers = layers
        self.variant = variant
        self.rec_bytes = REC_BYTES if variant == "full" else CLASSIC_REC_BYTES
        self.av_width = AV if variant == "full" else CLASSIC_AV
        self.param_count = lib().cfp_policy_param_count(self._h)

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            lib().cfp_policy_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:   # interpreter shutdown: module globals may be gone
            pass

    # -- parameters ----------------------------------------------------
    def set_params(self, host_params):
        a = np.ascontiguousarray(host_params, dtype=np.float32)
        _check(lib().cfp_policy_set_params(self._h, a.ctypes.data_as(C.c_void_p), a.size))

    def init_reference(self, seed=1234):
        """The reference's weight initialisation (cu_policy_init :11830-11845)."""
        _check(lib().cfp_policy_init_reference(self._h, int(seed)))

    def get_params(self):
        a = np.empty(self.param_count, dtype=np.float32)
        _check(lib().cfp_policy_get_params(self._h, a.ctypes.data_as(C.c_void_p), a.size))
        return a

    def refresh_weights(self):
        _check(lib().cfp_policy_refresh_weights(self._h, _stream()))

    def save_weights(self, path):
        """CFW1 checkpoint (cu_save_weights, craftax_full.cu:12248)."""
        _check(lib().cfp_save_weights(self._h, str(path).encode()))

    def load_weights(self, path):
        _check(lib().cfp_load_weights(self._h, str(path).encode()))

    def set_gemm_bf16(self, on=True):
        """Run the forward entry points with bf16 GEMM inputs and fp32 accumulation
        (the reference's CF_GEMM_BF16 mode, craftax_full.cu:11306-11316)."""
        _check(lib().cfp_policy_set_gemm_bf16(self._h, 1 if on else 0))

    def set_small_tiles(self, on=True):
        """16-env tiles for batches of at most 4096 envs (cfp_policy_set_small_tiles)."""
        _check(lib().cfp_policy_set_small_tiles(self._h, 1 if on else 0))

    @property
    def gemm_bf16(self):
        return bool(lib().cfp_policy_gemm_bf16(self._h))

    # -- forward entry points ------------------------------------------------
    def encode_step(self, rec=None, n=None):
        """records [n][996] u8 (None = the object's scratch) -> the object's h_enc."""
        if rec is not None:
            n = rec.shape[0]
        elif n is None:
            n = self.n
        _check(lib().cfp_encode_step(self._h, _ptr(rec), n, _stream()))
        return self.h_enc[:n]

    # -- library-owned device buffers, viewed as tensors (no copy) ---------------
    @property
    def params(self):
        return _wrap(lib().cfp_policy_params(self._h), (self.param_count,), "<f4")

    @property
    def state(self):
        return _wrap(lib().cfp_policy_state(self._h), (self.layers, self.n, HIDDEN), "<f4")

    @property
    def rec(self):
        return _wrap(lib().cfp_policy_rec(self._h), (self.n, self.rec_bytes), "|u1")

    @property
    def h_enc(self):
        return _wrap(lib().cfp_policy_h_enc(self._h), (self.n, HIDDEN), "<f4")

    @property
    def h3(self):
        return _wrap(lib().cfp_policy_h3(self._h), (self.n, HIDDEN), "<f4")

    @property
    def logits(self):
        return _wrap(lib().cfp_policy_logits(self._h), (self.n, self.av_width), "<f4")

    def gru_chain(self, x0, state, terminals, r_state_t=None, h3=None, chunk=0):
        n = x0.shape[0]
        if h3 is None:
            h3 = torch.empty((n, HIDDEN), dtype=torch.float32, device=x0.device)
        _check(lib().cfp_gru_chain(self._h, _ptr(x0), _ptr(state), _ptr(terminals),
                                   _ptr(r_state_t), _ptr(h3), n, chunk, _stream()))
        return h3

    def head(self, h3, av=None):
        n = h3.shape[0]
        if av is None:
            av = torch.empty((n, self.av_width), dtype=torch.float32, device=h3.device)
        _check(lib().cfp_head(self._h, _ptr(h3), _ptr(av), n, _stream()))
        return av

    def forward(self, rec, terminals, state, r_state_t=None, h_enc=None, h3=None,
                av=None, chunk=0):
        """Policy half of rollout_step: records -> logits/value, state updated in place."""
        n = rec.shape[0]
        if av is None:
            av = torch.empty((n, self.av_width), dtype=torch.float32, device=rec.device)
        _check(lib().cfp_policy_forward(self._h, _ptr(rec), _ptr(terminals), _ptr(state),
                                        _ptr(r_state_t), _ptr(h_enc), _ptr(h3),
                                        _ptr(av), n, chunk, _stream()))
        return av


    def forward_features(self, xobs, terminals, state, r_state_t=None, h_enc=None, h3=None,
                         av=None, chunk=0):
        """The same step from the fp32 feature matrix xobs[n][843] (cu_gemm_enc_fwd on
        xobs + bias, then the fused layers and heads)."""
        n = xobs.shape[0]
        if av is None:
            av = torch.empty((n, self.av_width), dtype=torch.float32, device=xobs.device)
        _check(lib().cfp_policy_forward_features(self._h, _ptr(xobs), _ptr(terminals), _ptr(state),
                                                 _ptr(r_state_t), _ptr(h_enc), _ptr(h3), _ptr(av),
                                                 n, chunk, _stream()))
        return av


class Trainer:
    """cfp_trainer handle (CuTrain, craftax_full.cu:12688): rollout slabs, windowed
    recompute backward, GAE, Adam."""

    def __init__(self, policy, T, **cfg):
        self.policy = policy
        self.cfg = _lib.PpoConfig()
        _check(lib().cfp_ppo_defaults(C.byref(self.cfg)))
        for k, v in cfg.items():
            assert hasattr(self.cfg, k), k
            setattr(self.cfg, k, v)
        self._h = C.c_void_p()
        _check(lib().cfp_train_create(C.byref(self._h), policy._h, T, C.byref(self.cfg)))
        self.T, self.n, self.layers = T, policy.n, policy.layers
        self.mb = lib().cfp_train_minibatch(self._h)
        self.window = lib().cfp_train_window(self._h)

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            lib().cfp_train_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def buf(self, name):
        T, n, L = self.T, self.n, self.layers
        shapes = {
            "r_obs": ((T, n, REC_BYTES), "|u1"), "r_state": ((T, L, n, HIDDEN), "<f4"),
            "r_act": ((T, n), "<i4"), "r_logprob": ((T, n), "<f4"),
            "r_value": ((T, n), "<f4"), "r_reward": ((T, n), "<f4"),
            "r_done": ((T, n), "|u1"), "adv": ((T, n), "<f4"), "ret": ((T, n), "<f4"),
            "v_boot": ((n,), "<f4"), "stats": ((2,), "<f8"), "loss_acc": ((3,), "<f8"),
            "grads": ((self.policy.param_count,), "<f4"),
            "adam_m": ((self.policy.param_count,), "<f4"),
            "adam_v": ((self.policy.param_count,), "<f4"), "lr": ((1,), "<f4"),
            "ent": ((1,), "<f4"), "step_ctr": ((1,), "<i8"),
        }
        shape, ts = shapes[name]
        return _wrap(lib().cfp_train_buffer(self._h, _lib.BUF[name]), shape, ts)

    def record_step(self, t, rec, terminals):
        _check(lib().cfp_train_record_step(self._h, t, _ptr(rec), _ptr(terminals), _stream()))

    def rollout_step(self, t, rec, prev_terminals, seed, env_actions=None):
        """Policy half of cu_rollout_step: forward + sample into the slab rows of step t."""
        _check(lib().cfp_rollout_step(self._h, t, _ptr(rec), _ptr(prev_terminals), seed,
                                      _ptr(env_actions), _stream()))

    def bootstrap(self, rec, terminals):
        """V(s_T) on a copy of the live state -> v_boot."""
        _check(lib().cfp_train_bootstrap(self._h, _ptr(rec), _ptr(terminals), _stream()))

    def set_bf16_storage(self, on=True):
        """bf16 storage of the window workspace (in effect with bf16 GEMM inputs only)."""
        _check(lib().cfp_train_set_bf16_storage(self._h, 1 if on else 0))

    def set_bf16_rstate(self, on=True):
        """The r_state slab as bf16 (cfp_train_set_bf16_rstate): bf16 forward and bf16 update only."""
        _check(lib().cfp_train_set_bf16_rstate(self._h, 1 if on else 0))

    def set_profile(self, on=True):
        """Phase timers of collect / update (cfp_train_set_profile); the update then runs eagerly."""
        _check(lib().cfp_train_set_profile(self._h, 1 if on else 0))

    def profile(self, reset=False):
        """Accumulated milliseconds per phase: rollout, gae, backward, adam."""
        ms = (C.c_double * 4)()
        _check(lib().cfp_train_profile(self._h, ms, 1 if reset else 0))
        return dict(zip(("rollout", "gae", "backward", "adam"), (float(x) for x in ms)))

    def set_gemm_mode(self, bf16=-1, split=-1):
        """This trainer's own GEMM mode (cfp_train_set_gemm_mode); -1 follows the process-wide switch."""
        _check(lib().cfp_train_set_gemm_mode(self._h, int(bf16), int(split)))

    def gemm_mode(self):
        """(bf16, split) the next update of this trainer runs with."""
        b, s_ = C.c_int(), C.c_int()
        _check(lib().cfp_train_gemm_mode(self._h, C.byref(b), C.byref(s_)))
        return b.value, s_.value

    def gae(self):
        _check(lib().cfp_train_gae(self._h, _stream()))

    def adv_stats(self):
        _check(lib().cfp_train_adv_stats(self._h, _stream()))

    def backward(self, env_start=0, env_count=None):
        _check(lib().cfp_train_backward(self._h, env_start,
                                        self.mb if env_count is None else env_count,
                                        _stream()))

    def zero_loss(self):
        _check(lib().cfp_train_zero_loss(self._h, _stream()))

    def adam(self):
        _check(lib().cfp_train_adam(self._h, _stream()))

    def update(self, use_graph=False):
        """cu_train_update (craftax_full.cu:13372) over the stored rollout."""
        _check(lib().cfp_train_update(self._h, 1 if use_graph else 0, _stream()))

    def loss(self):
        out = np.zeros(4)
        _check(lib().cfp_train_loss(self._h, out.ctypes.data_as(C.c_void_p), _stream()))
        return out


class _DevBuf:
    """Borrowed device memory exposed through __cuda_array_interface__."""

    def __init__(self, ptr, shape, typestr):
        self.__cuda_array_interface__ = {
            "shape": tuple(shape), "typestr": typestr, "data": (int(ptr), False),
            "version": 2, "strides": None}


def _wrap(ptr, shape, typestr):
    return torch.as_tensor(_DevBuf(ptr, shape, typestr), device="cuda")


# -- the dense-math seam -------------------------------------------------------
def set_gemm_bf16(on=True):
    """Process-wide: bf16 inputs / fp32 accumulation for cfp_gemm_* and the PPO update
    (the reference's CF_GEMM_BF16, craftax_full.cu:11306-11316)."""
    _check(lib().cfp_set_gemm_bf16(1 if on else 0))


def set_gemm_split(mode=1):
    """Process-wide: fp32 GEMMs of the update's shapes on the bf16 pipe.  1 (default):
    nine exact bf16 partial products per product; 2: the six largest; 0: fp32 MFMA
    everywhere."""
    _check(lib().cfp_set_gemm_split(int(mode)))


def gemm_fwd(W, x, y=None):
    """y[cols][m] = x[cols][k] . W[m][k]^T (cu_gemm_fwd :11604)."""
    m, k = W.shape
    cols = x.shape[0]
    if y is None:
        y = torch.empty((cols, m), dtype=torch.float32, device=x.device)
    _check(lib().cfp_gemm_fwd(m, cols, k, _ptr(W), _ptr(x), _ptr(y), _stream()))
    return y


def gemm_enc_fwd(W_enc, xobs, h=None):
    cols = xobs.shape[0]
    if h is None:
        h = torch.empty((cols, HIDDEN), dtype=torch.float32, device=xobs.device)
    _check(lib().cfp_gemm_enc_fwd(cols, _ptr(W_enc), _ptr(xobs), _ptr(h), _stream()))
    return h


def gemm_dh(W, dpre, dh=None):
    m3 = W.shape[0]
    cols = dpre.shape[0]
    if dh is None:
        dh = torch.empty((cols, HIDDEN), dtype=torch.float32, device=dpre.device)
    _check(lib().cfp_gemm_dh(m3, cols, _ptr(W), _ptr(dpre), _ptr(dh), _stream()))
    return dh


def gemm_dh_noalloc(W, dpre, dh):
    """cfp_gemm_dh_noalloc: as gemm_dh, the W mirror in the library's own device array;
    the caller brings the output (nothing is allocated on the way)."""
    _check(lib().cfp_gemm_dh_noalloc(W.shape[0], dpre.shape[0], _ptr(W), _ptr(dpre), _ptr(dh),
                                     _stream()))
    return dh


def seam_reserve():
    _check(lib().cfp_seam_reserve())


def gemm_dw(x, dpre, dW):
    """dW[rows][256] += dpre[cols][rows]^T . x[cols][256] (cu_gemm_dw :11642)."""
    cols, rows = dpre.shape
    _check(lib().cfp_gemm_dw(rows, cols, _ptr(x), _ptr(dpre), _ptr(dW), _stream()))
    return dW


def gemv_dwv(x, dv, dWv):
    cols = x.shape[0]
    _check(lib().cfp_gemv_dwv(_ptr(x), _ptr(dv), _ptr(dWv), cols, _stream()))
    return dWv


def expand_obs(r_obs, count, t0=0, mb=None, n=None, env_start=0, xobs=None):
    """k_expand_obs (:10028): records -> fp32 features [count][843]."""
    flat = r_obs.reshape(-1, REC_BYTES)
    if n is None:
        n = flat.shape[0]
    if mb is None:
        mb = count
    if xobs is None:
        xobs = torch.empty((count, OBS), dtype=torch.float32, device=r_obs.device)
    _check(lib().cfp_expand_obs(_ptr(flat), _ptr(xobs), t0, count, mb, n, env_start,
                                _stream()))
    return xobs


def add_bias(h, b):
    _check(lib().cfp_add_bias(_ptr(h), _ptr(b), h.shape[0], _stream()))
    return h


def mingru_epi_fwd(pre, x, state, terminals, r_state_store=None, h_out=None):
    cols = x.shape[0]
    if h_out is None:
        h_out = torch.empty_like(x)
    _check(lib().cfp_mingru_epi_fwd(_ptr(pre), _ptr(x), _ptr(state), _ptr(h_out),
                                    _ptr(r_state_store), _ptr(terminals), cols, _stream()))
    return h_out


def record_obs(scalars_u8, maps, item_maps, light_maps, n, env_stride, level_stride,
               rec=None):
    """k_record_obs (:9284): encoder-input state -> [n][996] records."""
    if rec is None:
        rec = torch.empty((n, REC_BYTES), dtype=torch.uint8, device=maps.device)
    _check(lib().cfp_record_obs(_ptr(scalars_u8), _ptr(maps), _ptr(item_maps),
                                _ptr(light_maps), env_stride, level_stride, _ptr(rec),
                                n, _stream()))
    return rec


# field arrays of cfp_env_soa in declaration order: (name, entries per env)
ENV_SOA_FIELDS = (
    ("player_position", 2), ("player_level", 1), ("player_direction", 1), ("player_health", 1),
    ("player_food", 1), ("player_drink", 1), ("player_energy", 1), ("player_mana", 1),
    ("player_xp", 1), ("player_dexterity", 1), ("player_strength", 1), ("player_intelligence", 1),
    ("is_sleeping", 1), ("is_resting", 1), ("inv_wood", 1), ("inv_stone", 1), ("inv_coal", 1),
    ("inv_iron", 1), ("inv_diamond", 1), ("inv_sapphire", 1), ("inv_ruby", 1), ("inv_sapling", 1),
    ("inv_torches", 1), ("inv_arrows", 1), ("inv_books", 1), ("inv_pickaxe", 1), ("inv_sword", 1),
    ("inv_bow", 1), ("inv_potions", 6), ("inv_armour", 4), ("sword_enchantment", 1),
    ("bow_enchantment", 1), ("armour_enchantments", 4), ("light_level", 1), ("learned_spells", 2),
    ("monsters_killed", 9), ("boss_timesteps_to_spawn_this_round", 1), ("mob_type_id", 135),
    ("mob_mask", 135), ("mob_position", 270))


def _env_soa_view(arrays, n_stride):
    """cfp_env_soa for a dict of device tensors, one per field, each [entries][n_stride]."""
    import ctypes as C
    fields = [(name, C.c_void_p) for name, _ in ENV_SOA_FIELDS] + [("n_stride", C.c_size_t)]
    view = type("cfp_env_soa", (C.Structure,), {"_fields_": fields})()
    for name, k in ENV_SOA_FIELDS:
        t = arrays[name]
        assert t.is_contiguous() and t.numel() == k * n_stride, name
        setattr(view, name, t.data_ptr())
    view.n_stride = n_stride
    return view


def record_obs_soa(arrays, n_stride, maps, item_maps, light_maps, n, env_stride, level_stride,
                   skip=None, rec=None):
    """k_record_obs (:9284) from the reference's per-field device arrays."""
    import ctypes as C
    if rec is None:
        rec = torch.empty((n, REC_BYTES), dtype=torch.uint8, device=maps.device)
    view = _env_soa_view(arrays, n_stride)
    _check(lib().cfp_record_obs_soa(C.addressof(view), _ptr(maps), _ptr(item_maps), _ptr(light_maps),
                                    env_stride, level_stride, _ptr(skip), _ptr(rec), n, _stream()))
    return rec


def record_obs_soa_list(arrays, n_stride, maps, item_maps, light_maps, n, env_stride, level_stride,
                        env_list, list_stride, count, max_count, rec):
    """k_record_obs_list (:9303): only the envs named by the first *count list entries."""
    import ctypes as C
    view = _env_soa_view(arrays, n_stride)
    _check(lib().cfp_record_obs_soa_list(C.addressof(view), _ptr(maps), _ptr(item_maps),
                                         _ptr(light_maps), env_stride, level_stride, _ptr(env_list),
                                         list_stride, _ptr(count), max_count, _ptr(rec), n,
                                         _stream()))
    return rec


def value_sample(av, seed, step_ctr=None, env_actions=None):
    """k_value_sample (:9714): av [n][A+1] -> (actions i32[n], logprobs f32[n], values f32[n])."""
    n, w = av.shape
    act = torch.empty(n, dtype=torch.int32, device=av.device)
    lp = torch.empty(n, dtype=torch.float32, device=av.device)
    val = torch.empty(n, dtype=torch.float32, device=av.device)
    _check(lib().cfp_value_sample(_ptr(av), n, w - 1, _ptr(env_actions), _ptr(act), _ptr(lp),
                                  _ptr(val), seed, _ptr(step_ctr), _stream()))
    return act, lp, val


def record_rd(rewards, terminals, r_reward_row, r_done_row):
    _check(lib().cfp_record_rd(_ptr(rewards), _ptr(terminals), _ptr(r_reward_row),
                               _ptr(r_done_row), rewards.shape[0], _stream()))


def synth_classic_records(n, seed, step, rec=None, device="cuda"):
    if rec is None:
        rec = torch.empty((n, CLASSIC_REC_BYTES), dtype=torch.uint8, device=device)
    _check(lib().cfp_synth_classic_records(_ptr(rec), n, seed, step, _stream()))
    return rec


def synth_records(n, seed, step, rec=None, device="cuda"):
    if rec is None:
        rec = torch.empty((n, REC_BYTES), dtype=torch.uint8, device=device)
    _check(lib().cfp_synth_records(_ptr(rec), n, seed, step, _stream()))
    return rec
