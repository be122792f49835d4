"""ctypes binding of libcfpolicy.so (the C ABI declared in include/cfp.h).

The library is built in-tree by build.py (hipcc --offload-arch=gfx950).  There
is no fallback: if the shared object is missing or a symbol is absent the
import fails, so a GPU run can never silently measure something else.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcfpolicy.so")

c_f32p = C.POINTER(C.c_float)
c_u8p = C.POINTER(C.c_uint8)
vp = C.c_void_p

# name -> (restype, argtypes); one entry per declaration in include/cfp.h
PROTOTYPES = {
    "cfp_last_error": (C.c_char_p, []),
    "cfp_abi_version": (C.c_int, []),
    "cfp_policy_create": (C.c_int, [C.POINTER(vp), C.c_int, C.c_int, C.c_uint64]),
    "cfp_policy_create_classic": (C.c_int, [C.POINTER(vp), C.c_int, C.c_int, C.c_uint64]),
    "cfp_policy_variant": (C.c_int, [vp]),
    "cfp_policy_destroy": (None, [vp]),
    "cfp_policy_num_envs": (C.c_int, [vp]),
    "cfp_policy_layers": (C.c_int, [vp]),
    "cfp_policy_param_count": (C.c_size_t, [vp]),
    "cfp_policy_set_params": (C.c_int, [vp, vp, C.c_size_t]),
    "cfp_policy_init_reference": (C.c_int, [vp, C.c_uint64]),
    "cfp_policy_get_params": (C.c_int, [vp, vp, C.c_size_t]),
    "cfp_policy_refresh_weights": (C.c_int, [vp, vp]),
    "cfp_save_weights": (C.c_int, [vp, C.c_char_p]),
    "cfp_load_weights": (C.c_int, [vp, C.c_char_p]),
    "cfp_policy_set_gemm_bf16": (C.c_int, [vp, C.c_int]),
    "cfp_policy_gemm_bf16": (C.c_int, [vp]),
    "cfp_policy_set_small_tiles": (C.c_int, [vp, C.c_int]),
    "cfp_policy_small_tiles": (C.c_int, [vp]),
    "cfp_policy_params": (vp, [vp]),
    "cfp_policy_state": (vp, [vp]),
    "cfp_policy_rec": (vp, [vp]),
    "cfp_policy_h_enc": (vp, [vp]),
    "cfp_policy_h3": (vp, [vp]),
    "cfp_policy_logits": (vp, [vp]),
    "cfp_policy_stream": (vp, [vp]),
    "cfp_encode_step": (C.c_int, [vp, vp, C.c_int, vp]),
    "cfp_gru_chain": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, vp]),
    "cfp_head": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "cfp_policy_forward": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int,
                                     C.c_int, vp]),
    "cfp_policy_forward_features": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int,
                                              C.c_int, vp]),
    "cfp_set_gemm_bf16": (C.c_int, [C.c_int]),
    "cfp_get_gemm_bf16": (C.c_int, []),
    "cfp_set_gemm_split": (C.c_int, [C.c_int]),
    "cfp_get_gemm_split": (C.c_int, []),
    "cfp_gemm_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp]),
    "cfp_gemm_enc_fwd": (C.c_int, [C.c_int, vp, vp, vp, vp]),
    "cfp_seam_reserve": (C.c_int, []),
    "cfp_gemm_dh": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp]),
    "cfp_gemm_dh_noalloc": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp]),
    "cfp_gemm_dw": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp]),
    "cfp_gemv_dwv": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "cfp_expand_obs": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int,
                                 C.c_int, vp]),
    "cfp_add_bias": (C.c_int, [vp, vp, C.c_int, vp]),
    "cfp_mingru_epi_fwd": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_int, vp]),
    "cfp_record_obs": (C.c_int, [vp, vp, vp, vp, C.c_size_t, C.c_size_t, vp,
                                 C.c_int, vp]),
    "cfp_record_obs_soa": (C.c_int, [vp, vp, vp, vp, C.c_size_t, C.c_size_t, vp, vp, C.c_int, vp]),
    "cfp_record_obs_soa_list": (C.c_int, [vp, vp, vp, vp, C.c_size_t, C.c_size_t, vp, C.c_size_t,
                                          vp, C.c_int, vp, C.c_int, vp]),
    "cfp_ppo_defaults": (C.c_int, [vp]),
    "cfp_train_create": (C.c_int, [C.POINTER(vp), vp, C.c_int, vp]),
    "cfp_train_destroy": (None, [vp]),
    "cfp_train_buffer": (vp, [vp, C.c_int]),
    "cfp_train_set_bf16_storage": (C.c_int, [vp, C.c_int]),
    "cfp_train_bf16_storage": (C.c_int, [vp]),
    "cfp_train_set_bf16_rstate": (C.c_int, [vp, C.c_int]),
    "cfp_train_bf16_rstate": (C.c_int, [vp]),
    "cfp_train_set_profile": (C.c_int, [vp, C.c_int]),
    "cfp_train_profile": (C.c_int, [vp, C.POINTER(C.c_double), C.c_int]),
    "cfp_train_set_gemm_mode": (C.c_int, [vp, C.c_int, C.c_int]),
    "cfp_train_gemm_mode": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "cfp_train_window": (C.c_int, [vp]),
    "cfp_train_minibatch": (C.c_int, [vp]),
    "cfp_train_record_step": (C.c_int, [vp, C.c_int, vp, vp, vp]),
    "cfp_rollout_step": (C.c_int, [vp, C.c_int, vp, vp, C.c_uint64, vp, vp]),
    "cfp_train_bootstrap": (C.c_int, [vp, vp, vp, vp]),
    "cfp_value_sample": (C.c_int, [vp, C.c_int, C.c_int, vp, vp, vp, vp, C.c_uint64, vp, vp]),
    "cfp_record_rd": (C.c_int, [vp, vp, vp, vp, C.c_int, vp]),
    "cfp_train_gae": (C.c_int, [vp]*2),
    "cfp_train_adv_stats": (C.c_int, [vp]*2),
    "cfp_train_backward": (C.c_int, [vp, C.c_int, C.c_int, vp]),
    "cfp_train_zero_loss": (C.c_int, [vp]*2),
    "cfp_train_adam": (C.c_int, [vp]*2),
    "cfp_train_update": (C.c_int, [vp, C.c_int, vp]),
    "cfp_train_loss": (C.c_int, [vp, vp, vp]),
    "cfp_synth_classic_records": (C.c_int, [vp, C.c_int, C.c_uint64, C.c_uint64, vp]),
    "cfp_synth_records": (C.c_int, [vp, C.c_int, C.c_uint64, C.c_uint64, vp]),
    # include/cfp_env.h
    "cfp_env_state_bytes": (C.c_size_t, []),
    "cfp_env_create": (C.c_int, [C.POINTER(vp), C.c_int, C.c_int]),
    "cfp_env_destroy": (None, [vp]),
    "cfp_env_num_envs": (C.c_int, [vp]),
    "cfp_env_pool_size": (C.c_int, [vp]),
    "cfp_env_init": (C.c_int, [vp, C.c_uint64, vp]),
    "cfp_env_reset": (C.c_int, [vp, vp]),
    "cfp_env_pool_fill": (C.c_int, [vp, C.c_uint64, vp]),
    "cfp_env_generate_host": (C.c_int, [C.c_uint32, C.c_int, vp]),
    "cfp_env_import": (C.c_int, [vp, C.c_int, C.c_int, vp]),
    "cfp_env_export": (C.c_int, [vp, C.c_int, C.c_int, vp]),
    "cfp_env_pool_import": (C.c_int, [vp, C.c_int, C.c_int, vp]),
    "cfp_env_light_table": (C.c_int, [vp, C.c_int]),
    "cfp_env_step": (C.c_int, [vp, vp, vp, vp, vp]),
    "cfp_env_seed_actions": (C.c_int, [vp, C.c_uint64, vp]),
    "cfp_env_reset_count": (vp, [vp]),
    "cfp_env_reset_list": (vp, [vp]),
    "cfp_env_fetch_resets": (C.c_int, [vp, vp, C.c_int, C.POINTER(C.c_int), vp]),
    "cfp_env_reset_from_pool": (C.c_int, [vp, vp]),
    "cfp_env_view": (C.c_int, [vp, vp, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp),
                               C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "cfp_env_record_obs": (C.c_int, [vp, vp, vp]),
    "cfp_env_actions": (vp, [vp]),
    "cfp_env_rewards": (vp, [vp]),
    "cfp_env_terminals": (vp, [vp]),
    "cfp_env_rollout_step": (C.c_int, [vp, vp, C.c_int, C.c_uint64, vp]),
    "cfp_env_run_step": (C.c_int, [vp, vp, C.c_uint64, vp]),
    "cfp_env_run_actions": (vp, [vp]),
    "cfp_env_run_logprobs": (vp, [vp]),
    "cfp_env_run_values": (vp, [vp]),
    "cfp_env_run_counter": (vp, [vp]),
    "cfp_train_collect": (C.c_int, [vp, vp, C.c_uint64, vp]),
}


class PpoConfig(C.Structure):
    """cfp_ppo_config of include/cfp.h."""
    _fields_ = [("lr", C.c_float), ("gamma", C.c_float), ("lam", C.c_float),
                ("clip", C.c_float), ("ent", C.c_float), ("vf", C.c_float),
                ("epochs", C.c_int), ("minibatches", C.c_int), ("bptt_split", C.c_int),
                ("bwd_win", C.c_int)]


BUF = {name: i for i, name in enumerate(
    ["r_obs", "r_state", "r_act", "r_logprob", "r_value", "r_reward", "r_done", "adv",
     "ret", "v_boot", "stats", "loss_acc", "grads", "adam_m", "adam_v", "lr", "ent", "step_ctr"])}


class CfpError(RuntimeError):
    pass


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import "
            "__graft_entry__ as g; g.build()'` (hipcc, gfx950); there is no "
            "CPU fallback for the policy path")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)   # AttributeError = header/library mismatch
        fn.restype = res
        fn.argtypes = args
    return lib


def check(lib, rc):
    if rc != 0:
        raise CfpError(lib.cfp_last_error().decode("utf-8", "replace"))
