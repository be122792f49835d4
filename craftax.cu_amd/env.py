"""Host-side mirror of the reference's env vector (CuVec, craftax_full.cu:10688-10946) over
the C ABI of include/cfp_env.h.  PyTorch owns the caller-side device buffers; every
computation is a call into libcfpolicy.so."""
import ctypes as C

import numpy as np
import torch

from . import _lib
from .policy import REC_BYTES, _check, _ptr, _stream, _wrap, lib


class Env:
    """cfp_env handle: `n` envs resident on the GPU, optionally with a pool of reset states."""

    def __init__(self, num_envs, pool=0):
        self._h = C.c_void_p()
        _check(lib().cfp_env_create(C.byref(self._h), num_envs, pool))
        self.n = num_envs
        self.pool = pool
        # the env vector's own slots (CuVec.d_actions / d_rewards / d_terminals)
        self.actions = _wrap(lib().cfp_env_actions(self._h), (num_envs,), "<f4")
        self.rewards = _wrap(lib().cfp_env_rewards(self._h), (num_envs,), "<f4")
        self.terminals = _wrap(lib().cfp_env_terminals(self._h), (num_envs,), "<f4")

    def close(self):
        if self._h:
            lib().cfp_env_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def state_bytes():
        return lib().cfp_env_state_bytes()

    def import_states(self, states, first=0):
        """states: contiguous numpy structured array of cfp_env_state records."""
        s = np.ascontiguousarray(states)
        assert s.dtype.itemsize == self.state_bytes()
        _check(lib().cfp_env_import(self._h, first, len(s), C.c_void_p(s.ctypes.data)))

    def import_pool(self, states, first=0):
        s = np.ascontiguousarray(states)
        assert s.dtype.itemsize == self.state_bytes()
        _check(lib().cfp_env_pool_import(self._h, first, len(s), C.c_void_p(s.ctypes.data)))

    def export_states(self, dtype, first=0, count=None):
        count = self.n - first if count is None else count
        out = np.zeros(count, dtype)
        assert out.dtype.itemsize == self.state_bytes()
        _check(lib().cfp_env_export(self._h, first, count, C.c_void_p(out.ctypes.data)))
        return out

    def init(self, seed):
        """k_env_init: env i = the env created from seed + i, worlds generated on the device."""
        _check(lib().cfp_env_init(self._h, seed, _stream()))

    def reset(self):
        """k_reset_list_block: new worlds for the envs on the reset list."""
        _check(lib().cfp_env_reset(self._h, _stream()))

    def pool_fill(self, seed=0):
        _check(lib().cfp_env_pool_fill(self._h, seed, _stream()))

    def seed_actions(self, seed):
        _check(lib().cfp_env_seed_actions(self._h, seed, _stream()))

    def step(self, actions=None):
        """k_step: one game step; actions float32[n] on the device, or None for the env's own
        xorshift32 % 43 stream.  Results land in self.rewards / self.terminals."""
        _check(lib().cfp_env_step(self._h, _ptr(actions), _ptr(self.rewards), _ptr(self.terminals), _stream()))

    def reset_list(self):
        """(count, records[count] as int32 (env, key0, key1) rows) of the last step, on the host."""
        recs = np.zeros((self.n, 3), np.int32)
        cnt = C.c_int(0)
        _check(lib().cfp_env_fetch_resets(self._h, C.c_void_p(recs.ctypes.data), self.n, C.byref(cnt), _stream()))
        return cnt.value, recs[:cnt.value]

    def reset_from_pool(self):
        _check(lib().cfp_env_reset_from_pool(self._h, _stream()))

    def rollout_step(self, trainer, t, seed):
        """cu_rollout_step with this env vector: record, policy forward + sample, env step,
        reward / done rows, pool reset."""
        _check(lib().cfp_env_rollout_step(trainer._h, self._h, t, seed, _stream()))

    def run_step(self, policy, seed):
        """cu_rollout_step_plain: the `run` mode's step (no slabs); results in run_actions /
        run_logprobs / run_values."""
        _check(lib().cfp_env_run_step(policy._h, self._h, seed, _stream()))

    def run_outputs(self):
        """(actions int32[n], logprobs f32[n], values f32[n], step counter u64[1]) of the run mode."""
        n = self.n
        return (_wrap(lib().cfp_env_run_actions(self._h), (n,), "<i4"),
                _wrap(lib().cfp_env_run_logprobs(self._h), (n,), "<f4"),
                _wrap(lib().cfp_env_run_values(self._h), (n,), "<f4"),
                _wrap(lib().cfp_env_run_counter(self._h), (1,), "<i8"))

    def collect(self, trainer, seed):
        """cu_train_collect: T rollout steps, bootstrap value, GAE."""
        _check(lib().cfp_train_collect(trainer._h, self._h, seed, _stream()))

    def record_obs(self, rec_row=None):
        if rec_row is None:
            rec_row = torch.empty(self.n, REC_BYTES, dtype=torch.uint8, device=self.rewards.device)
        _check(lib().cfp_env_record_obs(self._h, _ptr(rec_row), _stream()))
        return rec_row


def generate_host(dtype, seed, count):
    """States of envs created from seed, seed + 1, ... generated on the host."""
    out = np.zeros(count, dtype)
    assert out.dtype.itemsize == Env.state_bytes()
    _check(lib().cfp_env_generate_host(seed, count, C.c_void_p(out.ctypes.data)))
    return out


def light_table(count=100001):
    out = np.zeros(count, np.float32)
    _check(lib().cfp_env_light_table(C.c_void_p(out.ctypes.data), count))
    return out
