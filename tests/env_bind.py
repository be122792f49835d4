"""ctypes/numpy helpers for the env-step tests: the exchange struct cfp_env_state
(include/cfp_env.h) as a numpy dtype, the compiled reference (oracle/_ref) stepped env by
env, and the host build of the library's step text (oracle/libcfenvhost.so).  Test
infrastructure only."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)

L, M = 9, 48
STATE_DTYPE = np.dtype([
    ("player_position", "<i4", (2,)), ("player_level", "<i4"), ("player_direction", "<i4"),
    ("player_health", "<f4"), ("player_food", "<i4"), ("player_drink", "<i4"),
    ("player_energy", "<i4"), ("player_mana", "<i4"), ("is_sleeping", "<i4"), ("is_resting", "<i4"),
    ("player_recover", "<f4"), ("player_hunger", "<f4"), ("player_thirst", "<f4"),
    ("player_fatigue", "<f4"), ("player_recover_mana", "<f4"),
    ("player_xp", "<i4"), ("player_dexterity", "<i4"), ("player_strength", "<i4"),
    ("player_intelligence", "<i4"),
    ("wood", "<i4"), ("stone", "<i4"), ("coal", "<i4"), ("iron", "<i4"), ("diamond", "<i4"),
    ("sapling", "<i4"), ("pickaxe", "<i4"), ("sword", "<i4"), ("bow", "<i4"), ("arrows", "<i4"),
    ("armour", "<i4", (4,)), ("torches", "<i4"), ("ruby", "<i4"), ("sapphire", "<i4"),
    ("potions", "<i4", (6,)), ("books", "<i4"),
    ("mob_position", "<i4", (5, L, 3, 2)), ("mob_health", "<f4", (5, L, 3)),
    ("mob_attack_cooldown", "<i4", (5, L, 3)), ("mob_type_id", "<i4", (5, L, 3)),
    ("mob_mask", "<i4", (5, L, 3)),
    ("mob_projectile_directions", "<i4", (L, 3, 2)), ("player_projectile_directions", "<i4", (L, 3, 2)),
    ("growing_plants_positions", "<i4", (10, 2)), ("growing_plants_age", "<i4", (10,)),
    ("growing_plants_mask", "<i4", (10,)),
    ("potion_mapping", "<i4", (6,)), ("learned_spells", "<i4", (2,)),
    ("sword_enchantment", "<i4"), ("bow_enchantment", "<i4"), ("armour_enchantments", "<i4", (4,)),
    ("boss_progress", "<i4"), ("boss_timesteps_to_spawn_this_round", "<i4"),
    ("light_level", "<f4"), ("state_rng", "<u4", (2,)), ("timestep", "<i4"),
    ("down_ladders", "<i4", (L, 2)), ("up_ladders", "<i4", (L, 2)),
    ("monsters_killed", "<i4", (L,)), ("chests_opened", "<i4", (L,)),
    ("rng_key", "<u4", (2,)),
    ("achievements", "u1", (67,)), ("pad_", "u1", (5,)),
    ("mob_bits", "<u8", (L, M)), ("spawn_all_bits", "<u8", (L, M)),
    ("spawn_grave_bits", "<u8", (L, M)), ("spawn_water_bits", "<u8", (L, M)),
    ("map", "u1", (L, M, M)), ("item_map", "u1", (L, M, M)), ("light_map", "u1", (L, M, M)),
])
FLOAT_FIELDS = [n for n in STATE_DTYPE.names if STATE_DTYPE[n].base == np.dtype("<f4")]


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def diff_fields(a, b):
    """Names of the fields in which two state arrays differ (floats by bit pattern)."""
    out = []
    for n in STATE_DTYPE.names:
        if n == "pad_":
            continue
        x, y = a[n], b[n]
        if x.dtype == np.float32:
            x, y = x.view(np.uint32), y.view(np.uint32)
        if not np.array_equal(x, y):
            out.append(n)
    return out


# floor -> what half of its envs are put in front of (block id where it is a block)
DEEP_ENCOUNTERS = {0: 16, 2: 10, 3: 21, 4: 22, 5: 29, 7: None, 8: 32}


def deep_states(ref, n, seed):
    """n reference worlds (ref.init) with the player moved onto floor e % 9 at that floor's
    up ladder and given what a long episode collects: tools, weapons, arrows, torches, ores,
    potions, books, armour with enchantments, spells, attribute points, kills on every floor,
    a boss fight in progress on floor 8, a random hour of the day.  Random-action rollouts from
    the freshly generated worlds rarely leave floors 0..2; these states put every floor's mob
    table, the ranged mobs and their projectiles, spells, enchanting and the boss on the path.
    The states are imported into the reference env (slot e) and returned."""
    ref.init(n, seed)
    st = ref.export()
    rng = np.random.default_rng(seed)
    for e in range(n):
        s = st[e]
        lvl = e % L
        s["player_level"] = lvl
        if lvl > 0:
            s["player_position"] = s["up_ladders"][lvl]
        s["player_direction"] = rng.integers(1, 5)
        s["player_health"] = np.float32(rng.integers(4, 10))
        for f in ("player_food", "player_drink", "player_energy", "player_mana"):
            s[f] = rng.integers(3, 10)
        for f in ("player_dexterity", "player_strength", "player_intelligence"):
            s[f] = rng.integers(1, 6)
        s["player_xp"] = rng.integers(0, 4)
        for f in ("wood", "stone", "coal", "iron", "diamond", "sapling", "ruby", "sapphire"):
            s[f] = rng.integers(0, 10)
        s["pickaxe"] = rng.integers(0, 5)
        s["sword"] = rng.integers(0, 5)
        s["bow"] = rng.integers(0, 2)
        s["arrows"] = rng.integers(0, 20)
        s["torches"] = rng.integers(0, 10)
        s["books"] = rng.integers(0, 3)
        s["potions"] = rng.integers(0, 4, 6)
        s["armour"] = rng.integers(0, 3, 4)
        s["armour_enchantments"] = np.where(s["armour"] > 0, rng.integers(0, 3, 4), 0)
        s["sword_enchantment"] = rng.integers(0, 3) if s["sword"] > 0 else 0
        s["bow_enchantment"] = rng.integers(0, 3) if s["bow"] > 0 else 0
        s["learned_spells"] = rng.integers(0, 2, 2)
        s["monsters_killed"] = rng.choice([0, 3, 8, 12], L)
        s["timestep"] = rng.integers(0, 6000)
        s["light_level"] = ref.lib.cfref_light_level(int(s["timestep"]))
        if lvl == L - 1:
            s["boss_progress"] = rng.integers(0, 8)
            s["boss_timesteps_to_spawn_this_round"] = rng.integers(0, 12)
        # every other env of the two dungeons that have an enchantment table stands in front of
        # it (facing right) with the mana and the gems an enchantment costs
        tables = np.argwhere((s["map"][lvl] == 30) | (s["map"][lvl] == 31))
        if len(tables) and (e // L) % 2 == 0:
            r, c = tables[0]
            if c > 0 and s["map"][lvl, r, c - 1] == 7 and s["item_map"][lvl, r, c - 1] == 0:   # a free path cell
                s["player_position"] = (r, c - 1)
                s["player_direction"] = 2
                s["player_mana"] = 9
                s["ruby"] = max(int(s["ruby"]), 3)
                s["sapphire"] = max(int(s["sapphire"]), 3)
                s["sword"] = max(int(s["sword"]), 1)
                s["bow"] = 1
                s["armour"] = np.maximum(s["armour"], 1)
        # the other half of the envs of seven floors stand in front of what random play does not
        # reach: a ripe plant, a diamond, a sapphire, a ruby, an ice shrub (pickaxe 4), a wounded
        # ice elemental, the necromancer one hit from defeat with no guards and no timer
        # (deep_script forces the DO actions)
        elif (e // L) % 2 == 1 and lvl in DEEP_ENCOUNTERS:
            pr, pc = (int(v) for v in s["player_position"])
            steps_of = {1: (0, -1), 2: (0, 1), 3: (-1, 0), 4: (1, 0)}

            def free(r, c):
                return (0 <= r < M and 0 <= c < M and s["map"][lvl, r, c] in (2, 7, 25, 26)
                        and s["item_map"][lvl, r, c] == 0 and not (int(s["mob_bits"][lvl, r]) >> c) & 1)
            if lvl == L - 1:
                boss = np.argwhere(s["map"][lvl] == 32)
                for d, (dr, dc) in steps_of.items():
                    if len(boss) and free(int(boss[0][0]) - dr, int(boss[0][1]) - dc):
                        s["player_position"] = (boss[0][0] - dr, boss[0][1] - dc)
                        s["player_direction"] = d
                        s["boss_progress"] = 7
                        s["boss_timesteps_to_spawn_this_round"] = 0
                        s["mob_mask"][:3, lvl] = 0
                        s["mob_bits"][lvl] = 0
                        break
            else:
                for d, (dr, dc) in steps_of.items():
                    r, c = pr + dr, pc + dc
                    if not free(r, c):
                        continue
                    s["player_direction"] = d
                    if lvl == 0:
                        s["map"][lvl, r, c] = 16
                        s["growing_plants_positions"][0] = (r, c)
                        s["growing_plants_age"][0] = 700
                        s["growing_plants_mask"][0] = 1
                    elif lvl != 7:      # a diamond, a sapphire, a ruby, an ice shrub to be mined
                        s["map"][lvl, r, c] = DEEP_ENCOUNTERS[lvl]
                        s["pickaxe"] = 4
                    else:
                        s["mob_position"][2, lvl, 0] = (r, c)
                        s["mob_health"][2, lvl, 0] = 0.5
                        s["mob_mask"][2, lvl, 0] = 1
                        s["mob_type_id"][2, lvl, 0] = 7
                        s["mob_attack_cooldown"][2, lvl, 0] = 3
                        s["mob_bits"][lvl, r] |= np.uint64(1) << np.uint64(c)
                    break
        ref.import_(e, s)
        st[e] = ref.export([e])[0]      # the spawn bit planes follow the edited map
    return st


def deep_script(n):
    """Actions forced on the first two steps of deep_states' envs (-1: none): DO for the envs
    that were put in front of a plant, an ice elemental or the necromancer."""
    e = np.arange(n)
    special = ((e // L) % 2 == 1) & np.isin(e % L, list(DEEP_ENCOUNTERS))
    return np.where(special, 5, -1).astype(np.float32)


class Ref:
    """oracle/_ref/libcfref.so: the reference's own env, one global vector of envs."""

    def __init__(self, strict=False):
        """strict: the same source built with strict per-operation fp32 (oracle/Makefile)."""
        path = os.path.join(ROOT, "oracle", "_ref", "libcfref_strict.so" if strict else "libcfref.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.lib = lib = C.CDLL(path)
        lib.cfref_init.argtypes = [C.c_int, C.c_uint64]
        lib.cfref_exchange_bytes.restype = C.c_size_t
        lib.cfref_export_state.argtypes = [C.c_int, C.c_void_p]
        lib.cfref_import_state.argtypes = [C.c_int, C.c_void_p]
        lib.cfref_next_action.argtypes = [C.c_int]
        lib.cfref_next_action.restype = C.c_float
        lib.cfref_step_env.argtypes = [C.c_int, C.c_float, C.c_void_p, C.POINTER(C.c_float), C.c_void_p]
        lib.cfref_step_env.restype = C.c_int
        lib.cfref_light_level.argtypes = [C.c_int]
        lib.cfref_light_level.restype = C.c_float
        lib.cfref_fuzz_state.argtypes = [C.c_int, C.c_uint64]
        assert lib.cfref_exchange_bytes() == STATE_DTYPE.itemsize

    def init(self, n, seed):
        self.n = n
        self.lib.cfref_init(n, seed)

    def export(self, envs=None):
        envs = range(self.n) if envs is None else envs
        out = np.zeros(len(envs), STATE_DTYPE)
        for k, e in enumerate(envs):
            self.lib.cfref_export_state(e, C.c_void_p(out[k:k + 1].ctypes.data))
        return out

    def import_(self, env, state):
        s = np.ascontiguousarray(state.reshape(1))
        self.lib.cfref_import_state(env, ptr(s))

    def next_actions(self):
        return np.array([self.lib.cfref_next_action(e) for e in range(self.n)], np.float32)

    def step(self, actions):
        """Steps every env; returns (final states before any reset, rewards, terminals,
        reset keys).  Afterwards the reference holds the post-reset states."""
        final = np.zeros(self.n, STATE_DTYPE)
        rew = np.zeros(self.n, np.float32)
        term = np.zeros(self.n, np.float32)
        keys = np.zeros((self.n, 2), np.uint32)
        r = C.c_float()
        for e in range(self.n):
            d = self.lib.cfref_step_env(e, float(actions[e]), C.c_void_p(final[e:e + 1].ctypes.data),
                                        C.byref(r), C.c_void_p(keys[e:e + 1].ctypes.data))
            rew[e] = r.value
            term[e] = d
        return final, rew, term, keys


class HostStep:
    """oracle/libcfenvhost.so: env_logic.h compiled for the host."""

    def __init__(self):
        path = os.path.join(ROOT, "oracle", "libcfenvhost.so")
        self.lib = lib = C.CDLL(path)
        lib.cfhost_state_bytes.restype = C.c_size_t
        assert lib.cfhost_state_bytes() == STATE_DTYPE.itemsize
        lib.cfhost_light_table.argtypes = [C.c_void_p, C.c_int]
        lib.cfhost_step.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 5
        lib.cfhost_derive_spawn_planes.argtypes = [C.c_void_p, C.c_int]
        lib.cfhost_generate.argtypes = [C.c_uint32, C.c_int, C.c_void_p]
        lib.cfhost_reset.argtypes = [C.c_void_p, C.c_void_p]
        self.light = np.zeros(100001, np.float32)
        lib.cfhost_light_table(ptr(self.light), len(self.light))

    def generate(self, seed, n):
        out = np.zeros(n, STATE_DTYPE)
        self.lib.cfhost_generate(seed, n, ptr(out))
        return out

    def step(self, states, actions):
        n = len(states)
        rew = np.zeros(n, np.float32)
        term = np.zeros(n, np.float32)
        keys = np.zeros((n, 2), np.uint32)
        a = np.ascontiguousarray(actions, np.float32)
        self.lib.cfhost_step(ptr(states), n, ptr(a), ptr(self.light), ptr(rew), ptr(term), ptr(keys))
        return rew, term, keys
