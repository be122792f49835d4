// The env step on gfx950: device layout, step kernel, reset-from-pool kernel and the host
// side of cfp_env.h.
//
// Layout.  Every scalar member of an env's state is one array [sub_index][env] (stride = env
// count), the layout the reference's GPU port uses for its hot fields
// (CF_SOA_FIELDS, craftax_full.cu:613-723) and the one cfp_record_obs_soa reads; a
// wavefront of 64 consecutive envs loads a field as one 256-byte row.  The three byte maps
// stay per env (map | item_map | light_map, 9 levels x 48 x 48 each = 62 208 bytes): they are
// touched a cell at a time at env-dependent places.  Achievements, plant masks and chest
// flags are bit sets.
//
// Kernel.  One lane per env, one wavefront per workgroup.  The ~75 hot scalars of an env
// are registers for the whole step (env_logic.h, Hot).  The 14 mob slots of the level the
// player is on are the part of the state that is indexed with runtime indices (first free
// slot, the mob standing on a cell, ...); they are staged in LDS as [word][lane] -- 24 KB
// per wavefront, conflict-free for any per-lane word index -- and written back slot by
// slot if touched.  The spawn scan (27 rows of 48-bit bitmaps around the player, asked for
// by 5-15 % of the envs per step) runs after every lane is through its step, with the
// wavefront converged: the asking lanes scan together, their 54 row loads in flight at once.
//
// Arithmetic that the hot path is bound by: each env step moves ~0.3 KB of scalars in and
// out as whole rows plus ~0.8 KB of mob slots plus a few dozen single-byte map cells (one
// 64-byte sector each); it is latency- and divergence-bound, not HBM-bound.
#include "cfp_common.h"
#include "env_host.h"
#include "env_internal.h"
#include "cfp_internal.h"

#include <mutex>
#include <vector>

namespace cfp {
namespace {

using namespace cfenv;

constexpr int kWave = 64;
constexpr size_t kPlaneBytes = (size_t)kMap * kMap;                 // 2304
constexpr size_t kEnvPlaneBytes = 3 * (size_t)kLevels * kPlaneBytes;  // 62 208
constexpr int kMobSlots = CFP_ENV_MOB_CLASSES * kLevels * 3;         // 135

// ---- field registry ------------------------------------------------------------------------
// X(name, device type, entries per env, value of entry k read from an exchange struct `st`,
//   statement that writes value `v` of entry k into `st`)
#define CFE_FIELDS(X)                                                                                   \
    X(player_position, int32_t, 2, st.player_position[k], st.player_position[k] = v)                    \
    X(player_level, int32_t, 1, st.player_level, st.player_level = v)                                   \
    X(player_direction, int32_t, 1, st.player_direction, st.player_direction = v)                       \
    X(player_health, float, 1, st.player_health, st.player_health = v)                                  \
    X(player_food, int32_t, 1, st.player_food, st.player_food = v)                                      \
    X(player_drink, int32_t, 1, st.player_drink, st.player_drink = v)                                   \
    X(player_energy, int32_t, 1, st.player_energy, st.player_energy = v)                                \
    X(player_mana, int32_t, 1, st.player_mana, st.player_mana = v)                                      \
    X(is_sleeping, uint8_t, 1, (uint8_t)(st.is_sleeping != 0), st.is_sleeping = v)                      \
    X(is_resting, uint8_t, 1, (uint8_t)(st.is_resting != 0), st.is_resting = v)                         \
    X(player_recover, float, 1, st.player_recover, st.player_recover = v)                               \
    X(player_hunger, float, 1, st.player_hunger, st.player_hunger = v)                                  \
    X(player_thirst, float, 1, st.player_thirst, st.player_thirst = v)                                  \
    X(player_fatigue, float, 1, st.player_fatigue, st.player_fatigue = v)                               \
    X(player_recover_mana, float, 1, st.player_recover_mana, st.player_recover_mana = v)                \
    X(player_xp, int32_t, 1, st.player_xp, st.player_xp = v)                                            \
    X(player_dexterity, int32_t, 1, st.player_dexterity, st.player_dexterity = v)                       \
    X(player_strength, int32_t, 1, st.player_strength, st.player_strength = v)                          \
    X(player_intelligence, int32_t, 1, st.player_intelligence, st.player_intelligence = v)              \
    X(inv_wood, int32_t, 1, st.wood, st.wood = v)                                                       \
    X(inv_stone, int32_t, 1, st.stone, st.stone = v)                                                    \
    X(inv_coal, int32_t, 1, st.coal, st.coal = v)                                                       \
    X(inv_iron, int32_t, 1, st.iron, st.iron = v)                                                       \
    X(inv_diamond, int32_t, 1, st.diamond, st.diamond = v)                                              \
    X(inv_sapling, int32_t, 1, st.sapling, st.sapling = v)                                              \
    X(inv_pickaxe, int32_t, 1, st.pickaxe, st.pickaxe = v)                                              \
    X(inv_sword, int32_t, 1, st.sword, st.sword = v)                                                    \
    X(inv_bow, int32_t, 1, st.bow, st.bow = v)                                                          \
    X(inv_arrows, int32_t, 1, st.arrows, st.arrows = v)                                                 \
    X(inv_armour, int32_t, 4, st.armour[k], st.armour[k] = v)                                           \
    X(inv_torches, int32_t, 1, st.torches, st.torches = v)                                              \
    X(inv_ruby, int32_t, 1, st.ruby, st.ruby = v)                                                       \
    X(inv_sapphire, int32_t, 1, st.sapphire, st.sapphire = v)                                           \
    X(inv_potions, int32_t, 6, st.potions[k], st.potions[k] = v)                                        \
    X(inv_books, int32_t, 1, st.books, st.books = v)                                                    \
    X(learned_spells, uint8_t, 2, (uint8_t)(st.learned_spells[k] != 0), st.learned_spells[k] = v)       \
    X(sword_enchantment, int32_t, 1, st.sword_enchantment, st.sword_enchantment = v)                    \
    X(bow_enchantment, int32_t, 1, st.bow_enchantment, st.bow_enchantment = v)                          \
    X(armour_enchantments, int32_t, 4, st.armour_enchantments[k], st.armour_enchantments[k] = v)        \
    X(boss_progress, int32_t, 1, st.boss_progress, st.boss_progress = v)                                \
    X(boss_timesteps_to_spawn_this_round, int32_t, 1, st.boss_timesteps_to_spawn_this_round,            \
      st.boss_timesteps_to_spawn_this_round = v)                                                        \
    X(light_level, float, 1, st.light_level, st.light_level = v)                                        \
    X(timestep, int32_t, 1, st.timestep, st.timestep = v)                                               \
    X(state_rng, uint32_t, 2, st.state_rng[k], st.state_rng[k] = v)                                     \
    X(rng_key, uint32_t, 2, st.rng_key[k], st.rng_key[k] = v)                                           \
    X(ach_bits, uint32_t, 3, ach_word(st, k), set_ach_word(st, k, v))                                   \
    X(plant_mask, uint32_t, 1, plant_bits(st), set_plant_bits(st, v))                                   \
    X(plant_pos, int32_t, 20, (&st.growing_plants_positions[0][0])[k],                                  \
      (&st.growing_plants_positions[0][0])[k] = v)                                                      \
    X(plant_age, int32_t, 10, st.growing_plants_age[k], st.growing_plants_age[k] = v)                   \
    X(chest_bits, uint32_t, 1, chest_word(st), set_chest_word(st, v))                                   \
    X(potion_mapping, int32_t, 6, st.potion_mapping[k], st.potion_mapping[k] = v)                       \
    X(down_ladders, int32_t, 18, (&st.down_ladders[0][0])[k], (&st.down_ladders[0][0])[k] = v)          \
    X(up_ladders, int32_t, 18, (&st.up_ladders[0][0])[k], (&st.up_ladders[0][0])[k] = v)                \
    X(monsters_killed, int32_t, 9, st.monsters_killed[k], st.monsters_killed[k] = v)                    \
    X(mob_position, int32_t, 270, (&st.mob_position[0][0][0][0])[k], (&st.mob_position[0][0][0][0])[k] = v) \
    X(mob_health, float, 135, (&st.mob_health[0][0][0])[k], (&st.mob_health[0][0][0])[k] = v)           \
    X(mob_mask, uint8_t, 135, (uint8_t)((&st.mob_mask[0][0][0])[k] != 0), (&st.mob_mask[0][0][0])[k] = v) \
    X(mob_attack_cooldown, int32_t, 135, (&st.mob_attack_cooldown[0][0][0])[k],                         \
      (&st.mob_attack_cooldown[0][0][0])[k] = v)                                                        \
    X(mob_type_id, int32_t, 135, (&st.mob_type_id[0][0][0])[k], (&st.mob_type_id[0][0][0])[k] = v)      \
    X(mob_projectile_directions, int32_t, 54, (&st.mob_projectile_directions[0][0][0])[k],              \
      (&st.mob_projectile_directions[0][0][0])[k] = v)                                                  \
    X(player_projectile_directions, int32_t, 54, (&st.player_projectile_directions[0][0][0])[k],        \
      (&st.player_projectile_directions[0][0][0])[k] = v)                                               \
    X(mob_bits, uint64_t, 432, (&st.mob_bits[0][0])[k], (&st.mob_bits[0][0])[k] = v)                    \
    X(spawn_all_bits, uint64_t, 432, (&st.spawn_all_bits[0][0])[k], (&st.spawn_all_bits[0][0])[k] = v)  \
    X(spawn_grave_bits, uint64_t, 432, (&st.spawn_grave_bits[0][0])[k], (&st.spawn_grave_bits[0][0])[k] = v) \
    X(spawn_water_bits, uint64_t, 432, (&st.spawn_water_bits[0][0])[k], (&st.spawn_water_bits[0][0])[k] = v)

inline uint32_t ach_word(const cfp_env_state& st, int w) {
    uint32_t m = 0;
    for (int a = 32 * w; a < 32 * w + 32 && a < CFP_ENV_ACHIEVEMENTS; a++) m |= (uint32_t)(st.achievements[a] != 0) << (a & 31);
    return m;
}
inline void set_ach_word(cfp_env_state& st, int w, uint32_t m) {
    for (int a = 32 * w; a < 32 * w + 32 && a < CFP_ENV_ACHIEVEMENTS; a++) st.achievements[a] = (m >> (a & 31)) & 1u;
}
inline uint32_t plant_bits(const cfp_env_state& st) {
    uint32_t m = 0;
    for (int i = 0; i < kPlants; i++) m |= (uint32_t)(st.growing_plants_mask[i] != 0) << i;
    return m;
}
inline void set_plant_bits(cfp_env_state& st, uint32_t m) {
    for (int i = 0; i < kPlants; i++) st.growing_plants_mask[i] = (m >> i) & 1u;
}
inline uint32_t chest_word(const cfp_env_state& st) {
    uint32_t m = 0;
    for (int l = 0; l < kLevels; l++) m |= (uint32_t)(st.chests_opened[l] != 0) << l;
    return m;
}
inline void set_chest_word(cfp_env_state& st, uint32_t m) {
    for (int l = 0; l < kLevels; l++) st.chests_opened[l] = (m >> l) & 1u;
}

// The device arrays of one set of envs (the live envs, or the reset pool).
struct EnvArrays {
#define CFE_DECL(name, type, count, get, set) type* name;
    CFE_FIELDS(CFE_DECL)
#undef CFE_DECL
    uint8_t* planes;    // [n][map | item_map | light_map][9][48][48]
    uint32_t* action_rng;
    int n;              // env count = stride of every array
};

struct FieldDesc {
    size_t elem;
    int count;
    size_t offset;      // of the pointer inside EnvArrays
};
const FieldDesc kFieldTable[] = {
#define CFE_DESC(name, type, count, get, set) {sizeof(type), count, offsetof(EnvArrays, name)},
    CFE_FIELDS(CFE_DESC)
#undef CFE_DESC
};
constexpr int kNumFields = (int)(sizeof(kFieldTable) / sizeof(kFieldTable[0]));

// ---- storage object of the kernel -----------------------------------------------------------
constexpr int kSlotWords = 4;                     // (row, col), health, cooldown, (type, mask): 17 KiB a wavefront,
                                                  // so that registers, not LDS, set the eight wavefronts of a CU
constexpr int kLevelSlots = 14;                   // 3 + 3 + 2 + 3 + 3
constexpr int kLdsWords = kSlotWords * kLevelSlots + 12;  // + 6 projectile directions x 2
__device__ __forceinline__ int slot_of(int pool, int i) { return pool < 2 ? pool * 3 + i : (pool == 2 ? 6 + i : 8 + (pool - 3) * 3 + i); }

struct DevStore {
    const EnvArrays& A;
    uint32_t* lds;      // this lane's column: word w at lds[w * 64]
    uint8_t* planes;    // this env's maps
    const float* light;
    int e;
    int lvl;
    uint32_t dirty;     // bit g: slot g was written; bit 14 + j: direction pair j

    __device__ __forceinline__ size_t at(int sub) const { return (size_t)sub * (size_t)A.n + (size_t)e; }
    __device__ __forceinline__ int blk(int l, int r, int c) const { return planes[(size_t)l * kPlaneBytes + r * kMap + c]; }
    __device__ __forceinline__ void put_blk_raw(int l, int r, int c, int b) { planes[(size_t)l * kPlaneBytes + r * kMap + c] = (uint8_t)b; }
    __device__ __forceinline__ int item(int l, int r, int c) const { return planes[(size_t)(kLevels + l) * kPlaneBytes + r * kMap + c]; }
    __device__ __forceinline__ void put_item(int l, int r, int c, int v) { planes[(size_t)(kLevels + l) * kPlaneBytes + r * kMap + c] = (uint8_t)v; }
    __device__ __forceinline__ int lum(int l, int r, int c) const { return planes[(size_t)(2 * kLevels + l) * kPlaneBytes + r * kMap + c]; }
    __device__ __forceinline__ void put_lum(int l, int r, int c, int v) { planes[(size_t)(2 * kLevels + l) * kPlaneBytes + r * kMap + c] = (uint8_t)v; }
    __device__ __forceinline__ uint64_t mobrow(int l, int r) const { return A.mob_bits[at(l * kMap + r)]; }
    __device__ __forceinline__ void put_mobrow(int l, int r, uint64_t v) { A.mob_bits[at(l * kMap + r)] = v; }
    __device__ __forceinline__ uint64_t* plane_of(int kind) const {
        return kind == SK_ALL ? A.spawn_all_bits : (kind == SK_GRAVE ? A.spawn_grave_bits : A.spawn_water_bits);
    }
    __device__ __forceinline__ uint64_t spawnrow(int kind, int l, int r) const { return plane_of(kind)[at(l * kMap + r)]; }
    __device__ __forceinline__ void put_spawnrow(int kind, int l, int r, uint64_t v) { plane_of(kind)[at(l * kMap + r)] = v; }

    __device__ __forceinline__ uint32_t& word(int f, int g) const { return lds[(f * kLevelSlots + g) * kWave]; }
    // word 0: row and column as two int16 (positions stay within a step of the 48 x 48 map),
    // word 1: health, word 2: attack cooldown (counts down without bound), word 3: type id in
    // the low half, mask in bit 16
    static __device__ __forceinline__ int lo16(uint32_t w) { return (int)((int32_t)(w << 16) >> 16); }
    static __device__ __forceinline__ int hi16(uint32_t w) { return (int)((int32_t)w >> 16); }
    __device__ __forceinline__ int m_row(int p, int i) const { return lo16(word(0, slot_of(p, i))); }
    __device__ __forceinline__ int m_col(int p, int i) const { return hi16(word(0, slot_of(p, i))); }
    __device__ __forceinline__ float m_hp(int p, int i) const { return __uint_as_float(word(1, slot_of(p, i))); }
    __device__ __forceinline__ bool m_mask(int p, int i) const { return (word(3, slot_of(p, i)) >> 16) != 0; }
    __device__ __forceinline__ int m_cd(int p, int i) const { return (int)word(2, slot_of(p, i)); }
    __device__ __forceinline__ int m_type(int p, int i) const { return lo16(word(3, slot_of(p, i))); }
    __device__ __forceinline__ void touch(int g) { dirty |= 1u << g; }
    __device__ __forceinline__ void set_m_pos(int p, int i, int r, int c) {
        const int g = slot_of(p, i);
        word(0, g) = ((uint32_t)r & 0xffffu) | ((uint32_t)c << 16);
        touch(g);
    }
    __device__ __forceinline__ void set_m_hp(int p, int i, float v) {
        const int g = slot_of(p, i);
        word(1, g) = __float_as_uint(v);
        touch(g);
    }
    __device__ __forceinline__ void set_m_mask(int p, int i, bool v) {
        const int g = slot_of(p, i);
        word(3, g) = (word(3, g) & 0xffffu) | ((uint32_t)v << 16);
        touch(g);
    }
    __device__ __forceinline__ void set_m_cd(int p, int i, int v) {
        const int g = slot_of(p, i);
        word(2, g) = (uint32_t)v;
        touch(g);
    }
    __device__ __forceinline__ void set_m_type(int p, int i, int v) {
        const int g = slot_of(p, i);
        word(3, g) = (word(3, g) & ~0xffffu) | ((uint32_t)v & 0xffffu);
        touch(g);
    }
    __device__ __forceinline__ uint32_t& dword(int p, int i, int axis) const {
        return lds[(kSlotWords * kLevelSlots + ((p - P_MOB_PROJ) * 3 + i) * 2 + axis) * kWave];
    }
    __device__ __forceinline__ int pd_r(int p, int i) const { return (int)dword(p, i, 0); }
    __device__ __forceinline__ int pd_c(int p, int i) const { return (int)dword(p, i, 1); }
    __device__ __forceinline__ void set_pd(int p, int i, int r, int c) {
        dword(p, i, 0) = (uint32_t)r;
        dword(p, i, 1) = (uint32_t)c;
        dirty |= 1u << (kLevelSlots + (p - P_MOB_PROJ) * 3 + i);
    }

    __device__ __forceinline__ int kills(int l) const { return A.monsters_killed[at(l)]; }
    __device__ __forceinline__ void set_kills(int l, int v) { A.monsters_killed[at(l)] = v; }
    __device__ __forceinline__ bool chest(int l) const { return (A.chest_bits[at(0)] >> l) & 1u; }
    __device__ __forceinline__ void set_chest(int l) { A.chest_bits[at(0)] |= 1u << l; }
    __device__ __forceinline__ int ladder_down(int l, int a) const { return A.down_ladders[at(l * 2 + a)]; }
    __device__ __forceinline__ int ladder_up(int l, int a) const { return A.up_ladders[at(l * 2 + a)]; }
    __device__ __forceinline__ int potion_effect(int i) const { return A.potion_mapping[at(i)]; }
    __device__ __forceinline__ int plant_r(int i) const { return A.plant_pos[at(2 * i)]; }
    __device__ __forceinline__ int plant_c(int i) const { return A.plant_pos[at(2 * i + 1)]; }
    __device__ __forceinline__ int plant_age(int i) const { return A.plant_age[at(i)]; }
    __device__ __forceinline__ void set_plant(int i, int r, int c) {
        A.plant_pos[at(2 * i)] = r;
        A.plant_pos[at(2 * i + 1)] = c;
    }
    __device__ __forceinline__ void set_plant_age(int i, int a) { A.plant_age[at(i)] = a; }
    __device__ __forceinline__ void stamp(int) {}
    __device__ __forceinline__ float light_at(int t) const { return light[t < kMaxTimesteps ? t : kMaxTimesteps]; }

    __device__ __forceinline__ int global_slot(int g) const {  // CFM(pool, lvl, i) of slot g
        const int pool = g < 6 ? g / 3 : (g < 8 ? 2 : 3 + (g - 8) / 3);
        const int i = g < 6 ? g % 3 : (g < 8 ? g - 6 : (g - 8) % 3);
        return (pool * kLevels + lvl) * 3 + i;
    }
    // stage the 14 slots of level l
    __device__ __forceinline__ void open_level(int l) {
        lvl = l;
        dirty = 0;
#pragma unroll
        for (int g = 0; g < kLevelSlots; g++) {
            const int m = global_slot(g);
            word(0, g) = ((uint32_t)A.mob_position[at(2 * m)] & 0xffffu) | ((uint32_t)A.mob_position[at(2 * m + 1)] << 16);
            word(1, g) = __float_as_uint(A.mob_health[at(m)]);
            word(2, g) = (uint32_t)A.mob_attack_cooldown[at(m)];
            word(3, g) = ((uint32_t)A.mob_type_id[at(m)] & 0xffffu) | ((uint32_t)(A.mob_mask[at(m)] != 0) << 16);
        }
#pragma unroll
        for (int j = 0; j < 6; j++) {
            const int32_t* src = j < 3 ? A.mob_projectile_directions : A.player_projectile_directions;
            const int idx = (lvl * 3 + j % 3) * 2;
            lds[(kSlotWords * kLevelSlots + 2 * j) * kWave] = (uint32_t)src[at(idx)];
            lds[(kSlotWords * kLevelSlots + 2 * j + 1) * kWave] = (uint32_t)src[at(idx + 1)];
        }
    }
    // write the touched slots back
    __device__ __forceinline__ void close_level() {
#pragma unroll
        for (int g = 0; g < kLevelSlots; g++) {
            if (!((dirty >> g) & 1u)) continue;
            const int m = global_slot(g);
            A.mob_position[at(2 * m)] = lo16(word(0, g));
            A.mob_position[at(2 * m + 1)] = hi16(word(0, g));
            A.mob_health[at(m)] = __uint_as_float(word(1, g));
            A.mob_mask[at(m)] = (uint8_t)(word(3, g) >> 16);
            A.mob_attack_cooldown[at(m)] = (int32_t)word(2, g);
            A.mob_type_id[at(m)] = lo16(word(3, g));
        }
#pragma unroll
        for (int j = 0; j < 6; j++) {
            if (!((dirty >> (kLevelSlots + j)) & 1u)) continue;
            int32_t* dst = j < 3 ? A.mob_projectile_directions : A.player_projectile_directions;
            const int idx = (lvl * 3 + j % 3) * 2;
            dst[at(idx)] = (int32_t)lds[(kSlotWords * kLevelSlots + 2 * j) * kWave];
            dst[at(idx + 1)] = (int32_t)lds[(kSlotWords * kLevelSlots + 2 * j + 1) * kWave];
        }
    }
};

__device__ __forceinline__ void load_hot_dev(const EnvArrays& A, size_t e, Hot& h) {
    const size_t n = (size_t)A.n;
    h.pr = A.player_position[e];
    h.pc = A.player_position[n + e];
    h.level = A.player_level[e];
    h.dir = A.player_direction[e];
    h.health = A.player_health[e];
    h.food = A.player_food[e];
    h.drink = A.player_drink[e];
    h.energy = A.player_energy[e];
    h.mana = A.player_mana[e];
    h.sleeping = A.is_sleeping[e];
    h.resting = A.is_resting[e];
    h.recover = A.player_recover[e];
    h.hunger = A.player_hunger[e];
    h.thirst = A.player_thirst[e];
    h.fatigue = A.player_fatigue[e];
    h.recover_mana = A.player_recover_mana[e];
    h.xp = A.player_xp[e];
    h.dex = A.player_dexterity[e];
    h.str = A.player_strength[e];
    h.intel = A.player_intelligence[e];
    h.wood = A.inv_wood[e];
    h.stone = A.inv_stone[e];
    h.coal = A.inv_coal[e];
    h.iron = A.inv_iron[e];
    h.diamond = A.inv_diamond[e];
    h.sapling = A.inv_sapling[e];
    h.pickaxe = A.inv_pickaxe[e];
    h.sword = A.inv_sword[e];
    h.bow = A.inv_bow[e];
    h.arrows = A.inv_arrows[e];
#pragma unroll
    for (int i = 0; i < 4; i++) h.armour[i] = A.inv_armour[i * n + e];
    h.torches = A.inv_torches[e];
    h.ruby = A.inv_ruby[e];
    h.sapphire = A.inv_sapphire[e];
#pragma unroll
    for (int i = 0; i < 6; i++) h.potions[i] = A.inv_potions[i * n + e];
    h.books = A.inv_books[e];
    h.spell[0] = A.learned_spells[e];
    h.spell[1] = A.learned_spells[n + e];
    h.sword_ench = A.sword_enchantment[e];
    h.bow_ench = A.bow_enchantment[e];
#pragma unroll
    for (int i = 0; i < 4; i++) h.armour_ench[i] = A.armour_enchantments[i * n + e];
    h.boss_progress = A.boss_progress[e];
    h.boss_timer = A.boss_timesteps_to_spawn_this_round[e];
    h.light_level = A.light_level[e];
    h.timestep = A.timestep[e];
#pragma unroll
    for (int w = 0; w < 3; w++) h.ach[w] = A.ach_bits[w * n + e];
    h.plant_mask = A.plant_mask[e];
}

// Every scalar is written back: a field is one 256-byte row per wavefront, and keeping the
// step's input around to compare against would double the registers an env holds.
__device__ __forceinline__ void store_hot_dev(const EnvArrays& A, size_t e, const Hot& h) {
    const size_t n = (size_t)A.n;
    A.player_position[e] = h.pr;
    A.player_position[n + e] = h.pc;
    A.player_level[e] = h.level;
    A.player_direction[e] = h.dir;
    A.player_health[e] = h.health;
    A.player_food[e] = h.food;
    A.player_drink[e] = h.drink;
    A.player_energy[e] = h.energy;
    A.player_mana[e] = h.mana;
    A.is_sleeping[e] = (uint8_t)h.sleeping;
    A.is_resting[e] = (uint8_t)h.resting;
    A.player_recover[e] = h.recover;
    A.player_hunger[e] = h.hunger;
    A.player_thirst[e] = h.thirst;
    A.player_fatigue[e] = h.fatigue;
    A.player_recover_mana[e] = h.recover_mana;
    A.player_xp[e] = h.xp;
    A.player_dexterity[e] = h.dex;
    A.player_strength[e] = h.str;
    A.player_intelligence[e] = h.intel;
    A.inv_wood[e] = h.wood;
    A.inv_stone[e] = h.stone;
    A.inv_coal[e] = h.coal;
    A.inv_iron[e] = h.iron;
    A.inv_diamond[e] = h.diamond;
    A.inv_sapling[e] = h.sapling;
    A.inv_pickaxe[e] = h.pickaxe;
    A.inv_sword[e] = h.sword;
    A.inv_bow[e] = h.bow;
    A.inv_arrows[e] = h.arrows;
#pragma unroll
    for (int i = 0; i < 4; i++) A.inv_armour[i * n + e] = h.armour[i];
    A.inv_torches[e] = h.torches;
    A.inv_ruby[e] = h.ruby;
    A.inv_sapphire[e] = h.sapphire;
#pragma unroll
    for (int i = 0; i < 6; i++) A.inv_potions[i * n + e] = h.potions[i];
    A.inv_books[e] = h.books;
    A.learned_spells[e] = (uint8_t)h.spell[0];
    A.learned_spells[n + e] = (uint8_t)h.spell[1];
    A.sword_enchantment[e] = h.sword_ench;
    A.bow_enchantment[e] = h.bow_ench;
#pragma unroll
    for (int i = 0; i < 4; i++) A.armour_enchantments[i * n + e] = h.armour_ench[i];
    A.boss_progress[e] = h.boss_progress;
    A.boss_timesteps_to_spawn_this_round[e] = h.boss_timer;
    A.light_level[e] = h.light_level;
    A.timestep[e] = h.timestep;
#pragma unroll
    for (int w = 0; w < 3; w++) A.ach_bits[w * n + e] = h.ach[w];
    A.plant_mask[e] = h.plant_mask;
}

// run_spawns of env_logic.h with the wavefront kept together.  Some 5-15 % of the lanes roll
// a spawn in a step, nearly all of them for one kind of mob.  Each such lane scans its own 27
// bitmap rows (54 independent 8-byte loads in flight at once, then popcounts); lanes asking for
// different kinds run the same pass, since ring and terrain are per-lane values.  The wavefront
// repeats the pass only while some lane has a second or third kind pending.
__device__ __forceinline__ void run_spawns_lanes(DevStore& s, const Hot& h, const SpawnPlan& plan) {
    const int l = wrap_clamp(h.level, kLevels);
    uint32_t pending = plan.tries;
    while (__any(pending != 0)) {
        if (pending != 0) {
            const int w = __builtin_ctz(pending);
            pending &= pending - 1;
            int ring = 0, kind = 0, slot = 0, type = 0, key_lo = 0, key_hi = 0;
#pragma unroll
            for (int v = 0; v < 3; v++) {   // values, not addresses, are selected (see opaque)
                ring = w == v ? opaque(plan.ring[v]) : ring;
                kind = w == v ? opaque(plan.kind[v]) : kind;
                slot = w == v ? opaque(plan.slot[v]) : slot;
                type = w == v ? opaque(plan.type[v]) : type;
                key_lo = w == v ? opaque((int)(uint32_t)plan.key[v]) : key_lo;
                key_hi = w == v ? opaque((int)(uint32_t)(plan.key[v] >> 32)) : key_hi;
            }
            const uint64_t key = (uint64_t)(uint32_t)key_hi << 32 | (uint32_t)key_lo;
            // pass 1: candidates per row, one byte each (a row has at most 27)
            uint64_t counts[4] = {0, 0, 0, 0};
            int n = 0;
#pragma unroll 9
            for (int j = 0; j < 2 * kDespawn - 1; j++) {   // nine rows' loads in flight at a time
                const int cnt = __popcll(spawn_candidates(s, h, l, ring, kind, j - (kDespawn - 1)));
                counts[j >> 3] |= (uint64_t)cnt << (8 * (j & 7));
                n += cnt;
            }
            if (n != 0) {
                // pass 2: the row holding the drawn candidate, then that row once more
                int k = pick_index(n, key);
                int jrow = 0;
                bool found = false;
#pragma unroll
                for (int j = 0; j < 2 * kDespawn - 1; j++) {
                    const int cnt = (int)((counts[j >> 3] >> (8 * (j & 7))) & 0xff);
                    if (!found && k < cnt) {
                        jrow = j;
                        found = true;
                    }
                    k -= found ? 0 : cnt;
                }
                uint64_t m = spawn_candidates(s, h, l, ring, kind, jrow - (kDespawn - 1));
                for (; k > 0; k--) m &= m - 1;
                const int row = h.pr + jrow - (kDespawn - 1);
                const int col = __ffsll((long long)m) - 1;
                const int pool = spawn_pool(w);
                s.set_m_pos(pool, slot, row, col);
                s.set_m_hp(pool, slot, mob_health(type, spawn_class(w)));
                s.set_m_mask(pool, slot, true);
                s.put_mobrow(l, row, s.mobrow(l, row) | (1ull << col));
            }
        }
    }
}

// k_step (craftax_full.cu:8760-8779)
__global__ __launch_bounds__(kWave) void k_env_step(EnvArrays A, const float* __restrict__ light,
                                                    const float* __restrict__ actions, float* __restrict__ rewards,
                                                    float* __restrict__ terminals, cfp_env_reset_rec* __restrict__ resets,
                                                    int* __restrict__ reset_count, float* __restrict__ r_reward_row,
                                                    uint8_t* __restrict__ r_done_row) {
    __shared__ uint32_t lds[kLdsWords * kWave];
    const int lane = threadIdx.x;
    const size_t e = (size_t)blockIdx.x * kWave + lane;
    const size_t n = (size_t)A.n;
    // env counts are multiples of 32: the last wavefront may run half empty (the wavefront-wide
    // votes below count the lanes that are there)
    if (e >= n) return;

    Hot h;
    load_hot_dev(A, e, h);
    DevStore s{A, lds + lane, A.planes + e * kEnvPlaneBytes, light, (int)e, 0, 0};

    int action;
    if (actions != nullptr) {
        action = clamp_action(actions[e]);
    } else {
        const uint32_t x = xorshift32(A.action_rng[e]);
        A.action_rng[e] = x;
        action = (int)(x % (uint32_t)kNumActions);
    }
    const StepKeys keys = split_env_key((uint64_t)A.rng_key[n + e] << 32 | A.rng_key[e]);
    SpawnPlan plan;
    const StepOut out = step(s, h, action, keys.step_rng, plan);
    store_hot_dev(A, e, h);    // before the scans: they need the position only
    run_spawns_lanes(s, h, plan);
    s.close_level();
    A.state_rng[e] = (uint32_t)out.state_rng;
    A.state_rng[n + e] = (uint32_t)(out.state_rng >> 32);
    A.rng_key[e] = (uint32_t)keys.env_key;
    A.rng_key[n + e] = (uint32_t)(keys.env_key >> 32);
    rewards[e] = out.reward;
    terminals[e] = out.done ? 1.0f : 0.0f;
    if (r_reward_row != nullptr) {   // a trainer's slab rows (k_record_rd, craftax_full.cu:9758-9767)
        r_reward_row[e] = out.reward;
        r_done_row[e] = out.done ? 1 : 0;
    }

    // done list: one atomic per wavefront
    const unsigned long long done = __ballot(out.done);
    if (done != 0) {
        int base = 0;
        if (lane == 0) base = atomicAdd(reset_count, __popcll(done));
        base = __shfl(base, 0);
        if (out.done) {
            const int rank = __popcll(done & ((1ull << lane) - 1ull));
            cfp_env_reset_rec rec;
            rec.env = (int32_t)e;
            rec.key0 = (uint32_t)keys.reset_key;
            rec.key1 = (uint32_t)(keys.reset_key >> 32);
            resets[base + rank] = rec;
        }
    }
}

__global__ void k_env_zero(int* p) { *p = 0; }

__global__ void k_env_seed_actions(uint32_t* rng, int n, uint64_t seed) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) rng[i] = (uint32_t)(seed ^ ((uint64_t)i * 2654435761ull)) | 1u;
}

// craftax_reset_state_on_done with a static pool (craftax_full.c:3738-3741): one workgroup
// per finished env copies pool entry key0 % pool into it, field by field and the maps as
// 16-byte pieces.  The env's own key and action stream are kept (they are not state).
struct CopyTable {
    const void* src[kNumFields];
    void* dst[kNumFields];
    int elem[kNumFields];
    int count[kNumFields];
};
__global__ __launch_bounds__(256) void k_env_reset_from_pool(CopyTable t, EnvArrays live, EnvArrays pool,
                                                             const cfp_env_reset_rec* __restrict__ resets,
                                                             const int* __restrict__ reset_count, int rng_key_field) {
    const int total = *reset_count;
    for (int idx = blockIdx.x; idx < total; idx += gridDim.x) {
        const size_t e = (size_t)resets[idx].env;
        const size_t p = (size_t)(resets[idx].key0 % (uint32_t)pool.n);
        for (int f = 0; f < kNumFields; f++) {
            if (f == rng_key_field) continue;
            const int cnt = t.count[f], el = t.elem[f];
            for (int k = threadIdx.x; k < cnt; k += blockDim.x) {
                const size_t si = (size_t)k * pool.n + p, di = (size_t)k * live.n + e;
                if (el == 4) ((uint32_t*)t.dst[f])[di] = ((const uint32_t*)t.src[f])[si];
                else if (el == 8) ((uint64_t*)t.dst[f])[di] = ((const uint64_t*)t.src[f])[si];
                else ((uint8_t*)t.dst[f])[di] = ((const uint8_t*)t.src[f])[si];
            }
        }
        const u4* sp = (const u4*)(pool.planes + p * kEnvPlaneBytes);
        u4* dp = (u4*)(live.planes + e * kEnvPlaneBytes);
        for (int k = threadIdx.x; k < (int)(kEnvPlaneBytes / 16); k += blockDim.x) dp[k] = sp[k];
    }
}

// ---- world generation on the device ------------------------------------------------------------
// threads of a generator job: 256 where many worlds are made at once (three jobs share a
// CU), 512 where a step waits for a handful of worlds and a job's latency is what counts
constexpr int kGenThreads = 256, kGenThreadsFew = 512;
// jobs of one world: its nine floors and, as a job of its own, the scalar fields
constexpr int kGenJobs = kLevels + 1;
// the group of env_worldgen.h: one 256-thread workgroup, reductions through wave shuffles
// and four LDS words; cos / sin in double precision, rounded to float
template <int NT>
struct BlockGroup {
    static constexpr int kGenWaves = NT / 64;
    int t;
    float* fred;   // LDS, eight floats a wavefront
    int* ired;     // LDS, one int a wavefront
    __device__ __forceinline__ int tid() const { return t; }
    __device__ __forceinline__ int nt() const { return NT; }
    __device__ __forceinline__ void sync() { __syncthreads(); }
    // minima and maxima of four quantities over the group in one exchange
    __device__ __forceinline__ void gminmax4(float (&mn)[4], float (&mx)[4]) {
#pragma unroll
        for (int f = 0; f < 4; f++) {
#pragma unroll
            for (int d = 32; d > 0; d >>= 1) {
                mn[f] = fminf(mn[f], __shfl_xor(mn[f], d));
                mx[f] = fmaxf(mx[f], __shfl_xor(mx[f], d));
            }
        }
        if ((t & 63) == 0) {
#pragma unroll
            for (int f = 0; f < 4; f++) {
                fred[8 * (t >> 6) + f] = mn[f];
                fred[8 * (t >> 6) + 4 + f] = mx[f];
            }
        }
        __syncthreads();
#pragma unroll
        for (int f = 0; f < 4; f++) {
            mn[f] = fred[f];
            mx[f] = fred[4 + f];
#pragma unroll
            for (int w = 1; w < kGenWaves; w++) {
                mn[f] = fminf(mn[f], fred[8 * w + f]);
                mx[f] = fmaxf(mx[f], fred[8 * w + f + 4]);
            }
        }
        __syncthreads();
    }
    __device__ __forceinline__ int gmaxi(int v) {
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) v = max(v, __shfl_xor(v, d));
        if ((t & 63) == 0) ired[t >> 6] = v;
        __syncthreads();
        v = ired[0];
#pragma unroll
        for (int w = 1; w < kGenWaves; w++) v = max(v, ired[w]);
        __syncthreads();
        return v;
    }
    __device__ __forceinline__ int gscan(int v, int& total) {
        const int lane = t & 63, wave = t >> 6;
        int incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) ired[wave] = incl;
        __syncthreads();
        int before = 0;
        total = 0;
#pragma unroll
        for (int w = 0; w < kGenWaves; w++) {
            before += w < wave ? ired[w] : 0;
            total += ired[w];
        }
        __syncthreads();
        return before + incl - v;
    }
    __device__ __forceinline__ void stamp(int) {}   // phase marker of a profiling build
    __device__ __forceinline__ float cosine(float x) { return (float)cos((double)x); }
    __device__ __forceinline__ float sine(float x) { return (float)sin((double)x); }
};

struct FieldList {          // the per-field arrays of one EnvArrays, for table-driven fills
    void* ptr[kNumFields];
    int elem[kNumFields];
    int count[kNumFields];
};

// k_env_init / k_reset_list_block (craftax_full.cu:8669-8706, 8957-8975): one workgroup per
// floor of an env.  LIST: the envs of the reset list, world key from each record's reset key, the env's
// own key kept.  Otherwise: envs [0, A.n), env i created from seed0 + i as c_init does.
template <bool LIST, int NT>
__global__ __launch_bounds__(NT) void k_env_worldgen(EnvArrays A, FieldList fl, const float* __restrict__ light,
                                                              const cfp_env_reset_rec* __restrict__ resets,
                                                              const int* __restrict__ reset_count, uint64_t seed0,
                                                              int zero_fields) {
    __shared__ FloorScratch sc;
    __shared__ float fred[8 * (NT / 64)];
    __shared__ int ired[NT / 64];
    BlockGroup<NT> g{(int)threadIdx.x, fred, ired};
    const int t = threadIdx.x;
    const size_t n = (size_t)A.n;
    // one workgroup per (env, floor) and one per env for the scalar fields: the ten jobs of a
    // world are independent, and a step waits for its slowest reset
    const int total = (LIST ? *reset_count : A.n) * kGenJobs;
    for (int job = blockIdx.x; job < total; job += gridDim.x) {
        const int idx = job / kGenJobs, level = job - idx * kGenJobs;
        size_t e;
        uint64_t world_key, env_key = 0;
        if (LIST) {
            e = (size_t)resets[idx].env;
            world_key = world_key_of_reset((uint64_t)resets[idx].key1 << 32 | resets[idx].key0);
        } else {
            e = (size_t)idx;
            env_key = lcg(seed_key((uint32_t)(seed0 + (uint64_t)idx)));
            world_key = world_key_of_reset(lcg(env_key));
        }
        if (level == kLevels) {
            // scalars: the fields of `fl` are zero in a fresh state; the others are written below
            for (int f = 0; f < zero_fields; f++) {
                const int el = fl.elem[f];
                for (int k = t; k < fl.count[f]; k += NT) {
                    const size_t at = (size_t)k * n + e;
                    if (el == 4) ((uint32_t*)fl.ptr[f])[at] = 0u;
                    else if (el == 8) ((uint64_t*)fl.ptr[f])[at] = 0ull;
                    else ((uint8_t*)fl.ptr[f])[at] = 0;
                }
            }
            for (int k = t; k < kMobSlots; k += NT)
                A.mob_health[(size_t)k * n + e] = (k / 27 == P_RANGED && k % 3 == 2) ? 0.0f : 1.0f;
            for (int k = t; k < 54; k += NT) {
                A.mob_projectile_directions[(size_t)k * n + e] = 1;
                A.player_projectile_directions[(size_t)k * n + e] = 1;
            }
            if (t < kLevels) A.monsters_killed[(size_t)t * n + e] = t == 0 ? 10 : 0;
            if (t == 0) {
                int32_t perm[6];
                potion_permutation(world_key, perm);
                for (int i = 0; i < 6; i++) A.potion_mapping[(size_t)i * n + e] = perm[i];
                const uint64_t sk = world_state_key(world_key);
                A.state_rng[e] = (uint32_t)sk;
                A.state_rng[n + e] = (uint32_t)(sk >> 32);
                A.player_position[e] = kMap / 2;
                A.player_position[n + e] = kMap / 2;
                A.player_direction[e] = A_UP;
                A.player_health[e] = 9.0f;
                A.player_food[e] = 9;
                A.player_drink[e] = 9;
                A.player_energy[e] = 9;
                A.player_mana[e] = 9;
                A.player_dexterity[e] = 1;
                A.player_strength[e] = 1;
                A.player_intelligence[e] = 1;
                A.boss_timesteps_to_spawn_this_round[e] = 7;
                A.light_level[e] = light[0];
                if (!LIST) {
                    A.rng_key[e] = (uint32_t)env_key;
                    A.rng_key[n + e] = (uint32_t)(env_key >> 32);
                }
            }
            continue;   // (uniform over the workgroup)
        }
        uint8_t* planes = A.planes + e * kEnvPlaneBytes;
        generate_floor(g, sc, world_key, level);
        // the three byte planes, 16 bytes a thread
        for (int k = t; k < 3 * (int)(kPlaneBytes / 16); k += NT) {
            const int plane = k / (int)(kPlaneBytes / 16), off = k % (int)(kPlaneBytes / 16);
            const uint8_t* src = plane == 0 ? sc.map : (plane == 1 ? sc.item : sc.light);
            ((u4*)(planes + ((size_t)plane * kLevels + level) * kPlaneBytes))[off] = ((const u4*)src)[off];
        }
        // spawn bit planes of the level (craftax_refresh_spawn_bits_level), no mobs yet
        if (t < kMap) {
            uint64_t all = 0, grave = 0, water = 0;
            for (int c = 0; c < kMap; c++) {
                const int b = sc.map[t * kMap + c];
                all |= (uint64_t)in_set(kSpawnAll, b) << c;
                grave |= (uint64_t)in_set(kSpawnGrave, b) << c;
                water |= (uint64_t)in_set(kSpawnWater, b) << c;
            }
            const size_t at = (size_t)(level * kMap + t) * n + e;
            A.spawn_all_bits[at] = all;
            A.spawn_grave_bits[at] = grave;
            A.spawn_water_bits[at] = water;
            A.mob_bits[at] = 0;
        }
        if (t < 2) {
            A.down_ladders[(size_t)(level * 2 + t) * n + e] = sc.ladder_down[t];
            A.up_ladders[(size_t)(level * 2 + t) * n + e] = sc.ladder_up[t];
        }
        __syncthreads();
    }
}

int alloc_arrays(EnvArrays& A, int n) {
    memset(&A, 0, sizeof(A));
    A.n = n;
    char* base = reinterpret_cast<char*>(&A);
    for (int f = 0; f < kNumFields; f++) {
        void* p = nullptr;
        const size_t bytes = kFieldTable[f].elem * (size_t)kFieldTable[f].count * (size_t)n;
        CFP_HIP_TRY(hipMalloc(&p, bytes));
        CFP_HIP_TRY(hipMemset(p, 0, bytes));
        *reinterpret_cast<void**>(base + kFieldTable[f].offset) = p;
    }
    CFP_HIP_TRY(hipMalloc((void**)&A.planes, kEnvPlaneBytes * (size_t)n));
    CFP_HIP_TRY(hipMemset(A.planes, 0, kEnvPlaneBytes * (size_t)n));
    CFP_HIP_TRY(hipMalloc((void**)&A.action_rng, sizeof(uint32_t) * (size_t)n));
    CFP_HIP_TRY(hipMemset(A.action_rng, 0, sizeof(uint32_t) * (size_t)n));
    return 0;
}
void free_arrays(EnvArrays& A) {
    char* base = reinterpret_cast<char*>(&A);
    for (int f = 0; f < kNumFields; f++) (void)hipFree(*reinterpret_cast<void**>(base + kFieldTable[f].offset));
    (void)hipFree(A.planes);
    (void)hipFree(A.action_rng);
    memset(&A, 0, sizeof(A));
}

// host states <-> arrays: each field is transposed on the host into [entry][count] and
// moved with one strided copy
template <class T, class Get>
int upload_field(T* dev, int entries, int n, int first, int count, std::vector<unsigned char>& tmp, Get get) {
    tmp.resize(sizeof(T) * (size_t)entries * (size_t)count);
    T* t = reinterpret_cast<T*>(tmp.data());
    for (int k = 0; k < entries; k++)
        for (int i = 0; i < count; i++) t[(size_t)k * count + i] = get(i, k);
    CFP_HIP_TRY(hipMemcpy2D(dev + first, sizeof(T) * (size_t)n, t, sizeof(T) * (size_t)count, sizeof(T) * (size_t)count,
                            (size_t)entries, hipMemcpyHostToDevice));
    return 0;
}
template <class T, class Set>
int download_field(const T* dev, int entries, int n, int first, int count, std::vector<unsigned char>& tmp, Set set) {
    tmp.resize(sizeof(T) * (size_t)entries * (size_t)count);
    T* t = reinterpret_cast<T*>(tmp.data());
    CFP_HIP_TRY(hipMemcpy2D(t, sizeof(T) * (size_t)count, dev + first, sizeof(T) * (size_t)n, sizeof(T) * (size_t)count,
                            (size_t)entries, hipMemcpyDeviceToHost));
    for (int k = 0; k < entries; k++)
        for (int i = 0; i < count; i++) set(i, k, t[(size_t)k * count + i]);
    return 0;
}

int import_states(EnvArrays& A, int first, int count, const cfp_env_state* states) {
    std::vector<cfp_env_state> derived(states, states + count);
    for (auto& st : derived) derive_spawn_planes(st);
    std::vector<unsigned char> tmp;
#define CFE_UP(name, type, entries, get, set)                                                               \
    if (upload_field<type>(A.name, entries, A.n, first, count, tmp, [&](int i, int k) -> type {            \
            const cfp_env_state& st = derived[i];                                                           \
            (void)k;                                                                                        \
            return (type)(get);                                                                             \
        }))                                                                                                 \
        return 1;
    CFE_FIELDS(CFE_UP)
#undef CFE_UP
    CFP_HIP_TRY(hipMemcpy2D(A.planes + (size_t)first * kEnvPlaneBytes, kEnvPlaneBytes, &states[0].map[0][0][0],
                            sizeof(cfp_env_state), kEnvPlaneBytes, (size_t)count, hipMemcpyHostToDevice));
    return 0;
}
int export_states(const EnvArrays& A, int first, int count, cfp_env_state* states) {
    std::vector<unsigned char> tmp;
    memset(states, 0, sizeof(cfp_env_state) * (size_t)count);
#define CFE_DOWN(name, type, entries, get, set)                                                             \
    if (download_field<type>(A.name, entries, A.n, first, count, tmp, [&](int i, int k, type v) {           \
            cfp_env_state& st = states[i];                                                                  \
            (void)k;                                                                                        \
            set;                                                                                            \
        }))                                                                                                 \
        return 1;
    CFE_FIELDS(CFE_DOWN)
#undef CFE_DOWN
    CFP_HIP_TRY(hipMemcpy2D(&states[0].map[0][0][0], sizeof(cfp_env_state), A.planes + (size_t)first * kEnvPlaneBytes,
                            kEnvPlaneBytes, kEnvPlaneBytes, (size_t)count, hipMemcpyDeviceToHost));
    return 0;
}

}  // namespace
}  // namespace cfp

struct cfp_env {
    cfp::EnvArrays live;
    cfp::EnvArrays pool;
    int pool_size = 0;
    float* light = nullptr;
    cfp_env_reset_rec* resets = nullptr;
    int* reset_count = nullptr;
    float* slots = nullptr;   // actions | rewards | terminals, n floats each
    // the `run` mode's outputs (CuPolicy.d_act / d_logprob / d_value and step_ctr,
    // craftax_full.cu:11770-11773): sampled actions (int32) | log-probabilities | values, n each,
    // then the 8-byte step counter of the draws and a zeroed word for the sampler's ticket
    float* run = nullptr;
};

static_assert(sizeof(cfp_env_state) % 8 == 0, "exchange struct is 8-byte aligned");
static_assert(offsetof(cfp_env_state, item_map) - offsetof(cfp_env_state, map) == 9 * 48 * 48 &&
                  offsetof(cfp_env_state, light_map) - offsetof(cfp_env_state, item_map) == 9 * 48 * 48,
              "the three maps are contiguous in the exchange struct");

extern "C" {

size_t cfp_env_state_bytes(void) { return sizeof(cfp_env_state); }

int cfp_env_light_table(float* out, int count) {
    CFP_REQUIRE(out != nullptr && count >= 0 && count <= CFP_ENV_MAX_TIMESTEPS + 1,
                "cfp_env_light_table: count must be 0..%d", CFP_ENV_MAX_TIMESTEPS + 1);
    for (int t = 0; t < count; t++) out[t] = cfenv::light_level(t);
    return 0;
}

int cfp_env_create(cfp_env** out, int n, int pool) {
    CFP_REQUIRE(out != nullptr, "cfp_env_create: NULL out");
    *out = nullptr;
    // the reference's own constraint (--envs a multiple of 32, craftax_full.cu:11820), the policy's too
    CFP_REQUIRE(n > 0 && n % 32 == 0, "cfp_env_create: env count %d is not a positive multiple of 32", n);
    CFP_REQUIRE(pool >= 0, "cfp_env_create: pool size %d is negative", pool);
    cfp_env* e = new cfp_env();
    memset(&e->live, 0, sizeof(e->live));
    memset(&e->pool, 0, sizeof(e->pool));
    int rc = cfp::alloc_arrays(e->live, n);
    if (rc == 0 && pool > 0) rc = cfp::alloc_arrays(e->pool, pool);
    e->pool_size = pool;
    std::vector<float> table(CFP_ENV_MAX_TIMESTEPS + 1);
    for (int t = 0; t <= CFP_ENV_MAX_TIMESTEPS; t++) table[t] = cfenv::light_level(t);
    auto fail = [&](hipError_t err, const char* what) {
        cfp::set_error("cfp_env_create: %s -> %s", what, hipGetErrorString(err));
        cfp_env_destroy(e);
        return 1;
    };
    if (rc != 0) {
        cfp_env_destroy(e);
        return 1;
    }
    hipError_t err;
    if ((err = hipMalloc((void**)&e->light, sizeof(float) * table.size())) != hipSuccess) return fail(err, "hipMalloc(light)");
    if ((err = hipMemcpy(e->light, table.data(), sizeof(float) * table.size(), hipMemcpyHostToDevice)) != hipSuccess)
        return fail(err, "hipMemcpy(light)");
    if ((err = hipMalloc((void**)&e->resets, sizeof(cfp_env_reset_rec) * (size_t)n)) != hipSuccess) return fail(err, "hipMalloc(resets)");
    if ((err = hipMalloc((void**)&e->reset_count, sizeof(int))) != hipSuccess) return fail(err, "hipMalloc(reset_count)");
    if ((err = hipMemset(e->reset_count, 0, sizeof(int))) != hipSuccess) return fail(err, "hipMemset(reset_count)");
    if ((err = hipMalloc((void**)&e->slots, sizeof(float) * 3 * (size_t)n)) != hipSuccess) return fail(err, "hipMalloc(slots)");
    if ((err = hipMemset(e->slots, 0, sizeof(float) * 3 * (size_t)n)) != hipSuccess) return fail(err, "hipMemset(slots)");
    if ((err = hipMalloc((void**)&e->run, sizeof(float) * 3 * (size_t)n + 16)) != hipSuccess) return fail(err, "hipMalloc(run)");
    if ((err = hipMemset(e->run, 0, sizeof(float) * 3 * (size_t)n + 16)) != hipSuccess) return fail(err, "hipMemset(run)");
    *out = e;
    return 0;
}

void cfp_env_destroy(cfp_env* e) {
    if (e == nullptr) return;
    cfp::free_arrays(e->live);
    cfp::free_arrays(e->pool);
    (void)hipFree(e->light);
    (void)hipFree(e->resets);
    (void)hipFree(e->reset_count);
    (void)hipFree(e->slots);
    (void)hipFree(e->run);
    delete e;
}

int cfp_env_num_envs(const cfp_env* e) { return e ? e->live.n : 0; }
float* cfp_env_actions(const cfp_env* e) { return e ? e->slots : nullptr; }
float* cfp_env_rewards(const cfp_env* e) { return e ? e->slots + e->live.n : nullptr; }
float* cfp_env_terminals(const cfp_env* e) { return e ? e->slots + 2 * (size_t)e->live.n : nullptr; }
int cfp_env_pool_size(const cfp_env* e) { return e ? e->pool_size : 0; }
int32_t* cfp_env_run_actions(const cfp_env* e) { return e ? reinterpret_cast<int32_t*>(e->run) : nullptr; }
float* cfp_env_run_logprobs(const cfp_env* e) { return e ? e->run + e->live.n : nullptr; }
float* cfp_env_run_values(const cfp_env* e) { return e ? e->run + 2 * (size_t)e->live.n : nullptr; }
uint64_t* cfp_env_run_counter(const cfp_env* e) {
    return e ? reinterpret_cast<uint64_t*>(e->run + 3 * (size_t)e->live.n) : nullptr;
}

int cfp_env_import(cfp_env* e, int first, int count, const cfp_env_state* states) {
    CFP_REQUIRE(e != nullptr && states != nullptr, "cfp_env_import: NULL argument");
    CFP_REQUIRE(first >= 0 && count > 0 && first + count <= e->live.n, "cfp_env_import: envs [%d, %d) outside 0..%d", first,
                first + count, e->live.n);
    CFP_HIP_TRY(hipDeviceSynchronize());
    return cfp::import_states(e->live, first, count, states);
}
int cfp_env_pool_import(cfp_env* e, int first, int count, const cfp_env_state* states) {
    CFP_REQUIRE(e != nullptr && states != nullptr, "cfp_env_pool_import: NULL argument");
    CFP_REQUIRE(first >= 0 && count > 0 && first + count <= e->pool_size, "cfp_env_pool_import: entries [%d, %d) outside 0..%d",
                first, first + count, e->pool_size);
    CFP_HIP_TRY(hipDeviceSynchronize());
    return cfp::import_states(e->pool, first, count, states);
}
int cfp_env_export(cfp_env* e, int first, int count, cfp_env_state* states) {
    CFP_REQUIRE(e != nullptr && states != nullptr, "cfp_env_export: NULL argument");
    CFP_REQUIRE(first >= 0 && count > 0 && first + count <= e->live.n, "cfp_env_export: envs [%d, %d) outside 0..%d", first,
                first + count, e->live.n);
    CFP_HIP_TRY(hipDeviceSynchronize());
    return cfp::export_states(e->live, first, count, states);
}

int cfp_env_seed_actions(cfp_env* e, uint64_t seed, void* stream) {
    CFP_REQUIRE(e != nullptr, "cfp_env_seed_actions: NULL env");
    hipLaunchKernelGGL(cfp::k_env_seed_actions, dim3((e->live.n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       e->live.action_rng, e->live.n, seed);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_env_step(cfp_env* e, const float* d_actions, float* d_rewards, float* d_terminals, void* stream) {
    CFP_REQUIRE(e != nullptr && d_rewards != nullptr && d_terminals != nullptr, "cfp_env_step: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(cfp::k_env_zero, dim3(1), dim3(1), 0, st, e->reset_count);
    hipLaunchKernelGGL(cfp::k_env_step, dim3((e->live.n + cfp::kWave - 1) / cfp::kWave), dim3(cfp::kWave), 0, st, e->live, e->light, d_actions,
                       d_rewards, d_terminals, e->resets, e->reset_count, (float*)nullptr, (uint8_t*)nullptr);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

const int* cfp_env_reset_count(const cfp_env* e) { return e ? e->reset_count : nullptr; }
const cfp_env_reset_rec* cfp_env_reset_list(const cfp_env* e) { return e ? e->resets : nullptr; }

namespace cfp {
namespace {
// fields a fresh state holds zero in and that the generator kernel does not write itself
int zero_field_list(const EnvArrays& A, FieldList& fl) {
    const size_t skip[] = {offsetof(EnvArrays, rng_key), offsetof(EnvArrays, mob_health),
                           offsetof(EnvArrays, mob_projectile_directions), offsetof(EnvArrays, player_projectile_directions),
                           offsetof(EnvArrays, potion_mapping), offsetof(EnvArrays, state_rng),
                           offsetof(EnvArrays, monsters_killed), offsetof(EnvArrays, player_position),
                           offsetof(EnvArrays, mob_bits), offsetof(EnvArrays, spawn_all_bits),
                           offsetof(EnvArrays, spawn_grave_bits), offsetof(EnvArrays, spawn_water_bits),
                           offsetof(EnvArrays, down_ladders), offsetof(EnvArrays, up_ladders)};
    int m = 0;
    for (int f = 0; f < kNumFields; f++) {
        bool skipped = false;
        for (size_t off : skip) skipped = skipped || off == kFieldTable[f].offset;
        if (skipped) continue;
        fl.ptr[m] = *reinterpret_cast<void* const*>(reinterpret_cast<const char*>(&A) + kFieldTable[f].offset);
        fl.elem[m] = (int)kFieldTable[f].elem;
        fl.count[m] = kFieldTable[f].count;
        m++;
    }
    return m;
}
}  // namespace
}  // namespace cfp

int cfp_env_init(cfp_env* e, uint64_t seed, void* stream) {
    CFP_REQUIRE(e != nullptr, "cfp_env_init: NULL env");
    cfp::FieldList fl;
    const int m = cfp::zero_field_list(e->live, fl);
    const int grid = e->live.n * cfp::kGenJobs < 8192 ? e->live.n * cfp::kGenJobs : 8192;
    hipLaunchKernelGGL((cfp::k_env_worldgen<false, cfp::kGenThreads>), dim3(grid), dim3(cfp::kGenThreads), 0, (hipStream_t)stream, e->live, fl,
                       e->light, nullptr, nullptr, seed, m);
    CFP_HIP_TRY(hipGetLastError());
    return cfp_env_seed_actions(e, seed, stream);
}

int cfp_env_pool_fill(cfp_env* e, uint64_t seed, void* stream) {
    CFP_REQUIRE(e != nullptr, "cfp_env_pool_fill: NULL env");
    CFP_REQUIRE(e->pool_size > 0, "cfp_env_pool_fill: this env object was created without a reset pool");
    cfp::FieldList fl;
    const int m = cfp::zero_field_list(e->pool, fl);
    hipLaunchKernelGGL((cfp::k_env_worldgen<false, cfp::kGenThreads>), dim3(e->pool_size * cfp::kGenJobs < 8192 ? e->pool_size * cfp::kGenJobs : 8192),
                       dim3(cfp::kGenThreads), 0,
                       (hipStream_t)stream, e->pool, fl, e->light, nullptr, nullptr, seed, m);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_env_reset(cfp_env* e, void* stream) {
    CFP_REQUIRE(e != nullptr, "cfp_env_reset: NULL env");
    cfp::FieldList fl;
    const int m = cfp::zero_field_list(e->live, fl);
    // the list is short (a fraction of a percent of the envs per step): a fixed grid strides it
    const int grid = e->live.n * cfp::kGenJobs < 4608 ? e->live.n * cfp::kGenJobs : 4608;
    // about one env in 240 finishes per step under random actions: up to 16 384 envs that is
    // fewer jobs than the GPU holds at once, and the wider workgroup finishes each sooner
    if (e->live.n <= 16384)
        hipLaunchKernelGGL((cfp::k_env_worldgen<true, cfp::kGenThreadsFew>), dim3(grid), dim3(cfp::kGenThreadsFew), 0,
                           (hipStream_t)stream, e->live, fl, e->light, e->resets, e->reset_count, 0ull, m);
    else
        hipLaunchKernelGGL((cfp::k_env_worldgen<true, cfp::kGenThreads>), dim3(grid), dim3(cfp::kGenThreads), 0,
                           (hipStream_t)stream, e->live, fl, e->light, e->resets, e->reset_count, 0ull, m);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_env_generate_host(uint32_t seed, int count, cfp_env_state* states) {
    CFP_REQUIRE(states != nullptr && count >= 0, "cfp_env_generate_host: bad argument");
    std::vector<cfenv::FloorScratch> sc(1);
    for (int i = 0; i < count; i++) cfenv::generate_env_host(seed + (uint32_t)i, states[i], sc[0]);
    return 0;
}

int cfp_env_fetch_resets(const cfp_env* e, cfp_env_reset_rec* out, int max, int* count, void* stream) {
    CFP_REQUIRE(e != nullptr && count != nullptr && (out != nullptr || max == 0) && max >= 0,
                "cfp_env_fetch_resets: bad argument");
    CFP_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    CFP_HIP_TRY(hipMemcpy(count, e->reset_count, sizeof(int), hipMemcpyDeviceToHost));
    const int take = *count < max ? *count : max;
    if (take > 0) CFP_HIP_TRY(hipMemcpy(out, e->resets, sizeof(cfp_env_reset_rec) * (size_t)take, hipMemcpyDeviceToHost));
    return 0;
}

int cfp_env_reset_from_pool(cfp_env* e, void* stream) {
    CFP_REQUIRE(e != nullptr, "cfp_env_reset_from_pool: NULL env");
    CFP_REQUIRE(e->pool_size > 0, "cfp_env_reset_from_pool: this env object was created without a reset pool");
    cfp::CopyTable t;
    int rng_key_field = -1;
    for (int f = 0; f < cfp::kNumFields; f++) {
        const size_t off = cfp::kFieldTable[f].offset;
        t.src[f] = *reinterpret_cast<void* const*>(reinterpret_cast<const char*>(&e->pool) + off);
        t.dst[f] = *reinterpret_cast<void* const*>(reinterpret_cast<const char*>(&e->live) + off);
        t.elem[f] = (int)cfp::kFieldTable[f].elem;
        t.count[f] = cfp::kFieldTable[f].count;
        if (off == offsetof(cfp::EnvArrays, rng_key)) rng_key_field = f;
    }
    const int grid = e->live.n < 1024 ? e->live.n : 1024;
    hipLaunchKernelGGL(cfp::k_env_reset_from_pool, dim3(grid), dim3(256), 0, (hipStream_t)stream, t, e->live, e->pool,
                       e->resets, e->reset_count, rng_key_field);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_env_view(const cfp_env* e, cfp_env_soa* soa, const uint8_t** d_map, const uint8_t** d_item_map,
                 const uint8_t** d_light_map, size_t* env_stride, size_t* level_stride) {
    CFP_REQUIRE(e != nullptr && soa != nullptr, "cfp_env_view: NULL argument");
    const cfp::EnvArrays& A = e->live;
    soa->player_position = A.player_position;
    soa->player_level = A.player_level;
    soa->player_direction = A.player_direction;
    soa->player_health = A.player_health;
    soa->player_food = A.player_food;
    soa->player_drink = A.player_drink;
    soa->player_energy = A.player_energy;
    soa->player_mana = A.player_mana;
    soa->player_xp = A.player_xp;
    soa->player_dexterity = A.player_dexterity;
    soa->player_strength = A.player_strength;
    soa->player_intelligence = A.player_intelligence;
    soa->is_sleeping = A.is_sleeping;
    soa->is_resting = A.is_resting;
    soa->inv_wood = A.inv_wood;
    soa->inv_stone = A.inv_stone;
    soa->inv_coal = A.inv_coal;
    soa->inv_iron = A.inv_iron;
    soa->inv_diamond = A.inv_diamond;
    soa->inv_sapphire = A.inv_sapphire;
    soa->inv_ruby = A.inv_ruby;
    soa->inv_sapling = A.inv_sapling;
    soa->inv_torches = A.inv_torches;
    soa->inv_arrows = A.inv_arrows;
    soa->inv_books = A.inv_books;
    soa->inv_pickaxe = A.inv_pickaxe;
    soa->inv_sword = A.inv_sword;
    soa->inv_bow = A.inv_bow;
    soa->inv_potions = A.inv_potions;
    soa->inv_armour = A.inv_armour;
    soa->sword_enchantment = A.sword_enchantment;
    soa->bow_enchantment = A.bow_enchantment;
    soa->armour_enchantments = A.armour_enchantments;
    soa->light_level = A.light_level;
    soa->learned_spells = A.learned_spells;
    soa->monsters_killed = A.monsters_killed;
    soa->boss_timesteps_to_spawn_this_round = A.boss_timesteps_to_spawn_this_round;
    soa->mob_type_id = A.mob_type_id;
    soa->mob_mask = A.mob_mask;
    soa->mob_position = A.mob_position;
    soa->n_stride = (size_t)A.n;
    if (d_map) *d_map = A.planes;
    if (d_item_map) *d_item_map = A.planes + cfp::kLevels * cfp::kPlaneBytes;
    if (d_light_map) *d_light_map = A.planes + 2 * cfp::kLevels * cfp::kPlaneBytes;
    if (env_stride) *env_stride = cfp::kEnvPlaneBytes;
    if (level_stride) *level_stride = cfp::kPlaneBytes;
    return 0;
}

int cfp_env_record_obs(const cfp_env* e, uint8_t* d_rec_row, void* stream) {
    CFP_REQUIRE(e != nullptr && d_rec_row != nullptr, "cfp_env_record_obs: NULL argument");
    cfp_env_soa soa;
    const uint8_t *m, *im, *lm;
    size_t es, ls;
    if (cfp_env_view(e, &soa, &m, &im, &lm, &es, &ls)) return 1;
    return cfp_record_obs_soa(&soa, m, im, lm, es, ls, nullptr, d_rec_row, e->live.n, stream);
}

// cu_rollout_step_plain (craftax_full.cu:12089-12092): the step of the reference's `run` mode,
// no slabs.  Records of the current states into the policy's own record buffer, forward on its
// live state (zeroed where the last step ended an episode) and the draw, the env step with the
// drawn actions, finished envs replaced.
int cfp_env_run_step(cfp_policy* p, cfp_env* e, uint64_t seed, void* stream) {
    CFP_REQUIRE(p != nullptr && e != nullptr, "cfp_env_run_step: NULL argument");
    CFP_REQUIRE(p->n == e->live.n, "cfp_env_run_step: the policy holds %d envs, the env object %d", p->n, e->live.n);
    CFP_REQUIRE(p->variant == 0, "cfp_env_run_step: the env on the device is the full game");
    const size_t n = (size_t)e->live.n;
    if (cfp::env_record_obs_zero(e, p->rec, stream)) return 1;
    const cfp::SampleOut so{cfp_env_run_actions(e), cfp_env_run_logprobs(e), cfp_env_run_values(e), e->slots, seed,
                            cfp_env_run_counter(e), reinterpret_cast<unsigned*>(cfp_env_run_counter(e) + 1)};
    if (cfp::forward_and_sample(p, p->rec, e->slots + 2 * n, nullptr, e->live.n, so, (hipStream_t)stream)) return 1;
    if (cfp::env_step_rows(e, nullptr, nullptr, stream)) return 1;
    return e->pool_size > 0 ? cfp_env_reset_from_pool(e, stream) : cfp_env_reset(e, stream);
}

}  // extern "C"

int cfp::env_record_obs_zero(const cfp_env* e, uint8_t* d_rec_row, void* stream) {
    CFP_REQUIRE(e != nullptr && d_rec_row != nullptr, "env_record_obs_zero: NULL argument");
    cfp_env_soa soa;
    const uint8_t *m, *im, *lm;
    size_t es, ls;
    if (cfp_env_view(e, &soa, &m, &im, &lm, &es, &ls)) return 1;
    return cfp::record_obs_soa_zero(&soa, m, im, lm, es, ls, d_rec_row, e->live.n, e->reset_count, stream);
}

int cfp::env_step_rows(cfp_env* e, float* d_r_reward_row, uint8_t* d_r_done_row, void* stream) {
    CFP_REQUIRE(e != nullptr && (d_r_reward_row == nullptr) == (d_r_done_row == nullptr), "env_step_rows: bad argument");
    const size_t n = (size_t)e->live.n;
    hipLaunchKernelGGL(cfp::k_env_step, dim3((e->live.n + cfp::kWave - 1) / cfp::kWave), dim3(cfp::kWave), 0,
                       (hipStream_t)stream, e->live, e->light, e->slots, e->slots + n, e->slots + 2 * n, e->resets,
                       e->reset_count, d_r_reward_row, d_r_done_row);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}
