// Host-side pieces of the env step: the exchange struct <-> hot scalars, a storage object
// over one cfp_env_state (what the host build of env_logic.h runs on), the light-level
// table and the spawn bit planes derived from the map.
#pragma once

#include <math.h>
#include <string.h>

#include "../../include/cfp_env.h"
#include "env_logic.h"
#include "env_worldgen.h"

namespace cfenv {

inline void load_hot(const cfp_env_state& st, Hot& h) {
    h.pr = st.player_position[0];
    h.pc = st.player_position[1];
    h.level = st.player_level;
    h.dir = st.player_direction;
    h.health = st.player_health;
    h.food = st.player_food;
    h.drink = st.player_drink;
    h.energy = st.player_energy;
    h.mana = st.player_mana;
    h.sleeping = st.is_sleeping != 0;
    h.resting = st.is_resting != 0;
    h.recover = st.player_recover;
    h.hunger = st.player_hunger;
    h.thirst = st.player_thirst;
    h.fatigue = st.player_fatigue;
    h.recover_mana = st.player_recover_mana;
    h.xp = st.player_xp;
    h.dex = st.player_dexterity;
    h.str = st.player_strength;
    h.intel = st.player_intelligence;
    h.wood = st.wood;
    h.stone = st.stone;
    h.coal = st.coal;
    h.iron = st.iron;
    h.diamond = st.diamond;
    h.sapling = st.sapling;
    h.pickaxe = st.pickaxe;
    h.sword = st.sword;
    h.bow = st.bow;
    h.arrows = st.arrows;
    for (int i = 0; i < 4; i++) h.armour[i] = st.armour[i];
    h.torches = st.torches;
    h.ruby = st.ruby;
    h.sapphire = st.sapphire;
    for (int i = 0; i < 6; i++) h.potions[i] = st.potions[i];
    h.books = st.books;
    h.spell[0] = st.learned_spells[0] != 0;
    h.spell[1] = st.learned_spells[1] != 0;
    h.sword_ench = st.sword_enchantment;
    h.bow_ench = st.bow_enchantment;
    for (int i = 0; i < 4; i++) h.armour_ench[i] = st.armour_enchantments[i];
    h.boss_progress = st.boss_progress;
    h.boss_timer = st.boss_timesteps_to_spawn_this_round;
    h.light_level = st.light_level;
    h.timestep = st.timestep;
    h.ach[0] = h.ach[1] = h.ach[2] = 0;
    for (int a = 0; a < CFP_ENV_ACHIEVEMENTS; a++)
        if (st.achievements[a]) h.ach[a >> 5] |= 1u << (a & 31);
    h.plant_mask = 0;
    for (int i = 0; i < kPlants; i++)
        if (st.growing_plants_mask[i]) h.plant_mask |= 1u << i;
}

inline void store_hot(const Hot& h, cfp_env_state& st) {
    st.player_position[0] = h.pr;
    st.player_position[1] = h.pc;
    st.player_level = h.level;
    st.player_direction = h.dir;
    st.player_health = h.health;
    st.player_food = h.food;
    st.player_drink = h.drink;
    st.player_energy = h.energy;
    st.player_mana = h.mana;
    st.is_sleeping = h.sleeping;
    st.is_resting = h.resting;
    st.player_recover = h.recover;
    st.player_hunger = h.hunger;
    st.player_thirst = h.thirst;
    st.player_fatigue = h.fatigue;
    st.player_recover_mana = h.recover_mana;
    st.player_xp = h.xp;
    st.player_dexterity = h.dex;
    st.player_strength = h.str;
    st.player_intelligence = h.intel;
    st.wood = h.wood;
    st.stone = h.stone;
    st.coal = h.coal;
    st.iron = h.iron;
    st.diamond = h.diamond;
    st.sapling = h.sapling;
    st.pickaxe = h.pickaxe;
    st.sword = h.sword;
    st.bow = h.bow;
    st.arrows = h.arrows;
    for (int i = 0; i < 4; i++) st.armour[i] = h.armour[i];
    st.torches = h.torches;
    st.ruby = h.ruby;
    st.sapphire = h.sapphire;
    for (int i = 0; i < 6; i++) st.potions[i] = h.potions[i];
    st.books = h.books;
    st.learned_spells[0] = h.spell[0];
    st.learned_spells[1] = h.spell[1];
    st.sword_enchantment = h.sword_ench;
    st.bow_enchantment = h.bow_ench;
    for (int i = 0; i < 4; i++) st.armour_enchantments[i] = h.armour_ench[i];
    st.boss_progress = h.boss_progress;
    st.boss_timesteps_to_spawn_this_round = h.boss_timer;
    st.light_level = h.light_level;
    st.timestep = h.timestep;
    for (int a = 0; a < CFP_ENV_ACHIEVEMENTS; a++) st.achievements[a] = (h.ach[a >> 5] >> (a & 31)) & 1u;
    for (int i = 0; i < kPlants; i++) st.growing_plants_mask[i] = (h.plant_mask >> i) & 1u;
}

// craftax_refresh_spawn_bits_level (craftax_full.c:3336-3355) for all levels
inline void derive_spawn_planes(cfp_env_state& st) {
    for (int l = 0; l < kLevels; l++)
        for (int r = 0; r < kMap; r++) {
            uint64_t all = 0, grave = 0, water = 0;
            for (int c = 0; c < kMap; c++) {
                const int b = st.map[l][r][c];
                all |= (uint64_t)in_set(kSpawnAll, b) << c;
                grave |= (uint64_t)in_set(kSpawnGrave, b) << c;
                water |= (uint64_t)in_set(kSpawnWater, b) << c;
            }
            st.spawn_all_bits[l][r] = all;
            st.spawn_grave_bits[l][r] = grave;
            st.spawn_water_bits[l][r] = water;
        }
}

// craftax_calculate_light_level_native (craftax_full.c:3760-3767) as the reference's
// -ffast-math build evaluates it: the division by the day length is a multiplication by
// the rounded reciprocal, powf(x, 3) is x * x * x, and 1 - a * a * a is one fused
// multiply-add; cosf and fmodf are the C library's.  Kept in separate statements so that
// the host compiler cannot contract anything else.
inline float light_level(int timestep) {
    const float day = (float)timestep * (1.0f / 300.0f);
    const float progress = fmodf(day, 1.0f) + 0.3f;
    const float angle = 3.14159265358979323846f * progress;
    const float a = fabsf(cosf(angle));
    const float aa = a * a;
    return fmaf(-aa, a, 1.0f);
}

// Storage over one host state (see env_logic.h for the interface).
struct HostStore {
    cfp_env_state* st;
    const float* light;
    int lvl = 0;

    int blk(int l, int r, int c) const { return st->map[l][r][c]; }
    void put_blk_raw(int l, int r, int c, int b) { st->map[l][r][c] = (uint8_t)b; }
    int item(int l, int r, int c) const { return st->item_map[l][r][c]; }
    void put_item(int l, int r, int c, int v) { st->item_map[l][r][c] = (uint8_t)v; }
    int lum(int l, int r, int c) const { return st->light_map[l][r][c]; }
    void put_lum(int l, int r, int c, int v) { st->light_map[l][r][c] = (uint8_t)v; }
    uint64_t mobrow(int l, int r) const { return st->mob_bits[l][r]; }
    void put_mobrow(int l, int r, uint64_t v) { st->mob_bits[l][r] = v; }
    uint64_t* plane(int kind) {
        return kind == SK_ALL ? &st->spawn_all_bits[0][0] : kind == SK_GRAVE ? &st->spawn_grave_bits[0][0] : &st->spawn_water_bits[0][0];
    }
    uint64_t spawnrow(int kind, int l, int r) { return plane(kind)[l * kMap + r]; }
    void put_spawnrow(int kind, int l, int r, uint64_t v) { plane(kind)[l * kMap + r] = v; }

    int m_row(int p, int i) const { return st->mob_position[p][lvl][i][0]; }
    int m_col(int p, int i) const { return st->mob_position[p][lvl][i][1]; }
    int m_cd(int p, int i) const { return st->mob_attack_cooldown[p][lvl][i]; }
    int m_type(int p, int i) const { return st->mob_type_id[p][lvl][i]; }
    bool m_mask(int p, int i) const { return st->mob_mask[p][lvl][i] != 0; }
    float m_hp(int p, int i) const { return st->mob_health[p][lvl][i]; }
    void set_m_pos(int p, int i, int r, int c) {
        st->mob_position[p][lvl][i][0] = r;
        st->mob_position[p][lvl][i][1] = c;
    }
    void set_m_cd(int p, int i, int v) { st->mob_attack_cooldown[p][lvl][i] = v; }
    void set_m_type(int p, int i, int v) { st->mob_type_id[p][lvl][i] = v; }
    void set_m_mask(int p, int i, bool v) { st->mob_mask[p][lvl][i] = v; }
    void set_m_hp(int p, int i, float v) { st->mob_health[p][lvl][i] = v; }
    int32_t (*dirs(int p))[3][2] { return p == P_MOB_PROJ ? st->mob_projectile_directions : st->player_projectile_directions; }
    int pd_r(int p, int i) { return dirs(p)[lvl][i][0]; }
    int pd_c(int p, int i) { return dirs(p)[lvl][i][1]; }
    void set_pd(int p, int i, int r, int c) {
        dirs(p)[lvl][i][0] = r;
        dirs(p)[lvl][i][1] = c;
    }
    int kills(int l) const { return st->monsters_killed[l]; }
    void set_kills(int l, int v) { st->monsters_killed[l] = v; }
    bool chest(int l) const { return st->chests_opened[l] != 0; }
    void set_chest(int l) { st->chests_opened[l] = 1; }
    int ladder_down(int l, int a) const { return st->down_ladders[l][a]; }
    int ladder_up(int l, int a) const { return st->up_ladders[l][a]; }
    int potion_effect(int i) const { return st->potion_mapping[i]; }
    int plant_r(int i) const { return st->growing_plants_positions[i][0]; }
    int plant_c(int i) const { return st->growing_plants_positions[i][1]; }
    int plant_age(int i) const { return st->growing_plants_age[i]; }
    void set_plant(int i, int r, int c) {
        st->growing_plants_positions[i][0] = r;
        st->growing_plants_positions[i][1] = c;
    }
    void set_plant_age(int i, int a) { st->growing_plants_age[i] = a; }
    void open_level(int l) { lvl = l; }
    void stamp(int) {}
    float light_at(int t) const { return light[t < kMaxTimesteps ? t : kMaxTimesteps]; }
};

// a group of one thread for env_worldgen.h; cos / sin are the C library's
struct HostGroup {
    int tid() const { return 0; }
    int nt() const { return 1; }
    void sync() {}
    int gmaxi(int v) { return v; }
    void gminmax4(float (&)[4], float (&)[4]) {}   // one member: its own extrema are the group's
    int gscan(int v, int& total) {
        total = v;
        return 0;
    }
    void stamp(int) {}
    float cosine(float x) { return cosf(x); }
    float sine(float x) { return sinf(x); }
};

// craftax_generate_world_from_key (craftax_full.c:2050-2142): a fresh state from a world key.
// rng_key is left alone (it belongs to the env, not to the world).
inline void generate_world_host(uint64_t world_key, cfp_env_state& st, FloorScratch& sc) {
    const uint32_t keep0 = st.rng_key[0], keep1 = st.rng_key[1];
    memset(&st, 0, sizeof(st));
    st.rng_key[0] = keep0;
    st.rng_key[1] = keep1;
    HostGroup g;
    for (int l = 0; l < kLevels; l++) {
        generate_floor(g, sc, world_key, l);
        memcpy(st.map[l], sc.map, kCells);
        memcpy(st.item_map[l], sc.item, kCells);
        memcpy(st.light_map[l], sc.light, kCells);
        for (int a = 0; a < 2; a++) {
            st.down_ladders[l][a] = sc.ladder_down[a];
            st.up_ladders[l][a] = sc.ladder_up[a];
        }
    }
    for (int p = 0; p < CFP_ENV_MOB_CLASSES; p++)
        for (int l = 0; l < kLevels; l++)
            for (int i = 0; i < (p == P_RANGED ? 2 : 3); i++) st.mob_health[p][l][i] = 1.0f;
    for (int l = 0; l < kLevels; l++)
        for (int i = 0; i < 3; i++)
            for (int a = 0; a < 2; a++) st.mob_projectile_directions[l][i][a] = st.player_projectile_directions[l][i][a] = 1;
    int32_t perm[6];
    potion_permutation(world_key, perm);
    for (int i = 0; i < 6; i++) st.potion_mapping[i] = perm[i];
    const uint64_t sk = world_state_key(world_key);
    st.state_rng[0] = (uint32_t)sk;
    st.state_rng[1] = (uint32_t)(sk >> 32);
    st.monsters_killed[0] = 10;
    st.player_position[0] = st.player_position[1] = kMap / 2;
    st.player_direction = A_UP;
    st.player_health = 9.0f;
    st.player_food = st.player_drink = st.player_energy = st.player_mana = 9;
    st.player_dexterity = st.player_strength = st.player_intelligence = 1;
    st.boss_timesteps_to_spawn_this_round = 7;
    st.light_level = light_level(0);
    derive_spawn_planes(st);
}
// c_init's state for an env created with `seed` (craftax_reset_state_from_seed, :3601-3614)
inline void generate_env_host(uint32_t seed, cfp_env_state& st, FloorScratch& sc) {
    const uint64_t k = seed_key(seed);
    const uint64_t env_key = lcg(k), reset_key = lcg(env_key);
    generate_world_host(world_key_of_reset(reset_key), st, sc);
    st.rng_key[0] = (uint32_t)env_key;
    st.rng_key[1] = (uint32_t)(env_key >> 32);
}

// c_step_gameplay (craftax_full.c:3981-4011) without the reset, on one host state
inline void host_step(cfp_env_state& st, float action, const float* light, float* reward, float* terminal,
                      uint32_t reset_key[2]) {
    const StepKeys k = split_env_key((uint64_t)st.rng_key[1] << 32 | st.rng_key[0]);
    Hot h;
    load_hot(st, h);
    HostStore s{&st, light};
    SpawnPlan plan;
    const StepOut out = step(s, h, clamp_action(action), k.step_rng, plan);
    run_spawns(s, h, plan);
    store_hot(h, st);
    st.state_rng[0] = (uint32_t)out.state_rng;
    st.state_rng[1] = (uint32_t)(out.state_rng >> 32);
    st.rng_key[0] = (uint32_t)k.env_key;
    st.rng_key[1] = (uint32_t)(k.env_key >> 32);
    *reward = out.reward;
    *terminal = out.done ? 1.0f : 0.0f;
    reset_key[0] = (uint32_t)k.reset_key;
    reset_key[1] = (uint32_t)(k.reset_key >> 32);
}

}  // namespace cfenv
