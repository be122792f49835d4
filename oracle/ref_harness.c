/*
 * Compiled-reference checker.  TEST INFRASTRUCTURE ONLY.
 *
 * This translation unit #includes the reference's craftax_full.c from where it
 * lies (path given by -DCF_REF_SRC on the command line, see Makefile; nothing
 * of it is copied into this repository) with -DCRAFTAX_COMPACT_OBS, and wraps
 * its own functions -- cf_vec_init, c_step, the xorshift32 % 43 action stream
 * of cf_run_hash (craftax_full.c:8349-8353) and
 * craftax_encode_compact_observation (:2830) -- behind a small C interface
 * that the tests drive through ctypes.  For the env step it also converts the
 * reference's CraftaxState to and from the library's exchange struct
 * (cfp_env_state) and steps single envs with a given action, handing out the
 * state as it was before the reference's own reset replaced it.
 * Output: oracle/_ref/libcfref.so.
 */
#define main cf_ref_main
#include CF_REF_SRC
#undef main

#include "../include/cfp.h"
#include "../include/cfp_env.h"

static CfVec g_vec;
static int g_live = 0;

int cfref_obs_bytes(void) { return (int)(CRAFTAX_OBS_SIZE * sizeof(CraftaxObs)); }
int cfref_state_bytes(void) { return (int)sizeof(CraftaxState); }

void cfref_free(void) {
    if (g_live) cf_vec_free(&g_vec);
    g_live = 0;
}

/* cf_vec_init exactly as `craftax_full hash` calls it (single thread). */
int cfref_init(int num_envs, uint64_t seed) {
    cfref_free();
    cf_vec_init(&g_vec, num_envs, seed, /*parallel=*/0);
    g_live = 1;
    return 0;
}

/* One step of the deterministic random-action rollout (cf_run_hash loop body). */
void cfref_step(void) {
    for (int i = 0; i < g_vec.num_envs; i++) {
        g_vec.actions[i] =
            (float)(cf_xorshift32(&g_vec.action_rng[i]) % CRAFTAX_NUM_ACTIONS);
        c_step(&g_vec.envs[i]);
    }
}

const uint8_t* cfref_observations(void) { return (const uint8_t*)g_vec.observations; }
const float* cfref_terminals(void) { return g_vec.terminals; }
const float* cfref_rewards(void) { return g_vec.rewards; }

static void fill_mobs3(const CraftaxWGMobs3* m, int level, int slot0,
                       cfp_env_scalars* out) {
    for (int i = 0; i < 3; i++) {
        out->mob_type_id[slot0 + i] = m->type_id[level][i];
        out->mob_mask[slot0 + i] = m->mask[level][i] ? 1 : 0;
        out->mob_position[slot0 + i][0] = m->position[level][i][0];
        out->mob_position[slot0 + i][1] = m->position[level][i][1];
    }
}

/* The encoder's inputs for one env: scalars plus the three 48x48 planes of the
 * player's level (planes = map | item_map | light_map, 3 x 2304 bytes). */
void cfref_view(int env, cfp_env_scalars* out, uint8_t* planes) {
    const CraftaxWorldState* s =
        (const CraftaxWorldState*)(const void*)g_vec.envs[env].state;
    memset(out, 0, sizeof(*out));
    out->player_position[0] = s->player_position[0];
    out->player_position[1] = s->player_position[1];
    out->player_level = s->player_level;
    out->player_direction = s->player_direction;
    out->player_health = s->player_health;
    out->player_food = s->player_food;
    out->player_drink = s->player_drink;
    out->player_energy = s->player_energy;
    out->player_mana = s->player_mana;
    out->player_xp = s->player_xp;
    out->player_dexterity = s->player_dexterity;
    out->player_strength = s->player_strength;
    out->player_intelligence = s->player_intelligence;
    out->is_sleeping = s->is_sleeping ? 1 : 0;
    out->is_resting = s->is_resting ? 1 : 0;
    out->wood = s->inventory.wood;
    out->stone = s->inventory.stone;
    out->coal = s->inventory.coal;
    out->iron = s->inventory.iron;
    out->diamond = s->inventory.diamond;
    out->sapphire = s->inventory.sapphire;
    out->ruby = s->inventory.ruby;
    out->sapling = s->inventory.sapling;
    out->torches = s->inventory.torches;
    out->arrows = s->inventory.arrows;
    out->books = s->inventory.books;
    out->pickaxe = s->inventory.pickaxe;
    out->sword = s->inventory.sword;
    out->bow = s->inventory.bow;
    for (int i = 0; i < 6; i++) out->potions[i] = s->inventory.potions[i];
    for (int i = 0; i < 4; i++) out->armour[i] = s->inventory.armour[i];
    out->sword_enchantment = s->sword_enchantment;
    out->bow_enchantment = s->bow_enchantment;
    for (int i = 0; i < 4; i++) out->armour_enchantments[i] = s->armour_enchantments[i];
    out->light_level = s->light_level;
    out->learned_spells[0] = s->learned_spells[0] ? 1 : 0;
    out->learned_spells[1] = s->learned_spells[1] ? 1 : 0;
    out->monsters_killed_level = s->monsters_killed[s->player_level];
    out->boss_timesteps_to_spawn_this_round = s->boss_timesteps_to_spawn_this_round;
    const int ml = craftax_wg_jax_index(s->player_level, CRAFTAX_WG_NUM_LEVELS);
    fill_mobs3(&s->melee_mobs, ml, 0, out);
    fill_mobs3(&s->passive_mobs, ml, 3, out);
    for (int i = 0; i < 2; i++) {
        out->mob_type_id[6 + i] = s->ranged_mobs.type_id[ml][i];
        out->mob_mask[6 + i] = s->ranged_mobs.mask[ml][i] ? 1 : 0;
        out->mob_position[6 + i][0] = s->ranged_mobs.position[ml][i][0];
        out->mob_position[6 + i][1] = s->ranged_mobs.position[ml][i][1];
    }
    fill_mobs3(&s->mob_projectiles, ml, 8, out);
    fill_mobs3(&s->player_projectiles, ml, 11, out);
    if (planes) {
        const int lv = s->player_level;
        memcpy(planes, s->map[lv], CRAFTAX_WG_MAP_CELLS);
        memcpy(planes + CRAFTAX_WG_MAP_CELLS, s->item_map[lv], CRAFTAX_WG_MAP_CELLS);
        memcpy(planes + 2 * CRAFTAX_WG_MAP_CELLS, s->light_map[lv], CRAFTAX_WG_MAP_CELLS);
    }
}

/* The reference's own encoder on env's current state. */
void cfref_encode(int env, uint8_t* rec_out) {
    craftax_encode_compact_observation(
        (const CraftaxWorldState*)(const void*)g_vec.envs[env].state, rec_out);
}

static uint32_t fz_next(uint32_t* s) { return cf_xorshift32(s); }
static int fz_range(uint32_t* s, int lo, int hi) { /* inclusive */
    return lo + (int)(fz_next(s) % (uint32_t)(hi - lo + 1));
}

static void fuzz_mobs(uint32_t* r, int32_t (*pos)[2], bool* mask, int32_t* type,
                      int count, int pr, int pc) {
    for (int i = 0; i < count; i++) {
        /* mostly near the player so the 9x11 window and its edges are hit,
         * sometimes far away or off the map */
        if (fz_next(r) % 4) {
            pos[i][0] = pr + fz_range(r, -6, 6);
            pos[i][1] = pc + fz_range(r, -7, 7);
        } else {
            pos[i][0] = fz_range(r, -3, 50);
            pos[i][1] = fz_range(r, -3, 50);
        }
        mask[i] = (fz_next(r) % 4) != 0;
        type[i] = fz_range(r, -1, 9); /* includes the rejected ids -1, 8, 9 */
    }
}

/* Overwrite the encoder-visible part of env's state with seeded adversarial
 * values (edges of the map, light values around the > 12 threshold, mobs on
 * and off the window, several mobs of one class on one cell, all inventory
 * magnitudes 0..99). */
void cfref_fuzz_state(int env, uint64_t seed) {
    CraftaxWorldState* s = (CraftaxWorldState*)(void*)g_vec.envs[env].state;
    uint32_t r = (uint32_t)(seed * 2654435761u) | 1u;
    for (int i = 0; i < 8; i++) fz_next(&r);
    const int lv = fz_range(&r, 0, 8);
    s->player_level = lv;
    const int edge = fz_next(&r) % 3;
    s->player_position[0] = edge == 0 ? fz_range(&r, 0, 5) : edge == 1 ? fz_range(&r, 42, 47) : fz_range(&r, 0, 47);
    s->player_position[1] = edge == 0 ? fz_range(&r, 0, 6) : edge == 1 ? fz_range(&r, 41, 47) : fz_range(&r, 0, 47);
    s->player_direction = fz_range(&r, 1, 4);
    s->player_health = (float)fz_range(&r, 0, 180) * 0.05f;
    s->player_food = fz_range(&r, 0, 20);
    s->player_drink = fz_range(&r, 0, 20);
    s->player_energy = fz_range(&r, 0, 20);
    s->player_mana = fz_range(&r, 0, 20);
    s->player_xp = fz_range(&r, 0, 12);
    s->player_dexterity = fz_range(&r, 1, 5);
    s->player_strength = fz_range(&r, 1, 5);
    s->player_intelligence = fz_range(&r, 1, 5);
    s->is_sleeping = fz_next(&r) & 1;
    s->is_resting = fz_next(&r) & 1;
    int32_t* inv[] = {&s->inventory.wood, &s->inventory.stone, &s->inventory.coal,
                      &s->inventory.iron, &s->inventory.diamond, &s->inventory.sapphire,
                      &s->inventory.ruby, &s->inventory.sapling, &s->inventory.torches,
                      &s->inventory.arrows};
    for (int i = 0; i < 10; i++) *inv[i] = fz_range(&r, 0, 99);
    s->inventory.books = fz_range(&r, 0, 2);
    s->inventory.pickaxe = fz_range(&r, 0, 4);
    s->inventory.sword = fz_range(&r, 0, 4);
    s->inventory.bow = fz_range(&r, 0, 1);
    for (int i = 0; i < 6; i++) s->inventory.potions[i] = fz_range(&r, 0, 99);
    for (int i = 0; i < 4; i++) s->inventory.armour[i] = fz_range(&r, 0, 2);
    for (int i = 0; i < 4; i++) s->armour_enchantments[i] = fz_range(&r, 0, 2);
    s->sword_enchantment = fz_range(&r, 0, 2);
    s->bow_enchantment = fz_range(&r, 0, 2);
    s->light_level = (float)fz_range(&r, 0, 1000) * 0.001f;
    s->learned_spells[0] = fz_next(&r) & 1;
    s->learned_spells[1] = fz_next(&r) & 1;
    s->monsters_killed[lv] = fz_range(&r, 0, 12);
    s->boss_timesteps_to_spawn_this_round = fz_range(&r, -2, 3);
    /* random cells in the neighbourhood that the window and nearby mobs can
     * touch; the rest of the plane is zero (dark), which keeps the committed
     * fixtures small */
    memset(s->map[lv], 0, CRAFTAX_WG_MAP_CELLS);
    memset(s->item_map[lv], 0, CRAFTAX_WG_MAP_CELLS);
    memset(s->light_map[lv], 0, CRAFTAX_WG_MAP_CELLS);
    for (int row = s->player_position[0] - 8; row <= s->player_position[0] + 8; row++)
        for (int col = s->player_position[1] - 9; col <= s->player_position[1] + 9; col++) {
            if (row < 0 || row >= CRAFTAX_WG_MAP_SIZE || col < 0 || col >= CRAFTAX_WG_MAP_SIZE)
                continue;
            s->map[lv][row][col] = (uint8_t)fz_range(&r, 0, 36);
            s->item_map[lv][row][col] = (uint8_t)fz_range(&r, 0, 4);
            const uint32_t k = fz_next(&r) % 8;
            s->light_map[lv][row][col] =
                k < 3 ? (uint8_t)fz_range(&r, 10, 15) : (uint8_t)fz_range(&r, 0, 255);
        }
    const int pr = s->player_position[0], pc = s->player_position[1];
    fuzz_mobs(&r, s->melee_mobs.position[lv], s->melee_mobs.mask[lv], s->melee_mobs.type_id[lv], 3, pr, pc);
    fuzz_mobs(&r, s->passive_mobs.position[lv], s->passive_mobs.mask[lv], s->passive_mobs.type_id[lv], 3, pr, pc);
    fuzz_mobs(&r, s->ranged_mobs.position[lv], s->ranged_mobs.mask[lv], s->ranged_mobs.type_id[lv], 2, pr, pc);
    fuzz_mobs(&r, s->mob_projectiles.position[lv], s->mob_projectiles.mask[lv], s->mob_projectiles.type_id[lv], 3, pr, pc);
    fuzz_mobs(&r, s->player_projectiles.position[lv], s->player_projectiles.mask[lv], s->player_projectiles.type_id[lv], 3, pr, pc);
    if (fz_next(&r) % 3 == 0) { /* two melee mobs on one cell: last slot wins */
        s->melee_mobs.position[lv][2][0] = s->melee_mobs.position[lv][0][0];
        s->melee_mobs.position[lv][2][1] = s->melee_mobs.position[lv][0][1];
        s->melee_mobs.mask[lv][0] = s->melee_mobs.mask[lv][2] = true;
    }
    if (fz_next(&r) % 4 == 0) { /* boss-vulnerable: no melee / ranged alive */
        for (int i = 0; i < 3; i++) s->melee_mobs.mask[lv][i] = false;
        for (int i = 0; i < 2; i++) s->ranged_mobs.mask[lv][i] = false;
    }
}

/* Scalar tail of the reference for an inventory filled with `value`
 * (brute-force pin of the sqrtf(x)/10 arithmetic). */
void cfref_tail_probe(int value, float health, float* tail_out) {
    static CraftaxWorldState st;
    memset(&st, 0, sizeof(st));
    st.inventory.wood = st.inventory.stone = st.inventory.coal = value;
    st.inventory.iron = st.inventory.diamond = st.inventory.sapphire = value;
    st.inventory.ruby = st.inventory.sapling = st.inventory.torches = value;
    st.inventory.arrows = value;
    for (int i = 0; i < 6; i++) st.inventory.potions[i] = value;
    st.player_health = health;
    st.player_food = st.player_drink = st.player_energy = st.player_mana = value;
    st.player_xp = st.player_dexterity = st.player_strength = value;
    st.player_intelligence = value;
    st.player_direction = 1;
    craftax_encode_scalar_observation_tail_at(&st, tail_out, 0);
}

/* `craftax_full bench` timing loop (craftax_full.c:8392-8438): env steps per
 * second of the reference CPU env with random actions. */
double cfref_bench(int num_envs, int iters, int threads, uint64_t seed) {
    if (threads > 0) omp_set_num_threads(threads);
    CfVec v;
    cf_vec_init(&v, num_envs, seed, /*parallel=*/1);
    for (int k = 0; k < 5; k++) {
#pragma omp parallel for schedule(static)
        for (int i = 0; i < num_envs; i++) {
            v.actions[i] = (float)(cf_xorshift32(&v.action_rng[i]) % CRAFTAX_NUM_ACTIONS);
            c_step(&v.envs[i]);
        }
    }
    double t0 = cf_now_s();
    for (int k = 0; k < iters; k++) {
#pragma omp parallel for schedule(static)
        for (int i = 0; i < num_envs; i++) {
            v.actions[i] = (float)(cf_xorshift32(&v.action_rng[i]) % CRAFTAX_NUM_ACTIONS);
            c_step(&v.envs[i]);
        }
    }
    double dt = cf_now_s() - t0;
    cf_vec_free(&v);
    return (double)num_envs * (double)iters / dt;
}

/* ---- env step: whole states in the library's exchange format --------------- */
static void export_mobs3(const CraftaxMobs3* m, int cls, cfp_env_state* o) {
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++)
        for (int i = 0; i < 3; i++) {
            o->mob_position[cls][l][i][0] = m->position[l][i][0];
            o->mob_position[cls][l][i][1] = m->position[l][i][1];
            o->mob_health[cls][l][i] = m->health[l][i];
            o->mob_mask[cls][l][i] = m->mask[l][i] ? 1 : 0;
            o->mob_attack_cooldown[cls][l][i] = m->attack_cooldown[l][i];
            o->mob_type_id[cls][l][i] = m->type_id[l][i];
        }
}
static void import_mobs3(CraftaxMobs3* m, int cls, const cfp_env_state* o) {
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++)
        for (int i = 0; i < 3; i++) {
            m->position[l][i][0] = o->mob_position[cls][l][i][0];
            m->position[l][i][1] = o->mob_position[cls][l][i][1];
            m->health[l][i] = o->mob_health[cls][l][i];
            m->mask[l][i] = o->mob_mask[cls][l][i] != 0;
            m->attack_cooldown[l][i] = o->mob_attack_cooldown[cls][l][i];
            m->type_id[l][i] = o->mob_type_id[cls][l][i];
        }
}

static void state_to_exchange(const CraftaxState* s, const Craftax* env, cfp_env_state* o) {
    memset(o, 0, sizeof(*o));
    o->player_position[0] = s->player_position[0];
    o->player_position[1] = s->player_position[1];
    o->player_level = s->player_level;
    o->player_direction = s->player_direction;
    o->player_health = s->player_health;
    o->player_food = s->player_food;
    o->player_drink = s->player_drink;
    o->player_energy = s->player_energy;
    o->player_mana = s->player_mana;
    o->is_sleeping = s->is_sleeping ? 1 : 0;
    o->is_resting = s->is_resting ? 1 : 0;
    o->player_recover = s->player_recover;
    o->player_hunger = s->player_hunger;
    o->player_thirst = s->player_thirst;
    o->player_fatigue = s->player_fatigue;
    o->player_recover_mana = s->player_recover_mana;
    o->player_xp = s->player_xp;
    o->player_dexterity = s->player_dexterity;
    o->player_strength = s->player_strength;
    o->player_intelligence = s->player_intelligence;
    o->wood = s->inventory.wood;
    o->stone = s->inventory.stone;
    o->coal = s->inventory.coal;
    o->iron = s->inventory.iron;
    o->diamond = s->inventory.diamond;
    o->sapling = s->inventory.sapling;
    o->pickaxe = s->inventory.pickaxe;
    o->sword = s->inventory.sword;
    o->bow = s->inventory.bow;
    o->arrows = s->inventory.arrows;
    for (int i = 0; i < 4; i++) o->armour[i] = s->inventory.armour[i];
    o->torches = s->inventory.torches;
    o->ruby = s->inventory.ruby;
    o->sapphire = s->inventory.sapphire;
    for (int i = 0; i < 6; i++) o->potions[i] = s->inventory.potions[i];
    o->books = s->inventory.books;
    export_mobs3(&s->melee_mobs, 0, o);
    export_mobs3(&s->passive_mobs, 1, o);
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++)
        for (int i = 0; i < 2; i++) {
            o->mob_position[2][l][i][0] = s->ranged_mobs.position[l][i][0];
            o->mob_position[2][l][i][1] = s->ranged_mobs.position[l][i][1];
            o->mob_health[2][l][i] = s->ranged_mobs.health[l][i];
            o->mob_mask[2][l][i] = s->ranged_mobs.mask[l][i] ? 1 : 0;
            o->mob_attack_cooldown[2][l][i] = s->ranged_mobs.attack_cooldown[l][i];
            o->mob_type_id[2][l][i] = s->ranged_mobs.type_id[l][i];
        }
    export_mobs3(&s->mob_projectiles, 3, o);
    export_mobs3(&s->player_projectiles, 4, o);
    memcpy(o->mob_projectile_directions, s->mob_projectile_directions, sizeof(o->mob_projectile_directions));
    memcpy(o->player_projectile_directions, s->player_projectile_directions, sizeof(o->player_projectile_directions));
    memcpy(o->growing_plants_positions, s->growing_plants_positions, sizeof(o->growing_plants_positions));
    memcpy(o->growing_plants_age, s->growing_plants_age, sizeof(o->growing_plants_age));
    for (int i = 0; i < CRAFTAX_MAX_GROWING_PLANTS; i++) o->growing_plants_mask[i] = s->growing_plants_mask[i] ? 1 : 0;
    memcpy(o->potion_mapping, s->potion_mapping, sizeof(o->potion_mapping));
    o->learned_spells[0] = s->learned_spells[0] ? 1 : 0;
    o->learned_spells[1] = s->learned_spells[1] ? 1 : 0;
    o->sword_enchantment = s->sword_enchantment;
    o->bow_enchantment = s->bow_enchantment;
    for (int i = 0; i < 4; i++) o->armour_enchantments[i] = s->armour_enchantments[i];
    o->boss_progress = s->boss_progress;
    o->boss_timesteps_to_spawn_this_round = s->boss_timesteps_to_spawn_this_round;
    o->light_level = s->light_level;
    o->state_rng[0] = s->state_rng[0];
    o->state_rng[1] = s->state_rng[1];
    o->timestep = s->timestep;
    memcpy(o->down_ladders, s->down_ladders, sizeof(o->down_ladders));
    memcpy(o->up_ladders, s->up_ladders, sizeof(o->up_ladders));
    memcpy(o->monsters_killed, s->monsters_killed, sizeof(o->monsters_killed));
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++) o->chests_opened[l] = s->chests_opened[l] ? 1 : 0;
    o->rng_key[0] = env->rng_key.word[0];
    o->rng_key[1] = env->rng_key.word[1];
    for (int a = 0; a < CRAFTAX_NUM_ACHIEVEMENTS; a++) o->achievements[a] = s->achievements[a] ? 1 : 0;
    memcpy(o->mob_bits, s->mob_bits, sizeof(o->mob_bits));
    memcpy(o->spawn_all_bits, s->spawn_all_bits, sizeof(o->spawn_all_bits));
    memcpy(o->spawn_grave_bits, s->spawn_grave_bits, sizeof(o->spawn_grave_bits));
    memcpy(o->spawn_water_bits, s->spawn_water_bits, sizeof(o->spawn_water_bits));
    memcpy(o->map, s->map, sizeof(o->map));
    memcpy(o->item_map, s->item_map, sizeof(o->item_map));
    memcpy(o->light_map, s->light_map, sizeof(o->light_map));
}

static void exchange_to_state(const cfp_env_state* o, CraftaxState* s, Craftax* env) {
    s->player_position[0] = o->player_position[0];
    s->player_position[1] = o->player_position[1];
    s->player_level = o->player_level;
    s->player_direction = o->player_direction;
    s->player_health = o->player_health;
    s->player_food = o->player_food;
    s->player_drink = o->player_drink;
    s->player_energy = o->player_energy;
    s->player_mana = o->player_mana;
    s->is_sleeping = o->is_sleeping != 0;
    s->is_resting = o->is_resting != 0;
    s->player_recover = o->player_recover;
    s->player_hunger = o->player_hunger;
    s->player_thirst = o->player_thirst;
    s->player_fatigue = o->player_fatigue;
    s->player_recover_mana = o->player_recover_mana;
    s->player_xp = o->player_xp;
    s->player_dexterity = o->player_dexterity;
    s->player_strength = o->player_strength;
    s->player_intelligence = o->player_intelligence;
    s->inventory.wood = o->wood;
    s->inventory.stone = o->stone;
    s->inventory.coal = o->coal;
    s->inventory.iron = o->iron;
    s->inventory.diamond = o->diamond;
    s->inventory.sapling = o->sapling;
    s->inventory.pickaxe = o->pickaxe;
    s->inventory.sword = o->sword;
    s->inventory.bow = o->bow;
    s->inventory.arrows = o->arrows;
    for (int i = 0; i < 4; i++) s->inventory.armour[i] = o->armour[i];
    s->inventory.torches = o->torches;
    s->inventory.ruby = o->ruby;
    s->inventory.sapphire = o->sapphire;
    for (int i = 0; i < 6; i++) s->inventory.potions[i] = o->potions[i];
    s->inventory.books = o->books;
    import_mobs3(&s->melee_mobs, 0, o);
    import_mobs3(&s->passive_mobs, 1, o);
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++)
        for (int i = 0; i < 2; i++) {
            s->ranged_mobs.position[l][i][0] = o->mob_position[2][l][i][0];
            s->ranged_mobs.position[l][i][1] = o->mob_position[2][l][i][1];
            s->ranged_mobs.health[l][i] = o->mob_health[2][l][i];
            s->ranged_mobs.mask[l][i] = o->mob_mask[2][l][i] != 0;
            s->ranged_mobs.attack_cooldown[l][i] = o->mob_attack_cooldown[2][l][i];
            s->ranged_mobs.type_id[l][i] = o->mob_type_id[2][l][i];
        }
    import_mobs3(&s->mob_projectiles, 3, o);
    import_mobs3(&s->player_projectiles, 4, o);
    memcpy(s->mob_projectile_directions, o->mob_projectile_directions, sizeof(o->mob_projectile_directions));
    memcpy(s->player_projectile_directions, o->player_projectile_directions, sizeof(o->player_projectile_directions));
    memcpy(s->growing_plants_positions, o->growing_plants_positions, sizeof(o->growing_plants_positions));
    memcpy(s->growing_plants_age, o->growing_plants_age, sizeof(o->growing_plants_age));
    for (int i = 0; i < CRAFTAX_MAX_GROWING_PLANTS; i++) s->growing_plants_mask[i] = o->growing_plants_mask[i] != 0;
    memcpy(s->potion_mapping, o->potion_mapping, sizeof(o->potion_mapping));
    s->learned_spells[0] = o->learned_spells[0] != 0;
    s->learned_spells[1] = o->learned_spells[1] != 0;
    s->sword_enchantment = o->sword_enchantment;
    s->bow_enchantment = o->bow_enchantment;
    for (int i = 0; i < 4; i++) s->armour_enchantments[i] = o->armour_enchantments[i];
    s->boss_progress = o->boss_progress;
    s->boss_timesteps_to_spawn_this_round = o->boss_timesteps_to_spawn_this_round;
    s->light_level = o->light_level;
    s->state_rng[0] = o->state_rng[0];
    s->state_rng[1] = o->state_rng[1];
    s->timestep = o->timestep;
    memcpy(s->down_ladders, o->down_ladders, sizeof(o->down_ladders));
    memcpy(s->up_ladders, o->up_ladders, sizeof(o->up_ladders));
    memcpy(s->monsters_killed, o->monsters_killed, sizeof(o->monsters_killed));
    for (int l = 0; l < CRAFTAX_NUM_LEVELS; l++) s->chests_opened[l] = o->chests_opened[l] != 0;
    env->rng_key.word[0] = o->rng_key[0];
    env->rng_key.word[1] = o->rng_key[1];
    for (int a = 0; a < CRAFTAX_NUM_ACHIEVEMENTS; a++) s->achievements[a] = o->achievements[a] != 0;
    memcpy(s->mob_bits, o->mob_bits, sizeof(o->mob_bits));
    memcpy(s->map, o->map, sizeof(o->map));
    memcpy(s->item_map, o->item_map, sizeof(o->item_map));
    memcpy(s->light_map, o->light_map, sizeof(o->light_map));
    s->lazy_floors_pending = 0;
    craftax_refresh_spawn_bits_all(s);
}

size_t cfref_exchange_bytes(void) { return sizeof(cfp_env_state); }
void cfref_export_state(int env, cfp_env_state* out) {
    state_to_exchange(g_vec.envs[env].state, &g_vec.envs[env], out);
}
void cfref_import_state(int env, const cfp_env_state* in) {
    exchange_to_state(in, g_vec.envs[env].state, &g_vec.envs[env]);
}

/* The next action of env's xorshift32 % 43 stream (cf_run_hash, craftax_full.c:8349-8353). */
float cfref_next_action(int env) {
    return (float)(cf_xorshift32(&g_vec.action_rng[env]) % CRAFTAX_NUM_ACTIONS);
}

/* c_step_gameplay (craftax_full.c:3981-4011) for one env with the given action, its own
 * statements in its own order, plus one thing: the state the step ended in is handed out
 * before the reset that follows a terminal step replaces it.  Returns the terminal
 * flag; reward and reset key go to the out arguments. */
int cfref_step_env(int i, float action_f, cfp_env_state* final_state, float* reward_out,
                   uint32_t* reset_key_out) {
    Craftax* env = &g_vec.envs[i];
    env->actions[0] = action_f;
    env->rewards[0] = 0.0f;
    env->terminals[0] = 0.0f;
    int action = (int)env->actions[0];
    if (action < 0) action = CRAFTAX_ACTION_NOOP;
    if (action >= CRAFTAX_NUM_ACTIONS) action = CRAFTAX_NUM_ACTIONS - 1;
    CraftaxThreefryKey step_key, step_rng, reset_key;
    craftax_threefry_split(env->rng_key, &env->rng_key, &step_key);
    craftax_threefry_split(step_key, &step_rng, &reset_key);
    float reward = craftax_gameplay_step_native(env->state, action, step_rng);
    bool done = craftax_is_game_over_native(env->state);
    craftax_copy_achievements_to_env(env, env->state);
    env->rewards[0] = reward;
    env->terminals[0] = done ? 1.0f : 0.0f;
    env->episode_return_accum += reward;
    env->episode_length_accum += 1;
    if (final_state) state_to_exchange(env->state, env, final_state);
    if (done) {
        add_log(env);
        env->episode_return_accum = 0.0f;
        env->episode_length_accum = 0;
        memset(env->achievements, 0, sizeof(env->achievements));
        craftax_reset_state_on_done(env->state, reset_key);
    }
    *reward_out = reward;
    reset_key_out[0] = reset_key.word[0];
    reset_key_out[1] = reset_key.word[1];
    c_step_encode(env);
    return done ? 1 : 0;
}

float cfref_light_level(int timestep) { return craftax_calculate_light_level_native(timestep); }
