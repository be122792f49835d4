/*
 * Compiled-reference checker.  TEST INFRASTRUCTURE ONLY.
 *
 * This translation unit #includes the reference's craftax_full.c from where it
 * lies (path given by -DCF_REF_SRC on the command line, see Makefile; nothing
 * of it is copied into this repository) with -DCRAFTAX_COMPACT_OBS, and wraps
 * its own functions -- cf_vec_init, c_step, the xorshift32 % 43 action stream
 * of cf_run_hash (craftax_full.c:8349-8353) and
 * craftax_encode_compact_observation (:2830) -- behind a small C interface
 * that the tests drive through ctypes.  Output: oracle/_ref/libcfref.so.
 */
#define main cf_ref_main
#include CF_REF_SRC
#undef main

#include "../include/cfp.h"

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
