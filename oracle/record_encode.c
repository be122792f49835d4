/*
 * CPU restatement of the reference's compact observation encoder.
 * TEST INFRASTRUCTURE ONLY (see cfo.h).  Must be compiled WITHOUT -ffast-math:
 * the reference binary is built with it, which turns its `/ 10.0f` into a
 * multiply by the rounded reciprocal; that product is spelled out here.
 *
 * Follows craftax_full.c:
 *   map cells        craftax_encode_compact_map_base_observation  :2721-2745
 *   mob scatter      craftax_encode_mobs3_compact / mobs2_compact :2747-2825
 *   order of classes craftax_encode_compact_observation           :2830-2844
 *   scalar tail      craftax_encode_scalar_observation_tail_at    :2646-2703
 *   level clamp      craftax_wg_jax_index                         :2180-2191
 *   boss flag        craftax_wg_is_boss_vulnerable                :2205-2220
 */
#include <math.h>
#include <string.h>

#include "cfo.h"

enum { MAPSZ = 48, ROWS = 9, COLS = 11, CH = 8, MAPB = 792, TAILN = 51 };

static int jax_index(int index, int size) {
    if (index < 0) index += size;
    if (index < 0) return 0;
    if (index >= size) return size - 1;
    return index;
}

/* class channel (3 + class) of each of the 14 mob slots, in the order the
 * reference walks them: melee x3, passive x3, ranged x2, mob projectiles x3,
 * player projectiles x3. */
static const int kSlotClass[CFP_MOB_SLOTS] = {0, 0, 0, 1, 1, 1, 2, 2, 3, 3, 3, 4, 4, 4};

static void encode_tail(const cfp_env_scalars* s, float* t) {
    const float tenth = 1.0f / 10.0f;
    int i = 0;
    t[i++] = sqrtf((float)s->wood) * tenth;
    t[i++] = sqrtf((float)s->stone) * tenth;
    t[i++] = sqrtf((float)s->coal) * tenth;
    t[i++] = sqrtf((float)s->iron) * tenth;
    t[i++] = sqrtf((float)s->diamond) * tenth;
    t[i++] = sqrtf((float)s->sapphire) * tenth;
    t[i++] = sqrtf((float)s->ruby) * tenth;
    t[i++] = sqrtf((float)s->sapling) * tenth;
    t[i++] = sqrtf((float)s->torches) * tenth;
    t[i++] = sqrtf((float)s->arrows) * tenth;
    t[i++] = (float)s->books * 0.5f;
    t[i++] = (float)s->pickaxe * 0.25f;
    t[i++] = (float)s->sword * 0.25f;
    t[i++] = (float)s->sword_enchantment;
    t[i++] = (float)s->bow_enchantment;
    t[i++] = (float)s->bow;
    for (int k = 0; k < 6; k++) t[i++] = sqrtf((float)s->potions[k]) * tenth;
    t[i++] = s->player_health * tenth;
    t[i++] = (float)s->player_food * tenth;
    t[i++] = (float)s->player_drink * tenth;
    t[i++] = (float)s->player_energy * tenth;
    t[i++] = (float)s->player_mana * tenth;
    t[i++] = (float)s->player_xp * tenth;
    t[i++] = (float)s->player_dexterity * tenth;
    t[i++] = (float)s->player_strength * tenth;
    t[i++] = (float)s->player_intelligence * tenth;
    for (int k = 0; k < 4; k++) t[i++] = (k == s->player_direction - 1) ? 1.0f : 0.0f;
    for (int k = 0; k < 4; k++) t[i++] = (float)s->armour[k] * 0.5f;
    for (int k = 0; k < 4; k++) t[i++] = (float)s->armour_enchantments[k];
    t[i++] = s->light_level;
    t[i++] = s->is_sleeping ? 1.0f : 0.0f;
    t[i++] = s->is_resting ? 1.0f : 0.0f;
    t[i++] = s->learned_spells[0] ? 1.0f : 0.0f;
    t[i++] = s->learned_spells[1] ? 1.0f : 0.0f;
    t[i++] = (float)s->player_level * tenth;
    t[i++] = s->monsters_killed_level >= 8 ? 1.0f : 0.0f;
    int live = 0;
    for (int m = 0; m < 3; m++) live |= s->mob_mask[m] != 0;  /* melee  */
    for (int m = 6; m < 8; m++) live |= s->mob_mask[m] != 0;  /* ranged */
    t[i++] = (!live && s->boss_timesteps_to_spawn_this_round <= 0) ? 1.0f : 0.0f;
}

void cfo_encode_compact(const cfp_env_scalars* s, const uint8_t* map,
                        const uint8_t* item_map, const uint8_t* light_map,
                        size_t level_stride, uint8_t* obs) {
    const int top = s->player_position[0] - ROWS / 2;
    const int left = s->player_position[1] - COLS / 2;
    const size_t cell_off = (size_t)s->player_level * level_stride; /* raw level */
    const size_t mob_off = (size_t)jax_index(s->player_level, 9) * level_stride;

    memset(obs, 0, MAPB);
    for (int row = 0; row < ROWS; row++) {
        const int wr = top + row;
        if (wr < 0 || wr >= MAPSZ) continue;
        for (int col = 0; col < COLS; col++) {
            const int wc = left + col;
            if (wc < 0 || wc >= MAPSZ) continue;
            const size_t o = cell_off + (size_t)(wr * MAPSZ + wc);
            if (light_map[o] > 12) {
                uint8_t* cell = obs + (row * COLS + col) * CH;
                cell[0] = map[o];
                cell[1] = (uint8_t)(item_map[o] + 1);
                cell[2] = 1;
            }
        }
    }
    for (int m = 0; m < CFP_MOB_SLOTS; m++) {
        const int type = s->mob_type_id[m];
        if (type < 0 || type >= 8 || !s->mob_mask[m]) continue;
        const int wr = s->mob_position[m][0], wc = s->mob_position[m][1];
        const int lr = wr - s->player_position[0] + ROWS / 2;
        const int lc = wc - s->player_position[1] + COLS / 2;
        if (lr < 0 || lr >= ROWS || lc < 0 || lc >= COLS) continue;
        if (wr < 0 || wr >= MAPSZ || wc < 0 || wc >= MAPSZ) continue;
        if (light_map[mob_off + (size_t)(wr * MAPSZ + wc)] <= 12) continue;
        obs[(lr * COLS + lc) * CH + 3 + kSlotClass[m]] = (uint8_t)(type + 1);
    }
    float tail[TAILN];
    encode_tail(s, tail);
    memcpy(obs + MAPB, tail, sizeof(tail));
}

void cfo_encode_compact_batch(int n, const cfp_env_scalars* s, const uint8_t* map,
                              const uint8_t* item_map, const uint8_t* light_map,
                              size_t env_stride, size_t level_stride, uint8_t* rec) {
    for (int e = 0; e < n; e++)
        cfo_encode_compact(s + e, map + (size_t)e * env_stride,
                           item_map + (size_t)e * env_stride,
                           light_map + (size_t)e * env_stride, level_stride,
                           rec + (size_t)e * CFP_REC_BYTES);
}

void cfo_expand_record(const uint8_t* rec, float* x) {
    for (int f = 0; f < MAPB; f++) x[f] = (float)rec[f];
    memcpy(x + MAPB, rec + MAPB, TAILN * sizeof(float));
}
