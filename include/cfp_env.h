/*
 * cfp_env.h -- C ABI of the MI355X (gfx950) batched Craftax env step: the env half
 * of the reference's rollout step (cu_rollout_step, craftax_full.cu:12022-12087;
 * cu_step_launch :10914-10946).  One cfp_env object stands for the reference's CuVec
 * (:10688-10712): it owns every device array of `n` envs, is filled from host states
 * (or from a pool of them on reset) and is stepped by one kernel launch.
 *
 * Conventions are those of cfp.h: device pointers are d_*, `stream` is a
 * hipStream_t passed as void*, 0 = success, cfp_last_error() holds the message.
 */
#ifndef CFP_ENV_H_
#define CFP_ENV_H_

#include <stddef.h>
#include <stdint.h>

#include "cfp.h"

#ifdef __cplusplus
extern "C" {
#endif

#define CFP_ENV_LEVELS 9                /* craftax_full.c:2945 */
#define CFP_ENV_MAP 48                  /* craftax_full.c:2944 */
#define CFP_ENV_ACHIEVEMENTS 67         /* craftax_full.c:2965 */
#define CFP_ENV_PLANTS 10               /* craftax_full.c:2972 */
#define CFP_ENV_MOB_CLASSES 5           /* melee, passive, ranged, mob proj., player proj. */
#define CFP_ENV_MAX_TIMESTEPS 100000    /* craftax_full.c:2974 */

/* One env's complete state in host memory: every member of the reference's
 * CraftaxState (craftax_full.c:3203-3278) that the step reads or writes, under the
 * reference's names, plus the env's own key Craftax.rng_key (:3473).  The five mob
 * pools are one array indexed [class][level][slot] in the order melee, passive,
 * ranged (slot 2 unused), mob projectiles, player projectiles.  The three
 * spawn_*_bits planes are functions of `map` (:3305-3355): import ignores them and
 * derives them, export fills them.  This is the exchange format of
 * cfp_env_import / cfp_env_export; the device layout is per-field arrays
 * (cfp_env_view). */
typedef struct cfp_env_state {
    int32_t player_position[2];
    int32_t player_level;
    int32_t player_direction;
    float player_health;
    int32_t player_food, player_drink, player_energy, player_mana;
    int32_t is_sleeping, is_resting;
    float player_recover, player_hunger, player_thirst, player_fatigue, player_recover_mana;
    int32_t player_xp, player_dexterity, player_strength, player_intelligence;
    int32_t wood, stone, coal, iron, diamond, sapling, pickaxe, sword, bow, arrows;
    int32_t armour[4];
    int32_t torches, ruby, sapphire;
    int32_t potions[6];
    int32_t books;
    int32_t mob_position[CFP_ENV_MOB_CLASSES][CFP_ENV_LEVELS][3][2];
    float mob_health[CFP_ENV_MOB_CLASSES][CFP_ENV_LEVELS][3];
    int32_t mob_attack_cooldown[CFP_ENV_MOB_CLASSES][CFP_ENV_LEVELS][3];
    int32_t mob_type_id[CFP_ENV_MOB_CLASSES][CFP_ENV_LEVELS][3];
    int32_t mob_mask[CFP_ENV_MOB_CLASSES][CFP_ENV_LEVELS][3];
    int32_t mob_projectile_directions[CFP_ENV_LEVELS][3][2];
    int32_t player_projectile_directions[CFP_ENV_LEVELS][3][2];
    int32_t growing_plants_positions[CFP_ENV_PLANTS][2];
    int32_t growing_plants_age[CFP_ENV_PLANTS];
    int32_t growing_plants_mask[CFP_ENV_PLANTS];
    int32_t potion_mapping[6];
    int32_t learned_spells[2];
    int32_t sword_enchantment, bow_enchantment;
    int32_t armour_enchantments[4];
    int32_t boss_progress, boss_timesteps_to_spawn_this_round;
    float light_level;
    uint32_t state_rng[2];
    int32_t timestep;
    int32_t down_ladders[CFP_ENV_LEVELS][2];
    int32_t up_ladders[CFP_ENV_LEVELS][2];
    int32_t monsters_killed[CFP_ENV_LEVELS];
    int32_t chests_opened[CFP_ENV_LEVELS];
    uint32_t rng_key[2];
    uint8_t achievements[CFP_ENV_ACHIEVEMENTS];
    uint8_t pad_[5];
    /* bit c of row r of a level: a live melee, passive or ranged mob stands on (r, c).  The step
     * keeps the rows it touches equal to what the mob slots say and asks the slots, not these
     * rows, whether a cell is taken: an imported state has to hold the two in agreement, as
     * every state the game produces does (mob positions within the 48 x 48 map). */
    uint64_t mob_bits[CFP_ENV_LEVELS][CFP_ENV_MAP];
    uint64_t spawn_all_bits[CFP_ENV_LEVELS][CFP_ENV_MAP];
    uint64_t spawn_grave_bits[CFP_ENV_LEVELS][CFP_ENV_MAP];
    uint64_t spawn_water_bits[CFP_ENV_LEVELS][CFP_ENV_MAP];
    uint8_t map[CFP_ENV_LEVELS][CFP_ENV_MAP][CFP_ENV_MAP];
    uint8_t item_map[CFP_ENV_LEVELS][CFP_ENV_MAP][CFP_ENV_MAP];
    uint8_t light_map[CFP_ENV_LEVELS][CFP_ENV_MAP][CFP_ENV_MAP];
} cfp_env_state;

size_t cfp_env_state_bytes(void);

/* CraftaxResetRec (craftax_full.cu:8707-8711): an env that finished this step and
 * the key its new world is to be generated from (craftax_full.c:3993, 4009). */
typedef struct cfp_env_reset_rec {
    int32_t env;
    uint32_t key0;
    uint32_t key1;
} cfp_env_reset_rec;

typedef struct cfp_env cfp_env;

/* cu_vec_init without its worldgen (craftax_full.cu:10732-10880): allocates the device
 * arrays of `n` envs (a multiple of 32, as the reference asks of --envs) and of `pool` reset states (0 = none), zeroed,
 * and uploads the light-level table.  No env is playable before cfp_env_import. */
int cfp_env_create(cfp_env** out, int n, int pool);
void cfp_env_destroy(cfp_env* e);
int cfp_env_num_envs(const cfp_env* e);
int cfp_env_pool_size(const cfp_env* e);

/* k_env_init (craftax_full.cu:8669-8699; c_init, craftax_full.c:3883-3893): env i becomes the
 * env created from seed + i -- its key, the nine floors of its first world generated on the
 * device (all floors at once, as the reference's C build does; craftax_full.c:2050-2142) --
 * and its action stream is seeded as cfp_env_seed_actions does. */
int cfp_env_init(cfp_env* e, uint64_t seed, void* stream);
/* k_reset_list_block (craftax_full.cu:8957-8975; craftax_reset_state_on_done,
 * craftax_full.c:3731-3744): every env on the reset list gets a new world generated on the
 * device from its record's key; its own key and action stream continue. */
int cfp_env_reset(cfp_env* e, void* stream);
/* The reset pool filled on the device: entry i = the state of an env created from seed + i
 * (craftax_set_reset_pool_size, craftax_full.c:3568-3581, uses seeds 0, 1, ...). */
int cfp_env_pool_fill(cfp_env* e, uint64_t seed, void* stream);
/* The same states generated on the host, for callers that keep worlds there. */
int cfp_env_generate_host(uint32_t seed, int count, cfp_env_state* states);

/* Host states -> device arrays of envs [first, first + count) and back.  Both
 * synchronise with the device.  Import derives the spawn bit planes from `map`. */
int cfp_env_import(cfp_env* e, int first, int count, const cfp_env_state* states);
int cfp_env_export(cfp_env* e, int first, int count, cfp_env_state* states);
/* The same for the reset pool's entries (craftax_set_reset_pool_size,
 * craftax_full.c:3568-3581: worlds generated once, copied in on reset). */
int cfp_env_pool_import(cfp_env* e, int first, int count, const cfp_env_state* states);

/* The env vector's own action / reward / terminal slots, float[n] each on the device
 * (CuVec.d_actions / d_rewards / d_terminals, craftax_full.cu:10693-10695), zeroed at
 * creation.  cfp_env_step accepts any buffers; these are the ones the collect loop uses. */
float* cfp_env_actions(const cfp_env* e);
float* cfp_env_rewards(const cfp_env* e);
float* cfp_env_terminals(const cfp_env* e);

/* calculate_light_level(timestep) for timestep 0..CFP_ENV_MAX_TIMESTEPS as the step uses
 * it (craftax_full.c:3760-3767 under the reference's build flags; the reference's GPU
 * port also computes this table on the host, craftax_full.cu:10714-10729).  Host only. */
int cfp_env_light_table(float* out, int count);

/* k_step (craftax_full.cu:8760-8779; c_step_gameplay, craftax_full.c:3981-4011, without
 * the reset): one game step for every env.  d_actions float[n] is the env action slot
 * the sampler writes (clamped to 0..42 as :3985-3987), or NULL: then each env draws
 * xorshift32 % 43 from its own action stream (:8349-8353, seeded by
 * cfp_env_seed_actions).  Writes d_rewards[n], d_terminals[n] (1.0f = episode over),
 * zeroes the done count first and appends every finished env to the reset list.  A
 * finished env keeps its final state until a reset call replaces it. */
int cfp_env_step(cfp_env* e, const float* d_actions, float* d_rewards, float* d_terminals,
                 void* stream);
/* action_rng[i] = (uint32)(seed ^ i * 2654435761) | 1 (craftax_full.c:8318). */
int cfp_env_seed_actions(cfp_env* e, uint64_t seed, void* stream);

/* The reset list of the last step: device count and records (d_resets of CuVec). */
const int* cfp_env_reset_count(const cfp_env* e);
const cfp_env_reset_rec* cfp_env_reset_list(const cfp_env* e);
/* Host copy of the list (synchronises `stream`): up to max records into out, the full
 * count into *count.  For callers that produce the new states on the host and hand them
 * to cfp_env_import. */
int cfp_env_fetch_resets(const cfp_env* e, cfp_env_reset_rec* out, int max, int* count, void* stream);
/* craftax_reset_state_on_done with a static pool (craftax_full.c:3738-3741): every env
 * on the reset list becomes a copy of pool entry key0 % pool. */
int cfp_env_reset_from_pool(cfp_env* e, void* stream);

/* View of the device arrays in the form cfp_record_obs_soa reads, with the three map
 * planes' base addresses and strides. */
int cfp_env_view(const cfp_env* e, cfp_env_soa* soa, const uint8_t** d_map,
                 const uint8_t** d_item_map, const uint8_t** d_light_map,
                 size_t* env_stride, size_t* level_stride);
/* k_record_obs on this env's state: n records into d_rec_row (cfp_record_obs_soa on
 * cfp_env_view). */
int cfp_env_record_obs(const cfp_env* e, uint8_t* d_rec_row, void* stream);

/* cu_rollout_step (craftax_full.cu:12022-12087) with the env on the device: record the
 * envs' observations into r_obs[t], run the policy half (cfp_rollout_step: forward on the
 * live state with the env's terminals as the state-zeroing flags, sample into r_act /
 * r_logprob / r_value and the env's action slots), step the envs, store rewards and
 * terminals into r_reward[t] / r_done[t], reset finished envs: from the pool when the env
 * object has one, with freshly generated worlds otherwise.  The trainer's env count must equal the env object's. */
int cfp_env_rollout_step(cfp_trainer* tr, cfp_env* e, int t, uint64_t seed, void* stream);
/* cu_rollout_step_plain (craftax_full.cu:12089-12092), the step of the reference's `run` mode
 * (cu_run_rollout_bench, :12127-12176): the same sequence with no slabs -- records into the
 * policy's own buffer, forward on its live state, the draw with offset *counter (then
 * *counter += 1), the env step with the drawn actions, finished envs replaced.  The sampled
 * actions (int32), log-probabilities and values of the step lie in the env object
 * (CuPolicy.d_act / d_logprob / d_value, :11770-11773), as does the 8-byte device step counter
 * of the draws, zero at cfp_env_create.  The policy's env count must equal the env object's. */
int cfp_env_run_step(cfp_policy* p, cfp_env* e, uint64_t seed, void* stream);
int32_t* cfp_env_run_actions(const cfp_env* e);
float* cfp_env_run_logprobs(const cfp_env* e);
float* cfp_env_run_values(const cfp_env* e);
uint64_t* cfp_env_run_counter(const cfp_env* e);
/* cu_train_collect (craftax_full.cu:12980-13016): T rollout steps as above, the bootstrap
 * value on a copy of the live state from the post-rollout observations, GAE and the
 * advantage statistics. */
int cfp_train_collect(cfp_trainer* tr, cfp_env* e, uint64_t seed, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CFP_ENV_H_ */
