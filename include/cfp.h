/*
 * cfp.h -- C ABI of the MI355X (gfx950) batched Craftax policy path.
 *
 * Every entry point replaces one static function of the reference's single
 * translation unit craftax_full.cu (cited as file:line at each declaration).
 * The reference exposes no FFI for this path, so the seam kept here is the
 * call surface of its rollout/trainer layers: same argument order, same
 * tensor layouts, same "all work is enqueued on the given stream, nothing is
 * allocated inside a step" contract: a policy or trainer object owns every buffer
 * its entry points touch (allocated by its create call); the raw GEMM entry points
 * of the dense-math seam share one process-wide workspace, see cfp_seam_reserve.
 *
 * Conventions
 *   - All pointers named d_* / documented "device" are HIP device pointers.
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream).
 *   - Activations are env-major: element (k, env) of a [rows]-wide tensor
 *     sits at env*rows + k (the reference calls this col-major [rows][cols]).
 *   - Return value: 0 on success, nonzero on error; cfp_last_error() returns
 *     a thread-local message.  A library must not exit(); the reference's
 *     CU_CHECK (craftax_full.cu:8635) prints and exit(1)s instead.
 *   - Env counts must be multiples of 32, as in the reference
 *     (craftax_full.cu:11820).
 */
#ifndef CFP_H_
#define CFP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fixed architecture (craftax_full.cu:9086-9105) ---------------------- */
#define CFP_HIDDEN 256
#define CFP_GRU (3 * CFP_HIDDEN)        /* [zh | zg | zp] rows per layer      */
#define CFP_OBS 843                     /* 792 map features + 51 tail floats  */
#define CFP_OBS_MAP 792
#define CFP_OBS_TAIL 51
#define CFP_REC_BYTES 996               /* compact record, craftax_full.c:578 */
#define CFP_ACTIONS 43
#define CFP_AV (CFP_ACTIONS + 1)        /* fused head: 43 logits + value      */
#define CFP_MAX_LAYERS 3

/* Flat fp32 parameter arena offsets for `layers` MinGRU layers
 * (craftax_full.cu:9094-9102). */
#define CFP_OFF_W_ENC 0
#define CFP_OFF_B_ENC (CFP_OBS * CFP_HIDDEN)
#define CFP_OFF_W_GRU (CFP_OFF_B_ENC + CFP_HIDDEN)
#define CFP_OFF_W_A(layers) (CFP_OFF_W_GRU + (layers) * CFP_GRU * CFP_HIDDEN)
#define CFP_OFF_B_A(layers) (CFP_OFF_W_A(layers) + CFP_ACTIONS * CFP_HIDDEN)
#define CFP_OFF_W_V(layers) (CFP_OFF_B_A(layers) + CFP_ACTIONS)
#define CFP_OFF_B_V(layers) (CFP_OFF_W_V(layers) + CFP_HIDDEN)
#define CFP_PARAM_COUNT(layers) (CFP_OFF_B_V(layers) + 1)

/* Classic-game policy (craftax_classic.cu:38-59, 1522-1533): 1345-dim one-hot
 * observation carried as a 148-byte record, actor 17 / value 1, same MinGRU stack.
 * Its params arena has the same segment order with 1345 / 17 in place of 843 / 43. */
#define CFP_CLASSIC_OBS 1345
#define CFP_CLASSIC_REC_BYTES 148
#define CFP_CLASSIC_ACTIONS 17
#define CFP_CLASSIC_AV (CFP_CLASSIC_ACTIONS + 1)
#define CFP_CLASSIC_PARAM_COUNT(layers)                                           \
    (CFP_CLASSIC_OBS * CFP_HIDDEN + CFP_HIDDEN + (layers) * CFP_GRU * CFP_HIDDEN + \
     CFP_CLASSIC_ACTIONS * CFP_HIDDEN + CFP_CLASSIC_ACTIONS + CFP_HIDDEN + 1)

const char* cfp_last_error(void);
/* Library/ABI version, bumped when a signature changes. */
int cfp_abi_version(void);

/* ---- policy object: replaces CuPolicy (craftax_full.cu:11758-11796) ------ */
typedef struct cfp_policy cfp_policy;

/* cu_policy_init (craftax_full.cu:11819): allocates every device buffer the
 * forward needs for `num_envs` envs (params, packed weight mirrors, live
 * state [layers][n][256] zeroed, record scratch, h_enc, h3, fused head
 * output), fills params from `seed` (Xavier-uniform; the reference draws
 * U(+-1/sqrt(fan_in)) from cuRAND Philox, which is not reproducible off CUDA)
 * and builds the MFMA-ordered weight mirrors.  layers in 1..3. */
int cfp_policy_create(cfp_policy** out, int num_envs, int layers, uint64_t seed);
/* Classic-game variant: the Rollout object of main_classic.cu:326.  Every
 * forward entry point below then takes 148-byte records (layout
 * craftax_classic.cu:50-59: 63 block ids, 63 mob bitmasks, 12 inventory, 4
 * intrinsics, direction, sleeping, light fp32) and writes av[n][18]
 * (17 logits + value); the encoder is the gathered-column sum of
 * encode_obs_kernel (craftax_classic.cu:1714-1751) instead of a GEMM. */
int cfp_policy_create_classic(cfp_policy** out, int num_envs, int layers, uint64_t seed);
/* 0 = full game (843 features, 43 actions), 1 = classic. */
int cfp_policy_variant(const cfp_policy* p);
/* cu_policy_free (craftax_full.cu:11907). */
void cfp_policy_destroy(cfp_policy* p);

int cfp_policy_num_envs(const cfp_policy* p);
int cfp_policy_layers(const cfp_policy* p);
size_t cfp_policy_param_count(const cfp_policy* p);

/* Host <-> device copies of the flat params arena (the payload of the
 * reference's CFW1 checkpoint, cu_save_weights/cu_load_weights
 * craftax_full.cu:12248/12264).  set_params also rebuilds the mirrors. */
int cfp_policy_set_params(cfp_policy* p, const float* host_params, size_t count);
int cfp_policy_get_params(const cfp_policy* p, float* host_params, size_t count);
/* The reference's own initialisation (cu_policy_init, craftax_full.cu:11830-11845 with
 * k_nn_init_weights :9123-9131; main_classic.cu:366-374 for the classic game): the seven
 * arena segments s = 0..6 (W_enc, b_enc, W_gru, W_a, b_a, W_v, b_v) filled with
 * (2u - 1) * bound, bound = 1/sqrt(obs) for the first two and 1/sqrt(256) for the
 * rest, u = the first curand_uniform of a Philox4_32_10 state after
 * curand_init(seed, s, i) (the reference passes seed 1234).  Replaces the
 * Xavier-uniform weights cfp_policy_create made and refreshes the mirrors.  The
 * Philox block function is checked against published vectors, the mapping of
 * (seed, subsequence, offset) onto it against rocRAND's engine, which takes the same
 * three arguments; the float is cuRAND's x * 2^-32 + 2^-33. */
int cfp_policy_init_reference(cfp_policy* p, uint64_t seed);
/* Rebuild the MFMA-ordered weight mirrors from the params arena after the
 * arena changed on device: the role of cu_params_refresh_bf16 + cu_pack_wav
 * (craftax_full.cu:11805-11817) after init / Adam. */
int cfp_policy_refresh_weights(cfp_policy* p, void* stream);

/* cu_save_weights / cu_load_weights (craftax_full.cu:12248, :12264): the "CFW1"
 * file -- uint32 {0x31574643, hidden = 256, layers, param count} then the fp32
 * params arena.  Loading checks the header against the policy (error, params
 * untouched, on mismatch or truncation) and refreshes the weight mirrors. */
int cfp_save_weights(const cfp_policy* p, const char* path);
int cfp_load_weights(cfp_policy* p, const char* path);

/* bf16-input / fp32-accumulate GEMMs for the forward entry points of this policy
 * (encoder, gate and head GEMMs on bf16 MFMA; state, epilogue and outputs stay
 * fp32).  Replaces the reference's process-wide CF_GEMM_BF16 switch
 * (craftax_full.cu:11306-11316, bf16 wrappers :11688-11756) by a per-object
 * flag; off by default.  Accuracy: 2e-2 relative to an fp64 evaluation. */
int cfp_policy_set_gemm_bf16(cfp_policy* p, int on);
int cfp_policy_gemm_bf16(const cfp_policy* p);

/* 16-env tiles for small batches (no counterpart in the reference, whose cuBLAS GEMMs
 * take any width): with the flag on, cfp_policy_forward (and the trainer's rollout
 * steps built on it) runs batches of at most 4096 envs of the full game on 16-env
 * tiles -- 4096 envs then occupy every CU instead of every other one.  Same path, same
 * tolerance against the fp64 evaluation; the last bits differ from the 32-env kernels
 * (another MFMA shape sums its products in another order), which is why it is opt-in:
 * with the flag off every entry point and batch size produce the same bits for the
 * same env.  fp32 only; ignored by the bf16-input kernel. */
int cfp_policy_set_small_tiles(cfp_policy* p, int on);
int cfp_policy_small_tiles(const cfp_policy* p);

/* Borrowed device pointers owned by the policy object. */
float* cfp_policy_params(cfp_policy* p);    /* [param_count]                 */
float* cfp_policy_state(cfp_policy* p);     /* live h_state [layers][n][256] */
uint8_t* cfp_policy_rec(cfp_policy* p);     /* record scratch [n][996]       */
float* cfp_policy_h_enc(cfp_policy* p);     /* [n][256]                      */
float* cfp_policy_h3(cfp_policy* p);        /* [n][256]                      */
float* cfp_policy_logits(cfp_policy* p);    /* fused head out [n][44]        */
void* cfp_policy_stream(cfp_policy* p);     /* the object's own stream       */

/* cu_encode_step (craftax_full.cu:11931), record half onward: consumes
 * n 996-byte records (rec_row; NULL = the object's scratch) and writes
 * h_enc[n][256] = b_enc + W_enc^T x.  The reference runs k_expand_obs +
 * cublasSgemm + k_add_bias; here the byte->fp32 expansion is the GEMM's
 * operand load and the bias its epilogue, one kernel.  The state->record
 * half of cu_encode_step is cfp_record_obs below. */
int cfp_encode_step(cfp_policy* p, const uint8_t* d_rec_row, int n, void* stream);

/* cu_gru_chain (craftax_full.cu:11978): x0[n][256] -> `layers` MinGRU layers
 * -> h3[n][256].  state[layers][n][256] is read and overwritten; envs with
 * terminals[e] != 0 see a zero state; r_state_t (nullable) receives the
 * post-zero state inputs [layers][n][256].  `chunk` envs per launch
 * (0 = one launch; the reference fixes 16384, craftax_full.cu:11976). */
int cfp_gru_chain(cfp_policy* p, const float* d_x0, float* d_state,
                  const float* d_terminals, float* d_r_state_t, float* d_h3,
                  int n, int chunk, void* stream);

/* Fused head GEMM of cu_rollout_step (craftax_full.cu:12040-12045) plus the
 * bias adds of k_value_sample (craftax_full.cu:9726-9730):
 * av[e][a] = b_a[a] + W_a[a].h3[e] for a < 43, av[e][43] = b_v + W_v.h3[e]. */
int cfp_head(cfp_policy* p, const float* d_h3, float* d_av, int n, void* stream);

/* Policy half of cu_rollout_step (craftax_full.cu:12022-12048) in one launch
 * per chunk: records -> encoder -> MinGRU x layers -> heads.  Updates d_state
 * (NULL = the object's live state) in place, writes d_av[n][44] (NULL = the
 * object's logits buffer); d_r_state_t, d_h_enc, d_h3 are optional outputs
 * (NULL = not written).  `chunk` as in cfp_gru_chain. */
int cfp_policy_forward(cfp_policy* p, const uint8_t* d_rec_row,
                       const float* d_terminals, float* d_state,
                       float* d_r_state_t, float* d_h_enc, float* d_h3,
                       float* d_av, int n, int chunk, void* stream);

/* The same step from the fp32 feature matrix xobs[n][843] (ld 843) instead of records:
 * cu_gemm_enc_fwd on xobs + k_add_bias (craftax_full.cu:11616, :10056; what
 * cu_encode_step runs after k_expand_obs), then the fused MinGRU layers and heads.
 * d_h_enc (NULL = the object's buffer) receives the encoder output.  fp32 features are not
 * exact in bf16, so the record path's three-product encoder does not apply: with the split
 * kernels on (cfp_set_gemm_split, the default) both operands travel as exact three-term bf16
 * splits over K = 848 (nine products, or six / one in the other modes) and the bias is added
 * where the fused kernel stages h_enc (or by k_add_bias when the caller asked for d_h_enc);
 * with them off it is the seam's fp32 MFMA GEMM (cfp_gemm_enc_fwd) and the bias pass.
 * n must be a multiple of 32. */
int cfp_policy_forward_features(cfp_policy* p, const float* d_xobs, const float* d_terminals,
                                float* d_state, float* d_r_state_t, float* d_h_enc, float* d_h3,
                                float* d_av, int n, int chunk, void* stream);

/* ---- the dense-math seam (craftax_full.cu:11604-11666) ------------------- */
/* Workspace of the raw entry points below (cfp_gemm_fwd / dh / dw, cfp_gemv_dwv):
 * 1.1 MB for the split mirror of W, 110 MB of split-K partial sums, 256 KB of gemv
 * slices, allocated once per process -- by this call, or by the first of those entry
 * points that needs it (the reference warms cuBLAS's workspaces the same way before it
 * captures a graph, craftax_full.cu:12094-12122).  Call it before capturing a stream
 * that uses them.  The workspace has one user at a time: raw seam calls in flight
 * together must be on one stream.  Trainer objects do not use it (they own theirs).
 * cfp_set_gemm_bf16 / cfp_set_gemm_split are process-wide and not synchronised: set
 * them while no other thread is inside the library. */
int cfp_seam_reserve(void);
/* bf16 inputs with fp32 accumulation for every GEMM of this seam (cfp_gemm_fwd /
 * enc_fwd / dh / dw, hence the whole PPO update): the reference's process-wide
 * CF_GEMM_BF16 / g_gemm_bf16 switch (craftax_full.cu:11306-11316, wrappers
 * :11688-11756).  Operands stay fp32 in memory and are rounded to bf16 on the way
 * into the kernel; results stay fp32 (the reference also emits bf16 C for the gate
 * and dh GEMMs; this library does not).  Off by default. */
int cfp_set_gemm_bf16(int on);
int cfp_get_gemm_bf16(void);
/* fp32 GEMMs on the bf16 matrix pipe: every fp32 operand is split exactly into three
 * bf16 numbers and each product becomes the nine exact partial products, accumulated
 * in fp32 (same products as cublasSgemm adds up behind cu_gemm_dw / cu_gemm_dh,
 * craftax_full.cu:11642-11666, in 9/16 of the fp32 pipe time).  Used by cfp_gemm_dw and
 * cfp_gemm_dh for the shapes of the PPO update when bf16 inputs are off; other shapes
 * take the fp32 MFMA kernel.  mode 1 (default): all nine partial products; mode 2: the
 * six largest (mid*lo, lo*mid, lo*lo left out: at most 2^-21 of |a*b| per product,
 * about 2^-24 on average, the size of the roundings of the fp32 accumulation; opt-in); mode 3:
 * eight (only lo*lo left out: below 2^-30 of |a*b| per product, 1/64 of one rounding of the
 * fp32 accumulator; opt-in); mode 0: fp32 MFMA everywhere (and, with bf16 inputs on, the generic
 * bf16 kernel).  With cfp_set_gemm_bf16(1) and mode 1, 2 or 3 the same kernels run with both
 * operands rounded to bf16 and one product. */
int cfp_set_gemm_split(int mode);
int cfp_get_gemm_split(void);

/* cu_gemm_fwd (:11604): y[cols][m] = x[cols][k] . W[m][k]^T. */
int cfp_gemm_fwd(int m, int cols, int k, const float* d_W, const float* d_x,
                 float* d_y, void* stream);
/* cu_gemm_enc_fwd (:11616): h[cols][256] = xobs[cols][843] . W_enc[843][256]. */
int cfp_gemm_enc_fwd(int cols, const float* d_W_enc, const float* d_xobs,
                     float* d_h, void* stream);
/* cu_gemm_dh (:11629): dh[cols][256] = dpre[cols][m3] . W[m3][256]. */
int cfp_gemm_dh(int m3, int cols, const float* d_W, const float* d_dpre,
                float* d_dh, void* stream);
/* cfp_gemm_dh for callers that cannot allocate (code under graph capture, serving loops,
 * harnesses that forbid hipMalloc); no counterpart in the reference.  Same result, bit for
 * bit, as cfp_gemm_dh in the split modes (cfp_set_gemm_split 1, the default, and 2) with fp32
 * inputs; in split mode 0 or with cfp_set_gemm_bf16(1) cfp_gemm_dh runs other kernels and
 * this call still runs the split kernel (nine terms in mode 0).  The split mirror of W sits
 * in a 1.125 MiB array inside the library's device image instead of the process-wide
 * workspace, so the call never allocates.  The first call on a GPU resolves that array's
 * address (hipGetSymbolAddress, which may load the code object): make one call outside any
 * graph capture first.
 * Limits: m3 a multiple of 16 up to 768, cols a multiple of 32, d_dpre 16-byte aligned;
 * anything else is an error.  Calls on one GPU share that GPU's array: calls that overlap
 * (two streams, two threads) race on it. */
int cfp_gemm_dh_noalloc(int m3, int cols, const float* d_W, const float* d_dpre,
                        float* d_dh, void* stream);
/* cu_gemm_dw (:11642): dW[rows][256] += dpre[cols][rows]^T . x[cols][256]. */
int cfp_gemm_dw(int rows, int cols, const float* d_x, const float* d_dpre,
                float* d_dW, void* stream);
/* cu_gemv_dwv (:11655): dWv[256] += x[cols][256]^T . dv[cols]. */
int cfp_gemv_dwv(const float* d_x, const float* d_dv, float* d_dWv, int cols,
                 void* stream);

/* k_expand_obs (craftax_full.cu:10028): records -> fp32 features
 * xobs[count][843].  Sample w maps to record (t0 + w/mb)*n + env_start + w%mb,
 * the trainer's window addressing; for a plain batch pass t0=0, mb=n=count,
 * env_start=0. */
int cfp_expand_obs(const uint8_t* d_r_obs, float* d_xobs, int t0, int count,
                   int mb, int n, int env_start, void* stream);
/* k_add_bias (craftax_full.cu:10056): h[cols][256] += b[256]. */
int cfp_add_bias(float* d_h, const float* d_b, int cols, void* stream);
/* Unfused k_mingru_epi_fwd (craftax_full.cu:9350): pre[cols][768], x[cols][256],
 * state[cols][256] in/out, h_out[cols][256], r_state_store nullable. */
int cfp_mingru_epi_fwd(const float* d_pre, const float* d_x, float* d_state,
                       float* d_h_out, float* d_r_state_store,
                       const float* d_prev_terminals, int cols, void* stream);

/* ---- state -> record (k_record_obs, craftax_full.cu:9284; C spec
 *      craftax_encode_compact_observation, craftax_full.c:2830) ------------ */
#define CFP_MOB_SLOTS 14 /* melee 3, passive 3, ranged 2, mob-proj 3, player-proj 3 */
/* The fields of CraftaxState the encoder reads (craftax_full.c:2205-2220,
 * 2646-2703, 2721-2844), one struct per env.  Mob slots are the entries at
 * level jax_index(player_level, 9), in class order. */
typedef struct cfp_env_scalars {
    int32_t player_position[2];
    int32_t player_level;
    int32_t player_direction;            /* 1..4 */
    float player_health;
    int32_t player_food, player_drink, player_energy, player_mana;
    int32_t player_xp, player_dexterity, player_strength, player_intelligence;
    int32_t is_sleeping, is_resting;
    int32_t wood, stone, coal, iron, diamond, sapphire, ruby, sapling, torches,
        arrows, books, pickaxe, sword, bow;
    int32_t potions[6];
    int32_t armour[4];
    int32_t sword_enchantment, bow_enchantment;
    int32_t armour_enchantments[4];
    float light_level;
    int32_t learned_spells[2];
    int32_t monsters_killed_level;       /* monsters_killed[player_level] */
    int32_t boss_timesteps_to_spawn_this_round;
    int32_t mob_type_id[CFP_MOB_SLOTS];
    int32_t mob_mask[CFP_MOB_SLOTS];
    int32_t mob_position[CFP_MOB_SLOTS][2];
} cfp_env_scalars;

/* Writes n records.  map/item_map/light_map: u8 planes of 48x48; plane for
 * (env, level) starts at base + env*env_stride + level*level_stride (bytes);
 * level_stride = 0 when only the current level's plane is supplied. */
int cfp_record_obs(const cfp_env_scalars* d_scalars, const uint8_t* d_map,
                   const uint8_t* d_item_map, const uint8_t* d_light_map,
                   size_t env_stride, size_t level_stride, uint8_t* d_rec_row,
                   int n, void* stream);

/* The same records straight from the reference's device state, so that cu_encode_step
 * (craftax_full.cu:11931-11955) needs no staging kernel in front of this library.
 * cfp_env_soa is a view of the reference's per-field arrays (CF_SOA_FIELDS,
 * craftax_full.cu:620-690; the device pointers g_cf_<field> :703-705): every array is
 * laid out [sub_index][env] with stride n_stride (= g_cf_n) elements, bool fields are
 * one byte, and the mob arrays are indexed CFM(class, level, slot) = (class * 9 +
 * level) * 3 + slot (:706-712; mob_position: that * 2 + axis), classes in the order
 * melee, passive, ranged, mob projectiles, player projectiles.  Only the fields the
 * record encoder reads are listed; all forty pointers must be set.  The planes are the
 * map / item_map / light_map members of the reference's state block: pass their
 * addresses inside the first env's block, env_stride = sizeof(CraftaxState),
 * level_stride = 48 * 48. */
typedef struct cfp_env_soa {
    const int32_t* player_position;            /* 2 */
    const int32_t* player_level;
    const int32_t* player_direction;
    const float* player_health;
    const int32_t* player_food;
    const int32_t* player_drink;
    const int32_t* player_energy;
    const int32_t* player_mana;
    const int32_t* player_xp;
    const int32_t* player_dexterity;
    const int32_t* player_strength;
    const int32_t* player_intelligence;
    const uint8_t* is_sleeping;                /* bool */
    const uint8_t* is_resting;                 /* bool */
    const int32_t* inv_wood;
    const int32_t* inv_stone;
    const int32_t* inv_coal;
    const int32_t* inv_iron;
    const int32_t* inv_diamond;
    const int32_t* inv_sapphire;
    const int32_t* inv_ruby;
    const int32_t* inv_sapling;
    const int32_t* inv_torches;
    const int32_t* inv_arrows;
    const int32_t* inv_books;
    const int32_t* inv_pickaxe;
    const int32_t* inv_sword;
    const int32_t* inv_bow;
    const int32_t* inv_potions;                /* 6 */
    const int32_t* inv_armour;                 /* 4 */
    const int32_t* sword_enchantment;
    const int32_t* bow_enchantment;
    const int32_t* armour_enchantments;        /* 4 */
    const float* light_level;
    const uint8_t* learned_spells;             /* bool, 2 */
    const int32_t* monsters_killed;            /* 9 */
    const int32_t* boss_timesteps_to_spawn_this_round;
    const int32_t* mob_type_id;                /* 135 */
    const uint8_t* mob_mask;                   /* bool, 135 */
    const int32_t* mob_position;               /* 270 */
    size_t n_stride;
} cfp_env_soa;
/* k_record_obs (craftax_full.cu:9284-9296).  `soa` is a host struct, read during the call.
 * d_skip (or NULL): u8[n]; envs whose byte is non-zero are left untouched (the envs whose
 * reset has not joined yet, recorded afterwards by the list form). */
int cfp_record_obs_soa(const cfp_env_soa* soa, const uint8_t* d_map, const uint8_t* d_item_map,
                       const uint8_t* d_light_map, size_t env_stride, size_t level_stride,
                       const uint8_t* d_skip, uint8_t* d_rec_row, int n, void* stream);
/* k_record_obs_list (craftax_full.cu:9303-9320): records only the envs named by the
 * first *d_count entries of a device index list; entry i is the int32 at d_env_list +
 * i * list_stride bytes (a CraftaxResetRec array with its .env member: pass the address
 * of the first .env and sizeof(CraftaxResetRec)).  max_count (<= n) sizes the launch and
 * bounds the list: entries past min(*d_count, max_count) are never read, and an entry
 * outside 0..n-1 is skipped.  n is the env count the rows and arrays are laid out for. */
int cfp_record_obs_soa_list(const cfp_env_soa* soa, const uint8_t* d_map,
                            const uint8_t* d_item_map, const uint8_t* d_light_map,
                            size_t env_stride, size_t level_stride, const void* d_env_list,
                            size_t list_stride, const int* d_count, int max_count,
                            uint8_t* d_rec_row, int n, void* stream);

/* k_value_sample (craftax_full.cu:9714-9741) on the fused head's output
 * av[n][actions+1] (biases already added): values[e] = av[e][actions] (d_values
 * may be NULL), action ~ softmax(av[e][0..actions)) by inversion of the cumulative
 * sum (cf_nn_sample_action :9147-9165), logprob = log softmax at the action; the
 * action also goes to d_env_actions[e] as a float when that is not NULL (the
 * reference's env action slot).  The uniform is the reference's: the first
 * curand_uniform of a Philox4_32_10 state after curand_init(seed ^
 * 0xA5A5A5A5A5A5A5A5, subsequence e, offset *d_step_ctr or 0), computed directly
 * (Philox4x32-10 with key = seed, counter = subsequence * 2^64 + offset / 4, word
 * offset % 4; x * 2^-32 + 2^-33). */
int cfp_value_sample(const float* d_av, int n, int actions, float* d_env_actions,
                     int32_t* d_actions, float* d_logprobs, float* d_values, uint64_t seed,
                     const uint64_t* d_step_ctr, void* stream);
/* k_record_rd (craftax_full.cu:9758-9767): this step's rewards and terminals into
 * the rollout slab rows. */
int cfp_record_rd(const float* d_rewards, const float* d_terminals, float* d_r_reward_row,
                  uint8_t* d_r_done_row, int n, void* stream);

/* ---- PPO update: replaces CuTrain (craftax_full.cu:12688-12761) ----------- */
typedef struct cfp_trainer cfp_trainer;

/* CuPPOConfig + cu_ppo_defaults (craftax_full.cu:12637-12655).  bwd_win is the
 * reference's CF_BWD_WIN (steps per recompute window, :12670); 0 = automatic:
 * the whole horizon up to 262 144 window columns. */
typedef struct cfp_ppo_config {
    float lr, gamma, lam, clip, ent, vf;
    int epochs;
    int minibatches;   /* contiguous env-range slices per epoch          */
    int bptt_split;    /* BPTT segments per env in backward (1 = exact)  */
    int bwd_win;
} cfp_ppo_config;
int cfp_ppo_defaults(cfp_ppo_config* cfg);

/* cu_train_init (craftax_full.cu:12763): allocates the rollout slabs
 * r_obs[T][n][996], r_state[T][layers][n][256], r_act/r_logprob/r_value/
 * r_reward/adv/ret [T][n], r_done u8 [T][n], the grads arena (params layout),
 * Adam moments and the window workspace.  Same argument checks as the
 * reference: minibatches divides n, bptt_split divides T, n/minibatches is a
 * multiple of 32. */
int cfp_train_create(cfp_trainer** out, cfp_policy* p, int T, const cfp_ppo_config* cfg);
/* cu_train_free (craftax_full.cu:12929). */
void cfp_train_destroy(cfp_trainer* tr);

enum cfp_train_buf {
    CFP_BUF_R_OBS = 0, CFP_BUF_R_STATE, CFP_BUF_R_ACT, CFP_BUF_R_LOGPROB,
    CFP_BUF_R_VALUE, CFP_BUF_R_REWARD, CFP_BUF_R_DONE, CFP_BUF_ADV, CFP_BUF_RET,
    CFP_BUF_V_BOOT, CFP_BUF_STATS /* double[2] */, CFP_BUF_LOSS_ACC /* double[3] */,
    CFP_BUF_GRADS, CFP_BUF_ADAM_M, CFP_BUF_ADAM_V, CFP_BUF_LR /* float */,
    CFP_BUF_ENT /* float */, CFP_BUF_STEP_CTR /* uint64: rollout steps taken */
};
/* Borrowed device pointer to one of the trainer's buffers (NULL if unknown). */
void* cfp_train_buffer(cfp_trainer* tr, int which);
/* bf16 storage of the update's window workspace, the reference's CF_GEMM_BF16 storage
 * (craftax_full.cu:12694-12727: bf16 shadows of the gate pre-activations / their
 * gradients and of the layer inputs feed its bf16 GEMMs, reverse kernel's bf16 paths
 * :9538-9590).  In effect only while cfp_set_gemm_bf16(1) is on with the split kernels
 * (cfp_set_gemm_split != 0): the window recompute then writes the gate pre-activations
 * and layer inputs as bf16, the reverse sweep reads them and leaves the gate gradients
 * as bf16, the dW / dh GEMMs take those as their operands unconverted, and the
 * hidden-state gradients between the layers (the dh buffers) are bf16 as well -- half
 * the bytes of the kernels that bound the bf16 update.  r_state, the head rows and
 * every weight gradient stay fp32.  Needs envs per minibatch % 8 == 0 and window
 * columns (steps x envs) % 32 == 0; a window that does not fit runs with fp32 storage.
 * Off by default. */
int cfp_train_set_bf16_storage(cfp_trainer* tr, int on);
int cfp_train_bf16_storage(const cfp_trainer* tr);

/* bf16 r_state slab, the rest of the reference's CF_GEMM_BF16 storage
 * (craftax_full.cu:12694-12700, read paths :9470-9480, :9538-9590): the rollout's forward
 * writes the post-zero state rows as bf16 and the update's window recompute and reverse sweep
 * read them as bf16 -- half of the 805 MB the recompute reads at 262 144 columns and 2 of the
 * sweep's bytes per element.  The slab keeps its shape [T][layers][n][256] and its buffer
 * (CFP_BUF_R_STATE then holds bf16 elements in the first half of the allocation).  Both ends
 * exist on the bf16 path only: set it before the rollout writes the slab, on a policy with
 * cfp_policy_set_gemm_bf16(1); cfp_train_backward then requires the bf16 update mode
 * (bf16 GEMM inputs, split kernels, cfp_train_set_bf16_storage(1)) and fails with a clear
 * error otherwise, as does a forward on the fp32 kernels that is asked to write r_state.
 * The live state stays fp32.  Off by default. */
int cfp_train_set_bf16_rstate(cfp_trainer* tr, int on);
int cfp_train_bf16_rstate(const cfp_trainer* tr);

/* Phase timers of the training loop, the counterpart of CRAFTAX_CU_TRAIN_PROF
 * (craftax_full.cu:12925-12926, cu_prof_mark :12973-12980, read out at :13374 and :13659):
 * with the timers on, cfp_train_collect and cfp_train_update wait for the stream at every
 * phase boundary and add the host-clock time of each phase to four sums -- rollout (the T
 * steps of cfp_env_rollout_step), gae (last record, bootstrap value, advantages), backward,
 * adam -- and cfp_train_update runs eagerly whatever use_graph says, as the reference's does.
 * cfp_train_profile copies the sums (milliseconds) to host memory and, with reset != 0,
 * clears them.  Off by default; the waits cost throughput, so this is a diagnosis aid. */
int cfp_train_set_profile(cfp_trainer* tr, int on);
int cfp_train_profile(cfp_trainer* tr, double* ms4, int reset);

/* GEMM mode of one trainer's update.  The reference has one process-wide switch
 * (g_gemm_bf16, craftax_full.cu:11306-11316) and one trainer per process; here two trainers
 * may live in one process, each with a captured update graph, so a trainer can carry its own
 * mode: bf16 = 0 / 1 and split = 0 / 1 / 2 / 3 as in cfp_set_gemm_bf16 / cfp_set_gemm_split, or
 * -1 to follow the process-wide switch (the default for both).  cfp_train_backward and
 * cfp_train_update run with the trainer's mode whatever the process-wide switches say, and
 * cfp_train_update's graph is captured again only when the trainer's effective mode changed.
 * The raw seam calls (cfp_gemm_*) always follow the process-wide switches. */
int cfp_train_set_gemm_mode(cfp_trainer* tr, int bf16, int split);
/* The mode the trainer's next update runs with (its own, or the process-wide one). */
int cfp_train_gemm_mode(const cfp_trainer* tr, int* bf16, int* split);
int cfp_train_window(const cfp_trainer* tr);
int cfp_train_minibatch(const cfp_trainer* tr);

/* Policy half of one cu_train_collect step (craftax_full.cu:12987-12995): runs
 * the fused forward on the policy's live state for step t, storing the record
 * row into r_obs[t], the post-zero state inputs into r_state[t] and the value
 * into r_value[t]; logits stay in the policy's logits buffer.  Sampling and the
 * env step are the caller's. */
int cfp_train_record_step(cfp_trainer* tr, int t, const uint8_t* d_rec_row,
                          const float* d_terminals, void* stream);
/* Policy half of cu_rollout_step (craftax_full.cu:12022-12044): as
 * cfp_train_record_step, then samples an action per env from the logits
 * (cfp_value_sample with the trainer's device step counter as the sampler
 * offset) into r_act[t] / r_logprob[t] / r_value[t] and, when d_env_actions is
 * not NULL, into the env's float action slots; the step counter is then bumped
 * on the device (k_bump_ctr :9770), so a captured graph replays with fresh draws. */
int cfp_rollout_step(cfp_trainer* tr, int t, const uint8_t* d_rec_row,
                     const float* d_prev_terminals, uint64_t seed, float* d_env_actions,
                     void* stream);
/* Bootstrap value of cu_train_collect (craftax_full.cu:12996-13006): V(s_T) from
 * the post-rollout records on a COPY of the policy's live state (which is left
 * untouched), into v_boot. */
int cfp_train_bootstrap(cfp_trainer* tr, const uint8_t* d_rec_row, const float* d_terminals,
                        void* stream);
/* k_gae + k_adv_stats of cu_train_collect (craftax_full.cu:13007-13011). */
int cfp_train_gae(cfp_trainer* tr, void* stream);
/* k_adv_stats alone (when adv was filled by the caller). */
int cfp_train_adv_stats(cfp_trainer* tr, void* stream);
/* cu_train_backward (craftax_full.cu:13168): accumulates the gradients of the
 * minibatch [env_start, env_start+env_count) into the grads arena and the raw
 * loss sums (pg, v, ent) into loss_acc. */
int cfp_train_backward(cfp_trainer* tr, int env_start, int env_count, void* stream);
int cfp_train_zero_loss(cfp_trainer* tr, void* stream);
/* cu_train_adam (craftax_full.cu:13337): Adam step from the grads arena (which
 * it zeroes), bumps the step counter, rebuilds the weight mirrors. */
int cfp_train_adam(cfp_trainer* tr, void* stream);
/* cu_train_body without its collect + cu_train_update (craftax_full.cu:13348-13406):
 * one PPO iteration over the stored rollout (slabs, adv/ret and the advantage
 * statistics already in place): epochs x (loss sums reset, minibatches x
 * (cfp_train_backward of the m-th contiguous env slice, cfp_train_adam)), then a
 * synchronisation of the stream, as in the reference.  use_graph != 0 is the
 * reference's graph mode: the first call captures the iteration once on `stream`
 * (on a stream of the trainer's own when `stream` is NULL, which cannot be
 * captured) and replays it; later calls only replay.  No warm-up pass is needed
 * (the reference runs one for cuBLAS's lazy workspaces): the trainer owns every
 * buffer the iteration touches.  lr, the entropy
 * coefficient and the Adam step counter live in device memory, so replays see
 * their current values.  A change of cfp_set_gemm_split / cfp_set_gemm_bf16 /
 * cfp_policy_set_gemm_bf16 between calls makes the next call capture again.
 * Unlike the reference, a graph that cannot be instantiated is an error, not a
 * silent eager run: call again with use_graph = 0. */
int cfp_train_update(cfp_trainer* tr, int use_graph, void* stream);
/* cu_train_loss (craftax_full.cu:13414): full-batch PPO loss of the stored
 * rollout with live recurrence inside BPTT segments; host_loss4 = raw sums
 * (pg, v, ent) and the total (pg + vf*v - ent*H) / (n*T).  Synchronises. */
int cfp_train_loss(cfp_trainer* tr, double* host_loss4, void* stream);

/* ---- synthetic inputs for parity tests and bench (no reference
 *      counterpart; counter-based so host and device agree bit for bit) ---- */
/* Records: 792 map bytes, each U{0..40}; 51 tail floats U[0,1) on a 24-bit grid.
 * Dword d of env e at step s is a function of (seed, s, 249 e + d) alone. */
int cfp_synth_records(uint8_t* d_rec, int n, uint64_t seed, uint64_t step,
                      void* stream);

/* Classic records: block ids U{0..16}, mob bitmask nonzero for ~2 % of cells,
 * 16 scalars U{0..9}, direction U{1..4}, sleeping Bernoulli(1/2), light U[0,1). */
int cfp_synth_classic_records(uint8_t* d_rec, int n, uint64_t seed, uint64_t step,
                              void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CFP_H_ */
