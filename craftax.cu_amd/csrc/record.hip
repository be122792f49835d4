// Observation-record kernels: state -> 996-byte compact record, record ->
// fp32 features, and the unfused elementwise pieces of the forward
// (bias add, MinGRU gate/blend epilogue) kept for parity tests and for the
// PPO update's window recompute.
//
// Record format (craftax_full.c:578-581, encoder :2721-2844): 99 view cells
// (9 rows x 11 cols, row-major) x 8 bytes {block, item+1, visible, melee+1,
// passive+1, ranged+1, mob-projectile+1, player-projectile+1}, then 51 raw
// little-endian fp32 scalars.  All of it is integer/byte work bound by HBM
// gathers; sixteen lanes encode one env.
#include <cstring>

#include "cfp_common.h"
#include "env_internal.h"

namespace cfp {
namespace {

constexpr int MAP = 48;
constexpr int ROWS = 9, COLS = 11, CELLS = ROWS * COLS;

__device__ __forceinline__ int jax_index(int index, int size) {
    // craftax_wg_jax_index, craftax_full.c:2180
    if (index < 0) index += size;
    if (index < 0) return 0;
    if (index >= size) return size - 1;
    return index;
}

// How each of the 51 tail scalars is derived (craftax_full.c:2646-2703).
enum TailKind : uint8_t {
    T_SQRT10,   // sqrtf((float)i) * 0.1f
    T_HALF,     // (float)i * 0.5f
    T_QUARTER,  // (float)i * 0.25f
    T_INT,      // (float)i
    T_F10,      // f * 0.1f          (float field)
    T_I10,      // (float)i * 0.1f
    T_DIR,      // one-hot of player_direction - 1, slot in `aux`
    T_FLOAT,    // f
    T_BOOL,     // i != 0
    T_KILLED,   // i >= 8
    T_BOSS,     // boss vulnerable
};
struct TailSpec { uint8_t kind, field, aux; };

#define FLD(name) ((uint8_t)(offsetof(cfp_env_scalars, name) / 4))
__constant__ TailSpec kTail[CFP_OBS_TAIL] = {
    {T_SQRT10, FLD(wood), 0},      {T_SQRT10, FLD(stone), 0},
    {T_SQRT10, FLD(coal), 0},      {T_SQRT10, FLD(iron), 0},
    {T_SQRT10, FLD(diamond), 0},   {T_SQRT10, FLD(sapphire), 0},
    {T_SQRT10, FLD(ruby), 0},      {T_SQRT10, FLD(sapling), 0},
    {T_SQRT10, FLD(torches), 0},   {T_SQRT10, FLD(arrows), 0},
    {T_HALF, FLD(books), 0},       {T_QUARTER, FLD(pickaxe), 0},
    {T_QUARTER, FLD(sword), 0},    {T_INT, FLD(sword_enchantment), 0},
    {T_INT, FLD(bow_enchantment), 0}, {T_INT, FLD(bow), 0},
    {T_SQRT10, FLD(potions[0]), 0}, {T_SQRT10, FLD(potions[1]), 0},
    {T_SQRT10, FLD(potions[2]), 0}, {T_SQRT10, FLD(potions[3]), 0},
    {T_SQRT10, FLD(potions[4]), 0}, {T_SQRT10, FLD(potions[5]), 0},
    {T_F10, FLD(player_health), 0}, {T_I10, FLD(player_food), 0},
    {T_I10, FLD(player_drink), 0}, {T_I10, FLD(player_energy), 0},
    {T_I10, FLD(player_mana), 0},  {T_I10, FLD(player_xp), 0},
    {T_I10, FLD(player_dexterity), 0}, {T_I10, FLD(player_strength), 0},
    {T_I10, FLD(player_intelligence), 0},
    {T_DIR, FLD(player_direction), 0}, {T_DIR, FLD(player_direction), 1},
    {T_DIR, FLD(player_direction), 2}, {T_DIR, FLD(player_direction), 3},
    {T_HALF, FLD(armour[0]), 0},   {T_HALF, FLD(armour[1]), 0},
    {T_HALF, FLD(armour[2]), 0},   {T_HALF, FLD(armour[3]), 0},
    {T_INT, FLD(armour_enchantments[0]), 0}, {T_INT, FLD(armour_enchantments[1]), 0},
    {T_INT, FLD(armour_enchantments[2]), 0}, {T_INT, FLD(armour_enchantments[3]), 0},
    {T_FLOAT, FLD(light_level), 0}, {T_BOOL, FLD(is_sleeping), 0},
    {T_BOOL, FLD(is_resting), 0},  {T_BOOL, FLD(learned_spells[0]), 0},
    {T_BOOL, FLD(learned_spells[1]), 0}, {T_I10, FLD(player_level), 0},
    {T_KILLED, FLD(monsters_killed_level), 0}, {T_BOSS, 0, 0},
};
#undef FLD

// class (record channel - 3) of each of the 14 mob slots
__constant__ uint8_t kSlotClass[CFP_MOB_SLOTS] = {0, 0, 0, 1, 1, 1, 2, 2,
                                                  3, 3, 3, 4, 4, 4};

// Sixteen lanes per env, the record assembled in LDS and written out
// as 249 coalesced dwords: lanes walk the 99 view cells (block, item, visible),
// lanes 0..13 each judge one mob slot and drop its byte into its cell, the lanes
// share the 51 tail values.  LDS operations of a wave execute in program order, so
// the byte of a mob lands after the dword of its cell without a barrier.
constexpr int kRecLanes = 16;                   // lanes per env: four envs per wavefront,
constexpr int kRecEnvsPerWg = 256 / kRecLanes;  // more gathers in flight than with one (85 -> 42 us)

// Where an env's scalars come from.  SOA: the reference's device state (one array per
// field laid out [sub_index][env], craftax_full.cu:613-723); the kernel asks for the words
// of cfp_env_scalars it needs and a table says which array holds each.
constexpr int kSoaPtrs = 40;
constexpr int kSoaGather = 32;   // envs per gather round: one 128-byte line of an int32 field array (64 envs: slower)
constexpr int kSoaGatherFew = 16;   // up to kSoaFewItems envs: twice the workgroups for a GPU that is not full
constexpr int kSoaFewItems = 16384;  // (8192 envs: 24 -> 19 us; 65 536 envs: 69 -> 84 us with the small rounds)
struct SoaArgs {
    const void* p[kSoaPtrs];   // the pointer fields of cfp_env_soa, in declaration order
    size_t n_stride;
};
static_assert(sizeof(cfp_env_soa) == sizeof(SoaArgs), "cfp_env_soa is forty pointers and a stride");
constexpr int kScalarWords = (int)(sizeof(cfp_env_scalars) / 4);

// One descriptor per 4-byte word of cfp_env_scalars: the array it comes from, how its
// element is typed and how the sub-index is formed.
enum : uint8_t { K_I32 = 0, K_F32 = 1, K_BOOL = 2 };
enum : uint8_t { R_SUB = 0, R_LEVEL = 1, R_MOB = 2, R_MOBPOS0 = 3, R_MOBPOS1 = 4 };
struct SoaWord { uint8_t ptr, kind, rule, aux; };
// Mob words: the reference's arrays hold three slots per class and level, CFM(c, l, i) =
// (c * 9 + l) * 3 + i (craftax_full.cu:706-712); aux = c * 27 + i, so the element is
// aux + 3 * level (mob_position: twice that, plus the axis).  The 14 slots in class order:
// melee 0..2, passive 3..5, ranged 6..7, mob projectiles 8..10, player projectiles 11..13.
#define SW(ptr, kind, rule, aux) {ptr, kind, rule, aux}
#define SW_SLOTS(ptr, kind, rule)                                                               \
    SW(ptr, kind, rule, 0), SW(ptr, kind, rule, 1), SW(ptr, kind, rule, 2),                     \
    SW(ptr, kind, rule, 27), SW(ptr, kind, rule, 28), SW(ptr, kind, rule, 29),                  \
    SW(ptr, kind, rule, 54), SW(ptr, kind, rule, 55),                                           \
    SW(ptr, kind, rule, 81), SW(ptr, kind, rule, 82), SW(ptr, kind, rule, 83),                  \
    SW(ptr, kind, rule, 108), SW(ptr, kind, rule, 109), SW(ptr, kind, rule, 110)
#define SW_POS(aux) SW(39, K_I32, R_MOBPOS0, aux), SW(39, K_I32, R_MOBPOS1, aux)
__constant__ SoaWord kSoaWords[kScalarWords] = {
    SW(0, K_I32, R_SUB, 0), SW(0, K_I32, R_SUB, 1),            // player_position
    SW(1, K_I32, R_SUB, 0), SW(2, K_I32, R_SUB, 0),            // player_level, player_direction
    SW(3, K_F32, R_SUB, 0),                                    // player_health
    SW(4, K_I32, R_SUB, 0), SW(5, K_I32, R_SUB, 0), SW(6, K_I32, R_SUB, 0), SW(7, K_I32, R_SUB, 0),
    SW(8, K_I32, R_SUB, 0), SW(9, K_I32, R_SUB, 0), SW(10, K_I32, R_SUB, 0), SW(11, K_I32, R_SUB, 0),
    SW(12, K_BOOL, R_SUB, 0), SW(13, K_BOOL, R_SUB, 0),        // is_sleeping, is_resting
    // wood stone coal iron diamond sapphire ruby sapling torches arrows books pickaxe sword bow
    SW(14, K_I32, R_SUB, 0), SW(15, K_I32, R_SUB, 0), SW(16, K_I32, R_SUB, 0), SW(17, K_I32, R_SUB, 0),
    SW(18, K_I32, R_SUB, 0), SW(19, K_I32, R_SUB, 0), SW(20, K_I32, R_SUB, 0), SW(21, K_I32, R_SUB, 0),
    SW(22, K_I32, R_SUB, 0), SW(23, K_I32, R_SUB, 0), SW(24, K_I32, R_SUB, 0), SW(25, K_I32, R_SUB, 0),
    SW(26, K_I32, R_SUB, 0), SW(27, K_I32, R_SUB, 0),
    SW(28, K_I32, R_SUB, 0), SW(28, K_I32, R_SUB, 1), SW(28, K_I32, R_SUB, 2),   // potions
    SW(28, K_I32, R_SUB, 3), SW(28, K_I32, R_SUB, 4), SW(28, K_I32, R_SUB, 5),
    SW(29, K_I32, R_SUB, 0), SW(29, K_I32, R_SUB, 1), SW(29, K_I32, R_SUB, 2), SW(29, K_I32, R_SUB, 3),
    SW(30, K_I32, R_SUB, 0), SW(31, K_I32, R_SUB, 0),          // sword / bow enchantment
    SW(32, K_I32, R_SUB, 0), SW(32, K_I32, R_SUB, 1), SW(32, K_I32, R_SUB, 2), SW(32, K_I32, R_SUB, 3),
    SW(33, K_F32, R_SUB, 0),                                   // light_level
    SW(34, K_BOOL, R_SUB, 0), SW(34, K_BOOL, R_SUB, 1),        // learned_spells
    SW(35, K_I32, R_LEVEL, 0),                                 // monsters_killed[player_level]
    SW(36, K_I32, R_SUB, 0),                                   // boss_timesteps_to_spawn_this_round
    SW_SLOTS(37, K_I32, R_MOB),                                // mob_type_id[slot]
    SW_SLOTS(38, K_BOOL, R_MOB),                               // mob_mask[slot]
    SW_POS(0), SW_POS(1), SW_POS(2), SW_POS(27), SW_POS(28), SW_POS(29), SW_POS(54), SW_POS(55),
    SW_POS(81), SW_POS(82), SW_POS(83), SW_POS(108), SW_POS(109), SW_POS(110),   // mob_position
};
#undef SW_POS
#undef SW_SLOTS
#undef SW

// Which envs a launch records.  skip (or null): envs whose byte is set are left alone
// (the reference's k_record_obs, craftax_full.cu:9284-9296).  list (or null): only the envs
// named by *count entries of an index list are recorded, grid-strided
// (k_record_obs_list, :9303-9320); entry i is the int32 at list + i * list_stride.
struct RecWhich {
    const uint8_t* skip;
    const unsigned char* list;
    size_t list_stride;
    const int* count;
    int max_count;   // the list form never reads past this many entries, whatever *count says
    int* zero;       // not null: the first thread of the launch stores 0 there
};

constexpr int kWPos = (int)(offsetof(cfp_env_scalars, player_position) / 4);
constexpr int kWLevel = (int)(offsetof(cfp_env_scalars, player_level) / 4);
constexpr int kWBossTimer = (int)(offsetof(cfp_env_scalars, boss_timesteps_to_spawn_this_round) / 4);
constexpr int kWMobType = (int)(offsetof(cfp_env_scalars, mob_type_id) / 4);
constexpr int kWMobMask = (int)(offsetof(cfp_env_scalars, mob_mask) / 4);
constexpr int kWMobPos = (int)(offsetof(cfp_env_scalars, mob_position) / 4);

// SOA: the scalars of 32 envs are first gathered into LDS copies of cfp_env_scalars,
// transposed: thread (word group gw, env ge) fetches words gw, gw + 8, ... of env ge, so the
// 32 lanes of a word read 32 adjacent envs of one field array -- one 128-byte line -- and
// all of a thread's fourteen elements are in flight together.  The rest of the kernel then
// reads that copy exactly as it reads a caller-staged struct.
struct WordSrc {
    const uint32_t* w;
    __device__ __forceinline__ uint32_t word(int i) const { return w[i]; }
};

// ROW16: the three byte planes are read as one 16-byte piece per window row and plane (the
// 11 window bytes of a row lie inside a 4-byte-aligned 16-byte piece of the 48-byte map row)
// into an LDS strip, and the cells pick their bytes out of the strip: 27 sixteen-byte loads
// per env instead of 297 single-byte ones.  Needs 4-byte-aligned planes and strides.
template <bool SOA, bool ROW16, int SOA_GATHER = kSoaGather>
__global__ __launch_bounds__(256) void k_record_obs(
    const cfp_env_scalars* __restrict__ scalars, SoaArgs soa, RecWhich which,
    const uint8_t* __restrict__ map, const uint8_t* __restrict__ item_map,
    const uint8_t* __restrict__ light_map, size_t env_stride,
    size_t level_stride, uint8_t* __restrict__ rec_row, int n) {
    __shared__ uint32_t stage_all[kRecEnvsPerWg][CFP_REC_BYTES / 4 + 3];
    typedef unsigned int strip_u4 __attribute__((ext_vector_type(4)));
    __shared__ strip_u4 strip_all[ROW16 ? kRecEnvsPerWg : 1][3 * ROWS + 1];   // [plane * 9 + row], odd stride
    // SOA rounds take 32 envs: a 128-byte line of every field array is used by one workgroup
    constexpr int kGather = SOA ? SOA_GATHER : kRecEnvsPerWg;
    __shared__ uint32_t sc_all[SOA ? kGather : 1][kScalarWords + 1];
    __shared__ const void* ptrs[SOA ? kSoaPtrs : 1];
    __shared__ SoaWord words[SOA ? kScalarWords : 1];
    const int lane = threadIdx.x % kRecLanes;
    const int slot = threadIdx.x / kRecLanes;
    if (which.zero != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *which.zero = 0;
    if (SOA) {
#pragma unroll
        for (int i = 0; i < kSoaPtrs; i++)
            if ((int)threadIdx.x == i) ptrs[i] = soa.p[i];
        if ((int)threadIdx.x < kScalarWords) words[threadIdx.x] = kSoaWords[threadIdx.x];
    }
    const int total = which.list ? min(*which.count, which.max_count) : n;
    // the trip count is the same for every thread of the workgroup (barriers inside)
    for (int first = (int)blockIdx.x * kGather; first < total; first += (int)gridDim.x * kGather) {
        if (SOA) {
            __syncthreads();   // tables filled; the previous round's readers are done with sc_all
            constexpr int kGroups = 256 / kGather;
            const int ge = threadIdx.x % kGather, gw = threadIdx.x / kGather;
            const int gi = first + ge;
            int genv = gi;
            if (which.list && gi < total)
                genv = *reinterpret_cast<const int32_t*>(which.list + (size_t)gi * which.list_stride);
            // a list entry outside the env range is ignored (never used as an index)
            if (gi < total && (unsigned)genv < (unsigned)n && !(which.skip && which.skip[genv])) {
                const int lvl = static_cast<const int32_t*>(ptrs[1])[genv];
                const int lvl_c = lvl < 0 ? 0 : (lvl > 8 ? 8 : lvl);   // monsters_killed has nine entries
                const int ml3 = 3 * jax_index(lvl, 9);
                constexpr int kRounds = (kScalarWords + kGroups - 1) / kGroups;
                uint32_t val[kRounds];
#pragma unroll
                for (int r = 0; r < kRounds; r++) {
                    const int w = gw + kGroups * r;
                    const SoaWord d = words[w < kScalarWords ? w : 0];
                    size_t sub = d.aux;
                    if (d.rule == R_LEVEL) sub = (size_t)lvl_c;
                    if (d.rule == R_MOB) sub = (size_t)(d.aux + ml3);
                    if (d.rule >= R_MOBPOS0) sub = (size_t)(2 * (d.aux + ml3) + (d.rule - R_MOBPOS0));
                    const size_t idx = sub * soa.n_stride + (size_t)genv;
                    const void* base = ptrs[d.ptr];
                    val[r] = d.kind == K_BOOL
                                 ? (uint32_t)(static_cast<const uint8_t*>(base)[idx] != 0)
                                 : static_cast<const uint32_t*>(base)[idx];
                }
#pragma unroll
                for (int r = 0; r < kRounds; r++)
                    if (gw + kGroups * r < kScalarWords) sc_all[ge][gw + kGroups * r] = val[r];
            }
            __syncthreads();
        }
        for (int part = 0; part < kGather / kRecEnvsPerWg; part++) {
            const int item = first + part * kRecEnvsPerWg + slot;
            if (item >= total) continue;
            int env = item;
            if (which.list)
                env = *reinterpret_cast<const int32_t*>(which.list + (size_t)item * which.list_stride);
            if ((unsigned)env >= (unsigned)n) continue;
            if (which.skip && which.skip[env]) continue;
            uint32_t* stage = stage_all[slot];
            WordSrc s;
            s.w = SOA ? sc_all[part * kRecEnvsPerWg + slot] : reinterpret_cast<const uint32_t*>(scalars + env);
            const int level = (int)s.word(kWLevel);
            const int mlevel = jax_index(level, 9);
            const int pr = (int)s.word(kWPos), pc = (int)s.word(kWPos + 1);
            const size_t cell_plane = (size_t)env * env_stride + (size_t)level * level_stride;
            const size_t mob_plane = (size_t)env * env_stride + (size_t)mlevel * level_stride;

            // first map column of the 16-byte piece of every window row: a multiple of four at or
            // below the window's first column, inside the map
            const int wc0 = pc - COLS / 2;
            int cb = wc0 < 0 ? 0 : (wc0 & ~3);
            cb = cb > MAP - 16 ? MAP - 16 : cb;
            const bool strips = ROW16 && level >= 0 && level < 9 && pc >= -64 && pc < 2 * MAP;
            if (strips) {
                strip_u4* strip = strip_all[slot];
                for (int i = lane; i < 3 * ROWS; i += kRecLanes) {
                    const int plane = i / ROWS, row = i - plane * ROWS;
                    const int wr = pr - ROWS / 2 + row;
                    strip_u4 v = {0u, 0u, 0u, 0u};
                    if (wr >= 0 && wr < MAP) {
                        const uint8_t* base = plane == 0 ? map : (plane == 1 ? item_map : light_map);
                        v = *reinterpret_cast<const strip_u4*>(base + cell_plane + (size_t)(wr * MAP + cb));
                    }
                    strip[i] = v;
                }
                __builtin_amdgcn_wave_barrier();
            }
            for (int cell = lane; cell < CELLS; cell += kRecLanes) {
                const int row = cell / COLS, col = cell - row * COLS;
                const int wr = pr - ROWS / 2 + row, wc = pc - COLS / 2 + col;
                uint32_t lo = 0;
                if (wr >= 0 && wr < MAP && wc >= 0 && wc < MAP) {
                    uint32_t lv, bv, iv;
                    if (strips) {
                        const uint8_t* sb = reinterpret_cast<const uint8_t*>(strip_all[slot]) + row * 16 + (wc - cb);
                        bv = sb[0];
                        iv = sb[ROWS * 16];
                        lv = sb[2 * ROWS * 16];
                    } else {
                        // all three planes requested at once (one memory round trip, not two)
                        const size_t o = cell_plane + (size_t)(wr * MAP + wc);
                        lv = light_map[o]; bv = map[o]; iv = item_map[o];
                    }
                    if (lv > 12) lo = bv | ((uint32_t)(uint8_t)(iv + 1) << 8) | (1u << 16);
                }
                stage[2 * cell] = lo;
                stage[2 * cell + 1] = 0u;
            }

            // Mob slot m = lane contributes (cell, channel 3 + class, type + 1) when it passes
            // the predicates of craftax_encode_mobs{3,2}_compact (craftax_full.c:2747-2825).
            // Within a class the last slot on a cell wins: a slot stands back when one of the
            // (at most two) later slots of its class sits on the same cell.
            {
                const int m = lane < CFP_MOB_SLOTS ? lane : CFP_MOB_SLOTS - 1;
                const int type = (int)s.word(kWMobType + m);
                const int mr = (int)s.word(kWMobPos + 2 * m), mc = (int)s.word(kWMobPos + 2 * m + 1);
                const uint32_t mask = s.word(kWMobMask + m);
                const int lr = mr - pr + ROWS / 2, lc = mc - pc + COLS / 2;
                bool ok = lane < CFP_MOB_SLOTS && type >= 0 && type < 8 && mask != 0 &&
                          lr >= 0 && lr < ROWS && lc >= 0 && lc < COLS && mr >= 0 && mr < MAP &&
                          mc >= 0 && mc < MAP;
                if (ok) {
                    // a mob that passed the window test sits on a cell of the strip
                    if (strips && mlevel == level)
                        ok = reinterpret_cast<const uint8_t*>(strip_all[slot])[(2 * ROWS + lr) * 16 + (mc - cb)] > 12;
                    else
                        ok = light_map[mob_plane + (size_t)(mr * MAP + mc)] > 12;
                }
                const int cell = ok ? lr * COLS + lc : -1;
                const int cls = kSlotClass[m];
                bool over = false;
    #pragma unroll
                for (int d = 1; d <= 2; d++) {
                    const int oc = __shfl_down(cell, d, kRecLanes);
                    const int ocls = __shfl_down(cls, d, kRecLanes);
                    over = over || (lane + d < CFP_MOB_SLOTS && ocls == cls && oc == cell);
                }
                if (ok && !over)
                    reinterpret_cast<uint8_t*>(stage)[cell * 8 + 3 + cls] = (uint8_t)(type + 1);
            }

            for (int tj = lane; tj < CFP_OBS_TAIL; tj += kRecLanes) {
                const TailSpec ts = kTail[tj];
                const int iv = (int)s.word(ts.field);
                const float fv = __int_as_float(iv);
                const float xi = (float)iv;
                float v = 0.0f;
                switch (ts.kind) {
                    // IEEE sqrt: HIP's __fsqrt_rn is the approximate native sqrt unless
                    // OCML_BASIC_ROUNDED_OPERATIONS is defined; the fp64 root rounded
                    // to fp32 is the correctly rounded fp32 root (53 >= 2*24 + 2).
                    case T_SQRT10: v = (float)sqrt((double)xi) * 0.1f; break;
                    case T_HALF: v = xi * 0.5f; break;
                    case T_QUARTER: v = xi * 0.25f; break;
                    case T_INT: v = xi; break;
                    case T_F10: v = fv * 0.1f; break;
                    case T_I10: v = xi * 0.1f; break;
                    case T_DIR: v = (iv - 1 == (int)ts.aux) ? 1.0f : 0.0f; break;
                    case T_FLOAT: v = fv; break;
                    case T_BOOL: v = iv != 0 ? 1.0f : 0.0f; break;
                    case T_KILLED: v = iv >= 8 ? 1.0f : 0.0f; break;
                    case T_BOSS: {
                        // craftax_wg_is_boss_vulnerable, craftax_full.c:2205: no live
                        // melee (slots 0..2) or ranged (slots 6..7) mob, spawn timer <= 0
                        bool any = false;
                        for (int m = 0; m < 3; m++) any = any || s.word(kWMobMask + m) != 0;
                        for (int m = 6; m < 8; m++) any = any || s.word(kWMobMask + m) != 0;
                        v = (!any && (int)s.word(kWBossTimer) <= 0) ? 1.0f : 0.0f;
                    } break;
                }
                stage[CFP_OBS_MAP / 4 + tj] = __float_as_uint(v);
            }

            __builtin_amdgcn_wave_barrier();
            uint32_t* out = reinterpret_cast<uint32_t*>(rec_row + (size_t)env * CFP_REC_BYTES);
            for (int d = lane; d < CFP_REC_BYTES / 4; d += kRecLanes) out[d] = stage[d];
            __builtin_amdgcn_wave_barrier();   // the staging row is reused by the next item
        }
    }
}

__global__ void k_expand_obs(const uint8_t* __restrict__ r_obs,
                             float* __restrict__ xobs, int t0, size_t total,
                             int mb, int n, int env_start, int ld) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int f = (int)(idx % (size_t)ld);
    const size_t w = idx / (size_t)ld;
    if (f >= CFP_OBS) { xobs[idx] = 0.0f; return; }   // padding of a widened row
    const size_t t = (size_t)t0 + w / (size_t)mb;
    const size_t el = w % (size_t)mb;
    const uint8_t* rec = r_obs + (t * (size_t)n + env_start + el) * CFP_REC_BYTES;
    float x;
    if (f < CFP_OBS_MAP) {
        x = (float)rec[f];
    } else {
        const uint32_t* tail = reinterpret_cast<const uint32_t*>(rec + CFP_OBS_MAP);
        x = __uint_as_float(tail[f - CFP_OBS_MAP]);
    }
    xobs[idx] = x;
}

// Four features per thread, for rows whose width is a multiple of four floats
// and 16-byte aligned: one dword of the record in (four map bytes, or one to four
// tail floats), one 16-byte store out.  792 = 4 * 198, so a group never straddles
// the map / tail boundary.
__global__ void k_expand_obs_v4(const uint8_t* __restrict__ r_obs, f4* __restrict__ xobs4,
                                int t0, size_t total4, int mb, int n, int env_start, int ld4) {
    static_assert(CFP_OBS_MAP % 4 == 0, "map bytes end on a dword");
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total4) return;
    const unsigned w = (unsigned)(idx / (unsigned)ld4);
    const int f = 4 * (int)(idx - (size_t)w * (unsigned)ld4);
    const unsigned tr = w / (unsigned)mb;
    const unsigned el = w - tr * (unsigned)mb;
    const uint32_t* rec = reinterpret_cast<const uint32_t*>(
        r_obs + (((size_t)t0 + tr) * (size_t)n + env_start + el) * CFP_REC_BYTES);
    f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (f < CFP_OBS_MAP) {
        const uint32_t b = __builtin_nontemporal_load(rec + (f >> 2));
        v[0] = (float)(b & 0xffu);
        v[1] = (float)((b >> 8) & 0xffu);
        v[2] = (float)((b >> 16) & 0xffu);
        v[3] = (float)(b >> 24);
    } else {
        const uint32_t* tail = rec + CFP_OBS_MAP / 4 + (f - CFP_OBS_MAP);
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (f + j < CFP_OBS) v[j] = __uint_as_float(tail[j]);
    }
    __builtin_nontemporal_store(v, xobs4 + idx);
}

// Any row width, output base 16-byte aligned: thread i writes flat floats
// 4i .. 4i+3 with one 16-byte store; a group may run over the end of a row
// into the next sample.
__global__ void k_expand_obs_flat4(const uint8_t* __restrict__ r_obs, float* __restrict__ xobs,
                                   int t0, size_t total, int mb, int n, int env_start, int ld) {
    const size_t i0 = 4 * ((size_t)blockIdx.x * blockDim.x + threadIdx.x);
    if (i0 >= total) return;
    unsigned w = (unsigned)(i0 / (unsigned)ld);
    int f = (int)(i0 - (size_t)w * (unsigned)ld);
    auto rec_of = [&](unsigned ww) {
        const unsigned tr = ww / (unsigned)mb;
        const unsigned el = ww - tr * (unsigned)mb;
        return r_obs + (((size_t)t0 + tr) * (size_t)n + env_start + el) * CFP_REC_BYTES;
    };
    const uint8_t* rec = rec_of(w);
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float x = 0.0f;                                   // padding of a widened row
        if (i0 + j >= total) {
        } else if (f < CFP_OBS_MAP) x = (float)rec[f];
        else if (f < CFP_OBS)
            x = __uint_as_float(reinterpret_cast<const uint32_t*>(rec + CFP_OBS_MAP)[f - CFP_OBS_MAP]);
        v[j] = x;
        if (++f == ld) { f = 0; rec = rec_of(++w); }      // past the last sample: not read
    }
    if (i0 + 4 <= total) {
        const f4 o = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(o, reinterpret_cast<f4*>(xobs + i0));
    } else {
        for (int j = 0; i0 + j < total; j++) xobs[i0 + j] = v[j];
    }
}

__global__ void k_add_bias(float* __restrict__ h, const float* __restrict__ b,
                           size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    h[idx] += b[idx & (CFP_HIDDEN - 1)];
}

__device__ __forceinline__ float sigmoid_fast(float z) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-z));
}

// Four hidden units per thread: every operand is one 16-byte access (the three
// gate rows of a column are 256 floats apart), all seven loads in flight before
// the first use; pre and x are read once (streamed past the caches).
__global__ __launch_bounds__(256) void k_mingru_epi_fwd(const f4* __restrict__ pre,
                                                        const f4* __restrict__ x,
                                                        f4* __restrict__ state,
                                                        f4* __restrict__ h_out,
                                                        f4* __restrict__ r_state_store,
                                                        const float* __restrict__ prev_terminals,
                                                        size_t total4) {
    constexpr int H4 = CFP_HIDDEN / 4;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total4) return;
    const int k4 = (int)(idx & (H4 - 1));
    const size_t col = idx / H4;
    const size_t o3 = col * (CFP_GRU / 4) + k4;
    const f4 zh = __builtin_nontemporal_load(pre + o3);
    const f4 zg = __builtin_nontemporal_load(pre + o3 + H4);
    const f4 zp = __builtin_nontemporal_load(pre + o3 + 2 * H4);
    const f4 xv = __builtin_nontemporal_load(x + idx);
    f4 st = state[idx];
    if (prev_terminals && prev_terminals[col] != 0.0f) st = f4{0.0f, 0.0f, 0.0f, 0.0f};
    if (r_state_store) __builtin_nontemporal_store(st, r_state_store + idx);
    f4 out, h;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float gh = zh[j] >= 0.0f ? zh[j] + 0.5f : sigmoid_fast(zh[j]);
        out[j] = st[j] + sigmoid_fast(zg[j]) * (gh - st[j]);
        const float p = sigmoid_fast(zp[j]);
        h[j] = p * out[j] + (1.0f - p) * xv[j];
    }
    h_out[idx] = h;
    state[idx] = out;
}

}  // namespace
}  // namespace cfp

using namespace cfp;

namespace cfp {
int launch_expand_obs(const uint8_t* r_obs, float* xobs, int t0, int count, int mb, int n,
                      int env_start, int ld, hipStream_t st) {
    if (ld % 4 == 0 && (reinterpret_cast<uintptr_t>(xobs) & 15u) == 0) {
        const size_t total4 = (size_t)count * (ld / 4);
        hipLaunchKernelGGL(k_expand_obs_v4, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0,
                           st, r_obs, reinterpret_cast<f4*>(xobs), t0, total4, mb, n, env_start,
                           ld / 4);
        CFP_HIP_TRY(hipGetLastError());
        return 0;
    }
    const size_t total = (size_t)count * ld;
    if (ld >= 4 && (reinterpret_cast<uintptr_t>(xobs) & 15u) == 0) {
        const size_t groups = (total + 3) / 4;
        hipLaunchKernelGGL(k_expand_obs_flat4, dim3((unsigned)((groups + 255) / 256)), dim3(256),
                           0, st, r_obs, xobs, t0, total, mb, n, env_start, ld);
        CFP_HIP_TRY(hipGetLastError());
        return 0;
    }
    hipLaunchKernelGGL(k_expand_obs, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       r_obs, xobs, t0, total, mb, n, env_start, ld);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}
}  // namespace cfp

// the 16-byte row pieces need every plane row to start on a 4-byte boundary
static bool rows16_ok(const uint8_t* m, const uint8_t* im, const uint8_t* lm, size_t env_stride,
                      size_t level_stride) {
    return ((reinterpret_cast<uintptr_t>(m) | reinterpret_cast<uintptr_t>(im) |
             reinterpret_cast<uintptr_t>(lm) | env_stride | level_stride) & 3u) == 0;
}

extern "C" {

int cfp_record_obs(const cfp_env_scalars* d_scalars, const uint8_t* d_map,
                   const uint8_t* d_item_map, const uint8_t* d_light_map,
                   size_t env_stride, size_t level_stride, uint8_t* d_rec_row,
                   int n, void* stream) {
    CFP_REQUIRE(d_scalars && d_map && d_item_map && d_light_map && d_rec_row,
                "cfp_record_obs: NULL argument");
    CFP_REQUIRE(n > 0, "cfp_record_obs: n must be positive (got %d)", n);
    CFP_REQUIRE((reinterpret_cast<uintptr_t>(d_rec_row) & 3u) == 0,
                "record rows must be 4-byte aligned");
    CFP_REQUIRE(env_stride >= (size_t)MAP * MAP,
                "cfp_record_obs: env_stride smaller than one 48x48 plane");
    if (rows16_ok(d_map, d_item_map, d_light_map, env_stride, level_stride))
        hipLaunchKernelGGL((k_record_obs<false, true>), dim3((n + kRecEnvsPerWg - 1) / kRecEnvsPerWg),
                           dim3(256), 0, (hipStream_t)stream, d_scalars, SoaArgs{}, RecWhich{}, d_map,
                           d_item_map, d_light_map, env_stride, level_stride, d_rec_row, n);
    else
        hipLaunchKernelGGL((k_record_obs<false, false>), dim3((n + kRecEnvsPerWg - 1) / kRecEnvsPerWg),
                           dim3(256), 0, (hipStream_t)stream, d_scalars, SoaArgs{}, RecWhich{}, d_map,
                           d_item_map, d_light_map, env_stride, level_stride, d_rec_row, n);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

static int record_obs_soa(const cfp_env_soa* soa, const uint8_t* d_map, const uint8_t* d_item_map,
                          const uint8_t* d_light_map, size_t env_stride, size_t level_stride,
                          const RecWhich& which, int items, uint8_t* d_rec_row, int n,
                          void* stream) {
    CFP_REQUIRE(soa && d_map && d_item_map && d_light_map && d_rec_row,
                "cfp_record_obs_soa: NULL argument");
    CFP_REQUIRE(n > 0 && items > 0, "cfp_record_obs_soa: nothing to record");
    CFP_REQUIRE((reinterpret_cast<uintptr_t>(d_rec_row) & 3u) == 0,
                "record rows must be 4-byte aligned");
    CFP_REQUIRE(env_stride >= (size_t)MAP * MAP,
                "cfp_record_obs_soa: env_stride smaller than one 48x48 plane");
    CFP_REQUIRE(soa->n_stride >= (size_t)n, "cfp_record_obs_soa: n_stride %zu below the env count %d",
                soa->n_stride, n);
    SoaArgs a;
    std::memcpy(&a, soa, sizeof(a));
    for (int i = 0; i < kSoaPtrs; i++)
        CFP_REQUIRE(a.p[i] != nullptr, "cfp_record_obs_soa: field array %d of the view is NULL", i);
    const bool rows16 = rows16_ok(d_map, d_item_map, d_light_map, env_stride, level_stride);
    const bool few = items <= kSoaFewItems;
    const dim3 grid((items + (few ? kSoaGatherFew : kSoaGather) - 1) / (few ? kSoaGatherFew : kSoaGather));
#define CFP_REC_SOA(R16, G)                                                                              \
    hipLaunchKernelGGL((k_record_obs<true, R16, G>), grid, dim3(256), 0, (hipStream_t)stream, nullptr, a, \
                       which, d_map, d_item_map, d_light_map, env_stride, level_stride, d_rec_row, n)
    if (rows16 && few) CFP_REC_SOA(true, kSoaGatherFew);
    else if (rows16) CFP_REC_SOA(true, kSoaGather);
    else if (few) CFP_REC_SOA(false, kSoaGatherFew);
    else CFP_REC_SOA(false, kSoaGather);
#undef CFP_REC_SOA
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_record_obs_soa(const cfp_env_soa* soa, const uint8_t* d_map, const uint8_t* d_item_map,
                       const uint8_t* d_light_map, size_t env_stride, size_t level_stride,
                       const uint8_t* d_skip, uint8_t* d_rec_row, int n, void* stream) {
    RecWhich w{};
    w.skip = d_skip;
    return record_obs_soa(soa, d_map, d_item_map, d_light_map, env_stride, level_stride, w, n,
                          d_rec_row, n, stream);
}

int cfp_record_obs_soa_list(const cfp_env_soa* soa, const uint8_t* d_map,
                            const uint8_t* d_item_map, const uint8_t* d_light_map,
                            size_t env_stride, size_t level_stride, const void* d_env_list,
                            size_t list_stride, const int* d_count, int max_count,
                            uint8_t* d_rec_row, int n, void* stream) {
    CFP_REQUIRE(d_env_list && d_count && list_stride >= 4 && list_stride % 4 == 0,
                "cfp_record_obs_soa_list: bad list (entries are int32, stride a multiple of 4)");
    CFP_REQUIRE(max_count > 0 && max_count <= n,
                "cfp_record_obs_soa_list: max_count must be in 1..n (got %d)", max_count);
    RecWhich w{};
    w.list = static_cast<const unsigned char*>(d_env_list);
    w.list_stride = list_stride;
    w.count = d_count;
    w.max_count = max_count;
    return record_obs_soa(soa, d_map, d_item_map, d_light_map, env_stride, level_stride, w,
                          max_count, d_rec_row, n, stream);
}

}  // extern "C"

int cfp::record_obs_soa_zero(const cfp_env_soa* soa, const uint8_t* d_map, const uint8_t* d_item_map,
                             const uint8_t* d_light_map, size_t env_stride, size_t level_stride,
                             uint8_t* d_rec_row, int n, int* d_zero, void* stream) {
    RecWhich w{};
    w.zero = d_zero;
    return record_obs_soa(soa, d_map, d_item_map, d_light_map, env_stride, level_stride, w, n,
                               d_rec_row, n, stream);
}

extern "C" {

int cfp_expand_obs(const uint8_t* d_r_obs, float* d_xobs, int t0, int count,
                   int mb, int n, int env_start, void* stream) {
    CFP_REQUIRE(d_r_obs && d_xobs && count > 0 && mb > 0 && n > 0 && t0 >= 0 &&
                    env_start >= 0 && env_start + mb <= n,
                "cfp_expand_obs: bad argument");
    CFP_REQUIRE((reinterpret_cast<uintptr_t>(d_r_obs) & 3u) == 0,
                "records must be 4-byte aligned");
    return launch_expand_obs(d_r_obs, d_xobs, t0, count, mb, n, env_start, CFP_OBS,
                             (hipStream_t)stream);
}

int cfp_add_bias(float* d_h, const float* d_b, int cols, void* stream) {
    CFP_REQUIRE(d_h && d_b && cols > 0, "cfp_add_bias: bad argument");
    const size_t total = (size_t)cols * CFP_HIDDEN;
    hipLaunchKernelGGL(k_add_bias, dim3((unsigned)((total + 255) / 256)),
                       dim3(256), 0, (hipStream_t)stream, d_h, d_b, total);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_mingru_epi_fwd(const float* d_pre, const float* d_x, float* d_state,
                       float* d_h_out, float* d_r_state_store,
                       const float* d_prev_terminals, int cols, void* stream) {
    CFP_REQUIRE(d_pre && d_x && d_state && d_h_out && cols > 0,
                "cfp_mingru_epi_fwd: bad argument");
    const uintptr_t all = reinterpret_cast<uintptr_t>(d_pre) | reinterpret_cast<uintptr_t>(d_x) |
                          reinterpret_cast<uintptr_t>(d_state) |
                          reinterpret_cast<uintptr_t>(d_h_out) |
                          reinterpret_cast<uintptr_t>(d_r_state_store);
    CFP_REQUIRE((all & 15u) == 0, "cfp_mingru_epi_fwd: buffers must be 16-byte aligned");
    const size_t total4 = (size_t)cols * (CFP_HIDDEN / 4);
    hipLaunchKernelGGL(k_mingru_epi_fwd, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, reinterpret_cast<const f4*>(d_pre),
                       reinterpret_cast<const f4*>(d_x), reinterpret_cast<f4*>(d_state),
                       reinterpret_cast<f4*>(d_h_out), reinterpret_cast<f4*>(d_r_state_store),
                       d_prev_terminals, total4);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // extern "C"
