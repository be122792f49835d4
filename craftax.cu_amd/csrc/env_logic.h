// One Craftax game step as a function of (hot scalars, storage), written once for the
// gfx950 kernel and for a host build of the same text (the host build is a checker's
// aid: it lets the step be compared with the compiled reference without a GPU).
//
// What is restated here is the reference's C specification of the step,
// craftax_gameplay_step_native (craftax_full.c:3798-3878) and the subsystems it calls
// (:4210-8225); each function cites its part.  The organisation is this library's own:
// the ~60 hot scalars of an env live in a register struct (`Hot`) for the whole step,
// achievements and growing-plant / chest flags are bit sets, block classes are 64-bit
// membership masks, recipes are one table walk per action, the spawn scan works on the
// 48-bit row bitmaps without building candidate lists, and everything that is indexed
// with a runtime index (mob slots, map cells, per-level words) goes through the storage
// object `S`, which the kernel backs with LDS and global arrays and the host build with
// a plain struct.
//
// Floating point: the reference is a gcc -ffast-math build whose GPU port reproduces it
// with strict per-operation fp32 and reciprocal multiplication where a literal divisor
// appears (craftax_full.cu:5163, 6991; Makefile:27 -fmad=false).  This text follows
// that: compile it with -ffp-contract=off.  Sites where the host build of the checker
// here was found to fuse are marked FUSED and spelled with fmaf.
#pragma once

#include <stdint.h>

#if defined(__clang__)
// strict per-operation fp32 from here to the end of the translation unit (gcc: -ffp-contract=off)
#pragma clang fp contract(off)
#endif

#if defined(__HIPCC__)
#define CFE_FN __host__ __device__ __forceinline__
#else
#define CFE_FN inline
#endif

namespace cfenv {

constexpr int kMap = 48;
constexpr int kLevels = 9;
constexpr int kNumActions = 43;
constexpr int kMaxTimesteps = 100000;
constexpr int kDespawn = 14;          // CRAFTAX_MOB_DESPAWN_DISTANCE, craftax_full.c:2977
constexpr int kKillsToClear = 8;      // :2978
constexpr int kPlants = 10;           // :2972

// ---- ids (craftax_full.c:2983-3163) ------------------------------------------------
enum Block : int {
    B_INVALID = 0, B_OOB = 1, B_GRASS = 2, B_WATER = 3, B_STONE = 4, B_TREE = 5, B_WOOD = 6,
    B_PATH = 7, B_COAL = 8, B_IRON = 9, B_DIAMOND = 10, B_TABLE = 11, B_FURNACE = 12,
    B_SAND = 13, B_LAVA = 14, B_PLANT = 15, B_RIPE_PLANT = 16, B_WALL = 17, B_DARKNESS = 18,
    B_WALL_MOSS = 19, B_STALAGMITE = 20, B_SAPPHIRE = 21, B_RUBY = 22, B_CHEST = 23,
    B_FOUNTAIN = 24, B_FIRE_GRASS = 25, B_ICE_GRASS = 26, B_GRAVEL = 27, B_FIRE_TREE = 28,
    B_ICE_SHRUB = 29, B_ENCH_FIRE = 30, B_ENCH_ICE = 31, B_NECROMANCER = 32, B_GRAVE = 33,
    B_GRAVE2 = 34, B_GRAVE3 = 35, B_NECRO_VULNERABLE = 36,
};
enum Item : int { I_NONE = 0, I_TORCH = 1, I_LADDER_DOWN = 2, I_LADDER_UP = 3 };
enum Action : int {
    A_NOOP = 0, A_LEFT = 1, A_RIGHT = 2, A_UP = 3, A_DOWN = 4, A_DO = 5, A_SLEEP = 6,
    A_PLACE_STONE = 7, A_PLACE_TABLE = 8, A_PLACE_FURNACE = 9, A_PLACE_PLANT = 10,
    A_MAKE_WOOD_PICKAXE = 11, A_MAKE_STONE_PICKAXE = 12, A_MAKE_IRON_PICKAXE = 13,
    A_MAKE_WOOD_SWORD = 14, A_MAKE_STONE_SWORD = 15, A_MAKE_IRON_SWORD = 16, A_REST = 17,
    A_DESCEND = 18, A_ASCEND = 19, A_MAKE_DIAMOND_PICKAXE = 20, A_MAKE_DIAMOND_SWORD = 21,
    A_MAKE_IRON_ARMOUR = 22, A_MAKE_DIAMOND_ARMOUR = 23, A_SHOOT_ARROW = 24, A_MAKE_ARROW = 25,
    A_CAST_FIREBALL = 26, A_CAST_ICEBALL = 27, A_PLACE_TORCH = 28, A_DRINK_POTION_RED = 29,
    A_DRINK_POTION_YELLOW = 34, A_READ_BOOK = 35, A_ENCHANT_SWORD = 36, A_ENCHANT_ARMOUR = 37,
    A_MAKE_TORCH = 38, A_LEVEL_UP_DEX = 39, A_LEVEL_UP_STR = 40, A_LEVEL_UP_INT = 41,
    A_ENCHANT_BOW = 42,
};
enum Ach : int {
    ACH_COLLECT_WOOD = 0, ACH_PLACE_TABLE = 1, ACH_EAT_COW = 2, ACH_COLLECT_SAPLING = 3,
    ACH_COLLECT_DRINK = 4, ACH_MAKE_WOOD_PICKAXE = 5, ACH_MAKE_WOOD_SWORD = 6,
    ACH_PLACE_PLANT = 7, ACH_DEFEAT_ZOMBIE = 8, ACH_COLLECT_STONE = 9, ACH_PLACE_STONE = 10,
    ACH_EAT_PLANT = 11, ACH_DEFEAT_SKELETON = 12, ACH_MAKE_STONE_PICKAXE = 13,
    ACH_MAKE_STONE_SWORD = 14, ACH_WAKE_UP = 15, ACH_PLACE_FURNACE = 16, ACH_COLLECT_COAL = 17,
    ACH_COLLECT_IRON = 18, ACH_COLLECT_DIAMOND = 19, ACH_MAKE_IRON_PICKAXE = 20,
    ACH_MAKE_IRON_SWORD = 21, ACH_MAKE_ARROW = 22, ACH_MAKE_TORCH = 23, ACH_PLACE_TORCH = 24,
    ACH_MAKE_DIAMOND_SWORD = 25, ACH_MAKE_IRON_ARMOUR = 26, ACH_MAKE_DIAMOND_ARMOUR = 27,
    ACH_ENTER_GNOMISH_MINES = 28, ACH_ENTER_DUNGEON = 29, ACH_ENTER_SEWERS = 30,
    ACH_ENTER_VAULT = 31, ACH_ENTER_TROLL_MINES = 32, ACH_ENTER_FIRE_REALM = 33,
    ACH_ENTER_ICE_REALM = 34, ACH_ENTER_GRAVEYARD = 35, ACH_DEFEAT_GNOME_WARRIOR = 36,
    ACH_DEFEAT_GNOME_ARCHER = 37, ACH_DEFEAT_ORC_SOLIDER = 38, ACH_DEFEAT_ORC_MAGE = 39,
    ACH_DEFEAT_LIZARD = 40, ACH_DEFEAT_KOBOLD = 41, ACH_DEFEAT_TROLL = 42,
    ACH_DEFEAT_DEEP_THING = 43, ACH_DEFEAT_PIGMAN = 44, ACH_DEFEAT_FIRE_ELEMENTAL = 45,
    ACH_DEFEAT_FROST_TROLL = 46, ACH_DEFEAT_ICE_ELEMENTAL = 47, ACH_DAMAGE_NECROMANCER = 48,
    ACH_DEFEAT_NECROMANCER = 49, ACH_EAT_BAT = 50, ACH_EAT_SNAIL = 51, ACH_FIND_BOW = 52,
    ACH_FIRE_BOW = 53, ACH_COLLECT_SAPPHIRE = 54, ACH_LEARN_FIREBALL = 55,
    ACH_CAST_FIREBALL = 56, ACH_LEARN_ICEBALL = 57, ACH_CAST_ICEBALL = 58,
    ACH_COLLECT_RUBY = 59, ACH_MAKE_DIAMOND_PICKAXE = 60, ACH_OPEN_CHEST = 61,
    ACH_DRINK_POTION = 62, ACH_ENCHANT_SWORD = 63, ACH_ENCHANT_ARMOUR = 64,
    ACH_DEFEAT_KNIGHT = 65, ACH_DEFEAT_ARCHER = 66,
};
// Storage order of the five mob pools (the reference's device arrays, craftax_full.cu:706)
// and the class ids the game's tables are indexed with (craftax_full.c:3077-3082).
enum Pool : int { P_MELEE = 0, P_PASSIVE = 1, P_RANGED = 2, P_MOB_PROJ = 3, P_PLAYER_PROJ = 4 };
enum MobClass : int { MC_PASSIVE = 0, MC_MELEE = 1, MC_RANGED = 2, MC_PROJECTILE = 3 };
// spawn bit planes: which blocks a mob may appear on (craftax_full.c:3284-3303)
enum SpawnKind : int { SK_ALL = 0, SK_GRAVE = 1, SK_WATER = 2 };

constexpr uint64_t bit64(int b) { return 1ull << b; }
constexpr uint64_t kSolidBlocks =  // craftax_step_is_solid_block, craftax_full.c:4288-4317
    bit64(B_STONE) | bit64(B_TREE) | bit64(B_COAL) | bit64(B_IRON) | bit64(B_DIAMOND) |
    bit64(B_TABLE) | bit64(B_FURNACE) | bit64(B_PLANT) | bit64(B_RIPE_PLANT) | bit64(B_WALL) |
    bit64(B_WALL_MOSS) | bit64(B_STALAGMITE) | bit64(B_RUBY) | bit64(B_SAPPHIRE) |
    bit64(B_CHEST) | bit64(B_FOUNTAIN) | bit64(B_FIRE_TREE) | bit64(B_ENCH_FIRE) |
    bit64(B_ENCH_ICE) | bit64(B_GRAVE) | bit64(B_GRAVE2) | bit64(B_GRAVE3) | bit64(B_NECROMANCER);
constexpr uint64_t kSpawnAll = bit64(B_GRASS) | bit64(B_PATH) | bit64(B_FIRE_GRASS) | bit64(B_ICE_GRASS);
constexpr uint64_t kSpawnGrave = bit64(B_GRAVE) | bit64(B_GRAVE2) | bit64(B_GRAVE3);
constexpr uint64_t kSpawnWater = bit64(B_WATER);
constexpr uint64_t kItemGround =  // craftax_crafting_can_place_item, :5002-5013
    bit64(B_GRASS) | bit64(B_SAND) | bit64(B_PATH) | bit64(B_FIRE_GRASS) | bit64(B_ICE_GRASS);
constexpr uint64_t kRowMask = (1ull << kMap) - 1;

CFE_FN bool in_set(uint64_t set, int block) { return ((set >> (block & 63)) & 1ull) != 0; }
CFE_FN bool is_solid(int block) { return in_set(kSolidBlocks, block); }
CFE_FN uint64_t spawn_set(int kind) {
    return kind == SK_ALL ? kSpawnAll : kind == SK_GRAVE ? kSpawnGrave : kSpawnWater;
}
CFE_FN bool on_map(int r, int c) { return (unsigned)r < (unsigned)kMap && (unsigned)c < (unsigned)kMap; }
// jnp-style index: negative wraps once, then clamps (craftax_step_jax_index, :4210-4221)
CFE_FN int wrap_clamp(int i, int size) {
    if (i < 0) i += size;
    return i < 0 ? 0 : (i >= size ? size - 1 : i);
}
// scatter index: negative wraps once, anything else outside is dropped (:5922-5932, 6279-6289)
CFE_FN bool wrap_drop(int i, int size, int& out) {
    if (i < -size || i >= size) return false;
    out = i < 0 ? i + size : i;
    return true;
}
CFE_FN int imin(int a, int b) { return a < b ? a : b; }
CFE_FN int imax(int a, int b) { return a > b ? a : b; }
CFE_FN int iabs(int a) { return a < 0 ? -a : a; }
CFE_FN int isign(int a) { return a < 0 ? -1 : (a > 0 ? 1 : 0); }

// ---- the env's generator (craftax_full.c:27-142, 1079-1108): a 64-bit LCG walk whose
// states are the keys, a murmur3 finalizer for the draws ---------------------------------
CFE_FN uint64_t lcg(uint64_t s) { return s * 6364136223846793005ull + 1ull; }
// craftax_threefry_split(rng, &rng, &draw): advances rng one LCG step, the draw key is the
// step after it
CFE_FN uint64_t next_key(uint64_t& rng) {
    rng = lcg(rng);
    return lcg(rng);
}
CFE_FN uint64_t fmix64(uint64_t x) {
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}
CFE_FN uint32_t draw_u32(uint64_t key) {
    const uint64_t h = fmix64(key);
    return (uint32_t)h ^ (uint32_t)(h >> 32);
}
CFE_FN float bits_to_float(uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(b);
#else
    float f;
    __builtin_memcpy(&f, &b, 4);
    return f;
#endif
}
CFE_FN float draw_unit(uint64_t key) {  // [0, 1) on the 23-bit grid
    return bits_to_float((draw_u32(key) >> 9) | 0x3F800000u) - 1.0f;
}
CFE_FN int draw_int(uint64_t key, int lo, int hi) {  // [lo, hi)
    const uint32_t span = (uint32_t)hi > (uint32_t)lo ? (uint32_t)hi - (uint32_t)lo : 1u;
    if ((span & (span - 1)) == 0) return (int)((uint32_t)lo + (draw_u32(key) & (span - 1)));
    const uint64_t h = fmix64(key);
    return (int)((uint32_t)lo + (uint32_t)(((h >> 32) * (uint64_t)span) >> 32));
}
// craftax_medium_choice_weighted (:5210-5229) for up to five weights
template <int N>
CFE_FN int draw_weighted(uint64_t key, const float (&w)[N]) {
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < N; i++) total += w[i];
    const float draw = total * (1.0f - draw_unit(key));
    float cum = 0.0f;
    int pick = N - 1;
    bool found = false;
#pragma unroll
    for (int i = 0; i < N; i++) {
        cum += w[i];
        if (!found && cum >= draw) {
            pick = i;
            found = true;
        }
    }
    return pick;
}

// ---- hot scalars: one env's registers for the step ---------------------------------------
struct Hot {
    int32_t pr, pc, level, dir;
    float health;
    int32_t food, drink, energy, mana;
    int32_t sleeping, resting;
    float recover, hunger, thirst, fatigue, recover_mana;
    int32_t xp, dex, str, intel;
    int32_t wood, stone, coal, iron, diamond, sapling, pickaxe, sword, bow, arrows;
    int32_t armour[4];
    int32_t torches, ruby, sapphire;
    int32_t potions[6];
    int32_t books;
    int32_t spell[2];
    int32_t sword_ench, bow_ench;
    int32_t armour_ench[4];
    int32_t boss_progress, boss_timer;
    float light_level;
    int32_t timestep;
    uint32_t ach[3];        // bit a of the set = achievements[a]
    uint32_t plant_mask;    // bit i = growing_plants_mask[i]
};

// An empty asm the value passes through.  Reading element i of a small array of the register
// struct is a chain of selects over all its elements; the optimiser would rewrite a select of
// two loads as one load from a selected address, and that runtime address keeps the whole
// struct in (scratch) memory.  A value that went through here is no longer a load.
CFE_FN int opaque(int x) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm("" : "+v"(x));
#else
    asm("" : "+r"(x));
#endif
    return x;
}
// (no runtime index into the register struct: a select per word)
CFE_FN void unlock_if(Hot& h, int a, bool c) {
    const uint32_t bit = (uint32_t)c << (a & 31);
    const int w = a >> 5;
    h.ach[0] |= w == 0 ? bit : 0u;
    h.ach[1] |= w == 1 ? bit : 0u;
    h.ach[2] |= w == 2 ? bit : 0u;
}
CFE_FN void unlock(Hot& h, int a) { unlock_if(h, a, true); }
CFE_FN bool has(const Hot& h, int a) {
    const int w = a >> 5;
    const uint32_t word = (uint32_t)(w == 0 ? opaque((int)h.ach[0]) : (w == 1 ? opaque((int)h.ach[1]) : opaque((int)h.ach[2])));
    return (word >> (a & 31)) & 1u;
}
template <int N>
CFE_FN int pick(const int32_t (&a)[N], int i) {
    // prvalues on both arms: a conditional between two lvalues is an lvalue, i.e. a select of
    // addresses, which keeps the whole register struct in memory
    int v = opaque(a[0]);
#pragma unroll
    for (int k = 1; k < N; k++) v = (i == k) ? opaque(a[k]) : v;
    return v;
}
template <int N>
CFE_FN void put(int32_t (&a)[N], int i, int v) {
#pragma unroll
    for (int k = 0; k < N; k++) a[k] = (i == k) ? v : opaque(a[k]);
}

CFE_FN int max_health(const Hot& h) { return 8 + h.str; }
CFE_FN int max_food(const Hot& h) { return 7 + 2 * h.dex; }   // food, drink and energy alike
CFE_FN int max_mana(const Hot& h) { return 6 + 3 * h.intel; }
CFE_FN bool at_boss(const Hot& h) { return h.level == kLevels - 1; }

struct Vec2 {
    int r, c;
};
// craftax_step_direction (:4273-4286): 1 left, 2 right, 3 up, 4 down, else none
CFE_FN Vec2 dir_vec(int a) {
    return Vec2{a == A_UP ? -1 : (a == A_DOWN ? 1 : 0), a == A_LEFT ? -1 : (a == A_RIGHT ? 1 : 0)};
}

// ---- tables --------------------------------------------------------------------------
// mob defence against (physical, fire, ice) by [type][game class] (:5659-5719); only five
// entries are non-zero
CFE_FN float mob_defence(int type, int mc, int comp) {
    type = wrap_clamp(type, 8);
    if (mc != MC_MELEE && mc != MC_RANGED) return 0.0f;
    if (type == 4) return comp == 0 ? 0.5f : 0.0f;
    if (type == 5) return (mc == MC_MELEE && comp == 0) ? 0.2f : 0.0f;
    if (type == 6) return comp == 0 ? 0.9f : (comp == 1 ? 1.0f : 0.0f);
    if (type == 7) return comp == 0 ? 0.9f : (comp == 2 ? 1.0f : 0.0f);
    return 0.0f;
}
// achievement for killing a mob of [game class][type] (:5721-5761)
CFE_FN int kill_achievement(int mc, int type) {
    type = wrap_clamp(type, 8);
    mc = wrap_clamp(mc, 3);
    if (mc == MC_PASSIVE) return type == 0 ? ACH_EAT_COW : type == 1 ? ACH_EAT_BAT : type == 2 ? ACH_EAT_SNAIL : 0;
    const uint64_t melee = (uint64_t)ACH_DEFEAT_ZOMBIE | (uint64_t)ACH_DEFEAT_GNOME_WARRIOR << 8 |
                           (uint64_t)ACH_DEFEAT_ORC_SOLIDER << 16 | (uint64_t)ACH_DEFEAT_LIZARD << 24 |
                           (uint64_t)ACH_DEFEAT_KNIGHT << 32 | (uint64_t)ACH_DEFEAT_TROLL << 40 |
                           (uint64_t)ACH_DEFEAT_PIGMAN << 48 | (uint64_t)ACH_DEFEAT_FROST_TROLL << 56;
    const uint64_t ranged = (uint64_t)ACH_DEFEAT_SKELETON | (uint64_t)ACH_DEFEAT_GNOME_ARCHER << 8 |
                            (uint64_t)ACH_DEFEAT_ORC_MAGE << 16 | (uint64_t)ACH_DEFEAT_KOBOLD << 24 |
                            (uint64_t)ACH_DEFEAT_ARCHER << 32 | (uint64_t)ACH_DEFEAT_DEEP_THING << 40 |
                            (uint64_t)ACH_DEFEAT_FIRE_ELEMENTAL << 48 | (uint64_t)ACH_DEFEAT_ICE_ELEMENTAL << 56;
    return (int)(((mc == MC_MELEE ? melee : ranged) >> (8 * type)) & 0xff);
}
// damage a mob deals as (physical, fire, ice) by [type][game class] (:6423-6487); only the
// melee and projectile classes deal any, one nibble per component
CFE_FN void mob_damage(int type, int mc, float (&d)[3]) {
    type = wrap_clamp(type, 8);
    //                         type:   7      6      5      4      3      2      1      0
    const uint32_t melee_p = 0x43665342u, melee_f = 0x05100000u, melee_i = 0x50100000u;
    const uint32_t proj_p = 0x43450042u, proj_f = 0x05300300u, proj_i = 0x50303000u;
    const int sh = 4 * type;
    if (mc == MC_MELEE) {
        d[0] = (float)((melee_p >> sh) & 15u);
        d[1] = (float)((melee_f >> sh) & 15u);
        d[2] = (float)((melee_i >> sh) & 15u);
    } else if (mc == MC_PROJECTILE) {
        d[0] = (float)((proj_p >> sh) & 15u);
        d[1] = (float)((proj_f >> sh) & 15u);
        d[2] = (float)((proj_i >> sh) & 15u);
    } else {
        d[0] = d[1] = d[2] = 0.0f;
    }
}
// what a mob of [type][game class] cannot stand on: bit 0 ground, bit 1 water, bit 2 lava
// (:6489-6553)
CFE_FN int mob_collision(int type, int mc) {
    type = wrap_clamp(type, 8);
    if (mc == MC_PASSIVE) return type == 1 ? 0 : 6;
    if (mc == MC_MELEE) return type == 3 ? 4 : 6;
    if (mc == MC_RANGED) return type == 5 ? 5 : (type >= 6 ? 0 : 6);
    return 0;
}
CFE_FN int ranged_projectile(int type) {  // :6555-6573
    type = wrap_clamp(type, 8);
    //                      type: 7 6 5 4 3 2 1 0
    return (int)((0x76541200u >> (4 * type)) & 15u);
}
CFE_FN int floor_mob_type(int floor, int mc) {  // :7544-7554, [level][passive, melee, ranged]
    floor = wrap_clamp(floor, kLevels);
    mc = wrap_clamp(mc, 3);
    // level:                                   8     7     6     5     4     3     2     1     0
    const uint64_t passive = 0x011122120ull, melee = 0x076543120ull, ranged = 0x076543120ull;
    return (int)(((mc == MC_PASSIVE ? passive : mc == MC_MELEE ? melee : ranged) >> (4 * floor)) & 15u);
}
CFE_FN float mob_health(int type, int mc) {  // :7575-7587
    type = wrap_clamp(type, 8);
    mc = wrap_clamp(mc, 4);
    if (mc == MC_PASSIVE) return type == 0 ? 3.0f : type == 1 ? 4.0f : type == 2 ? 6.0f : type == 3 ? 8.0f : 0.0f;
    if (mc == MC_MELEE) {
        const float v[8] = {5.0f, 7.0f, 9.0f, 11.0f, 12.0f, 20.0f, 20.0f, 24.0f};
        float r = v[0];
#pragma unroll
        for (int k = 1; k < 8; k++) r = type == k ? v[k] : r;
        return r;
    }
    if (mc == MC_RANGED) {
        const float v[8] = {3.0f, 5.0f, 6.0f, 8.0f, 12.0f, 4.0f, 14.0f, 16.0f};
        float r = v[0];
#pragma unroll
        for (int k = 1; k < 8; k++) r = type == k ? v[k] : r;
        return r;
    }
    return 0.0f;
}
// torch light by squared distance (:5015-5028): the table's entry at (dr, dc) is
// max(0, 1 - sqrt(dr^2 + dc^2) / 5) as the reference spells it out digit by digit
CFE_FN float torch_light(int dr, int dc) {
    const int d2 = dr * dr + dc * dc;
    switch (d2) {
        case 0: return 1.0f;
        case 1: return 0.8f;
        case 2: return 0.71715724f;
        case 4: return 0.6f;
        case 5: return 0.55278647f;
        case 8: return 0.43431455f;
        case 9: return 0.39999998f;
        case 10: return 0.36754447f;
        case 13: return 0.27888972f;
        case 16: return 0.19999999f;
        case 17: return 0.17537886f;
        case 18: return 0.15147191f;
        case 20: return 0.10557288f;
        default: return 0.0f;
    }
}
CFE_FN float achievement_reward(int a) {  // CRAFTAX_ACHIEVEMENT_REWARD_MAP, :3490-3500
    if (a < 25) return 1.0f;
    if (a < 30) return 3.0f;
    if (a < 33) return 5.0f;
    if (a < 36) return 8.0f;
    if (a < 40) return 3.0f;
    if (a < 44) return 5.0f;
    if (a < 50) return 8.0f;
    if (a < 55) return 3.0f;
    if (a < 59) return 5.0f;
    if (a < 63) return 3.0f;
    return 5.0f;
}

// ---- storage interface -------------------------------------------------------------------
// A storage object S provides (level = the level the call names; mob accessors work on
// the level the storage was opened at, i.e. the player's level after change_floor):
//   int  blk(l, r, c) / put_blk_raw(l, r, c, b); int item(l, r, c) / put_item; int lum(l, r, c) / put_lum
//   uint64_t mobrow(l, r) / put_mobrow(l, r, v); uint64_t spawnrow(kind, l, r) / put_spawnrow
//   int m_row(p, i), m_col(p, i), m_cd(p, i), m_type(p, i); bool m_mask(p, i); float m_hp(p, i)
//   set_m_pos(p, i, r, c), set_m_cd, set_m_type, set_m_mask, set_m_hp
//   int pd_r(p, i), pd_c(p, i) / set_pd(p, i, r, c)      (p = P_MOB_PROJ or P_PLAYER_PROJ)
//   int kills(l) / set_kills; bool chest(l) / set_chest(l); int ladder_down(l, axis), ladder_up(l, axis)
//   int potion_effect(i); int plant_r(i), plant_c(i), plant_age(i) / set_plant(i, r, c), set_plant_age(i, a)
//   void open_level(l): called once per step when the step's level is known
//   float light_at(timestep)
//   void stamp(k): phase boundary k of the step passed (a hook for timing builds; empty otherwise)

// craftax_set_map_block (:3325-3334): the block and its three spawn bits
template <class S>
CFE_FN void set_block(S& s, int l, int r, int c, int b) {
    const int old = s.blk(l, r, c);
    s.put_blk_raw(l, r, c, b);
    const uint64_t bit = 1ull << c;
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const bool was = in_set(spawn_set(k), old), is = in_set(spawn_set(k), b);
        if (was != is) {
            const uint64_t row = s.spawnrow(k, l, r);
            s.put_spawnrow(k, l, r, is ? (row | bit) : (row & ~bit));
        }
    }
}

// The level's mob bitmap is, at every point of a step, the set of cells of the live melee,
// passive and ranged mobs of that level (a mob's bit is set where it appears, moved with it and
// cleared where it dies or despawns; no two of them share a cell).  The step therefore asks
// the mob slots -- which the storage holds close by -- where it needs occupancy, and writes a
// bitmap row as what the slots say; it never waits for a bitmap row from memory.
// The eight movers' cells as one word each (row in the high half, column in the low half; a
// dead slot holds a cell no query names), read from the slots with no branch between the
// reads, so that they travel together, and kept in registers while the mobs move.
struct MoverKeys {
    uint32_t key[8];
};
constexpr uint32_t kNoCell = 0x80008000u;
CFE_FN uint32_t cell_key(int r, int c) { return ((uint32_t)r << 16) | ((uint32_t)c & 0xffffu); }
CFE_FN int mover_pool(int k) { return k < 3 ? P_MELEE : (k < 6 ? P_PASSIVE : P_RANGED); }
CFE_FN int mover_slot(int k) { return k < 6 ? k % 3 : k - 6; }
template <class S>
CFE_FN MoverKeys load_mover_keys(S& s) {
    MoverKeys m;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int p = mover_pool(k), i = mover_slot(k);
        const uint32_t cell = cell_key(s.m_row(p, i), s.m_col(p, i));
        m.key[k] = s.m_mask(p, i) ? cell : kNoCell;
    }
    return m;
}
CFE_FN bool keys_at(const MoverKeys& m, int r, int c) {
    const uint32_t want = cell_key(r, c);
    bool any = false;
#pragma unroll
    for (int k = 0; k < 8; k++) any = any | (m.key[k] == want);
    return any;
}
CFE_FN uint64_t keys_row(const MoverKeys& m, int row) {
    uint64_t bits = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) bits |= (m.key[k] >> 16) == (uint32_t)row ? 1ull << (m.key[k] & 63u) : 0ull;
    return bits & kRowMask;
}
template <class S>
CFE_FN bool mover_at(S& s, int r, int c) { return keys_at(load_mover_keys(s), r, c); }
template <class S>
CFE_FN uint64_t movers_row(S& s, int row) { return keys_row(load_mover_keys(s), row); }

// craftax_step_is_in_mob (:4319-4330): the bitmap's bit at the clamped cell, or the player
template <class S>
CFE_FN bool mob_or_player_at(S& s, const Hot& h, int r, int c) {
    return mover_at(s, wrap_clamp(r, kMap), wrap_clamp(c, kMap)) || (h.pr == r && h.pc == c);
}

// craftax_move_player_native (:4332-4379)
template <class S>
CFE_FN void move_player(S& s, Hot& h, int action) {
    const Vec2 d = dir_vec(action);
    if (d.r == 0 && d.c == 0) return;
    const int r = h.pr + d.r, c = h.pc + d.c;
    bool ok = on_map(r, c);
    if (ok) {
        const int b = s.blk(wrap_clamp(h.level, kLevels), r, c);
        ok = !mob_or_player_at(s, h, r, c) && !is_solid(b) && b != B_WATER && b != B_LAVA;
    }
    if (ok) {
        h.pr = r;
        h.pc = c;
    }
    h.dir = action;
}

// craftax_change_floor_native (:5460-5517); floors are all present (no lazy generation)
template <class S>
CFE_FN void change_floor(S& s, Hot& h, int action) {
    const int l = wrap_clamp(h.level, kLevels);
    bool down = false, up = false;
    if (action == A_DESCEND || action == A_ASCEND) {
        const int it = s.item(l, wrap_clamp(h.pr, kMap), wrap_clamp(h.pc, kMap));
        down = action == A_DESCEND && it == I_LADDER_DOWN && s.kills(l) >= kKillsToClear && h.level < kLevels - 1;
        up = action == A_ASCEND && it == I_LADDER_UP && h.level > 0;
    }
    const int new_level = h.level + (int)down - (int)up;
    static_assert(ACH_ENTER_DUNGEON == 29 && ACH_ENTER_GNOMISH_MINES == 28, "enter-floor ids");
    // :5282-5303: floors 1..8 -> dungeon, gnomish mines, sewers, vault, troll mines, fire, ice, graveyard
    const int nl = wrap_clamp(new_level, kLevels);
    const int ach = nl == 0 ? ACH_COLLECT_WOOD : nl == 1 ? ACH_ENTER_DUNGEON : nl == 2 ? ACH_ENTER_GNOMISH_MINES
                                                                                       : ACH_ENTER_SEWERS + (nl - 3);
    const bool first_visit = new_level != 0 && !has(h, ach);
    if (down) {
        const int ll = wrap_clamp(h.level + 1, kLevels);
        h.pr = s.ladder_up(ll, 0);
        h.pc = s.ladder_up(ll, 1);
    } else if (up) {
        const int ll = wrap_clamp(h.level - 1, kLevels);
        h.pr = s.ladder_down(ll, 0);
        h.pc = s.ladder_down(ll, 1);
    }
    h.level = new_level;
    unlock_if(h, ach, new_level != 0);
    h.xp += (int)first_visit;
}

// craftax_crafting_is_near_block (:4768-4799): bit 0 = a crafting table, bit 1 = a furnace
// among the eight neighbours
template <class S>
CFE_FN int nearby_stations(S& s, const Hot& h) {
    const int l = wrap_clamp(h.level, kLevels);
    int found = 0;
    for (int dr = -1; dr <= 1; dr++)
        for (int dc = -1; dc <= 1; dc++) {
            if (dr == 0 && dc == 0) continue;
            const int r = h.pr + dr, c = h.pc + dc;
            if (!on_map(r, c)) continue;
            const int b = s.blk(l, r, c);
            found |= (b == B_TABLE ? 1 : 0) | (b == B_FURNACE ? 2 : 0);
        }
    return found;
}

// first armour slot below `threshold`, -1 if none (craftax_crafting_first_armour_below)
CFE_FN int first_armour_below(const Hot& h, int threshold) {
    int first = -1;
#pragma unroll
    for (int i = 3; i >= 0; i--) first = h.armour[i] < threshold ? i : first;
    return first;
}

// craftax_do_crafting_native (:4816-5000).  One action fires at most one recipe, so the
// reference's chain of independent recipes is a dispatch on the action.
template <class S>
CFE_FN void craft(S& s, Hot& h, int action) {
    const bool tool = (action >= A_MAKE_WOOD_PICKAXE && action <= A_MAKE_IRON_SWORD) ||
                      (action >= A_MAKE_DIAMOND_PICKAXE && action <= A_MAKE_DIAMOND_ARMOUR) ||
                      action == A_MAKE_ARROW || action == A_MAKE_TORCH;
    if (!tool) return;
    const int near = nearby_stations(s, h);
    const bool table = near & 1, furnace = near & 2;
    if (!table) return;
    // tiers: 1 wood, 2 stone, 3 iron, 4 diamond; the diamond tier needs 3 (pickaxe) or 2 (sword)
    int tier = 0;
    bool is_pickaxe = false;
    switch (action) {
        case A_MAKE_WOOD_PICKAXE: tier = 1; is_pickaxe = true; break;
        case A_MAKE_STONE_PICKAXE: tier = 2; is_pickaxe = true; break;
        case A_MAKE_IRON_PICKAXE: tier = 3; is_pickaxe = true; break;
        case A_MAKE_DIAMOND_PICKAXE: tier = 4; is_pickaxe = true; break;
        case A_MAKE_WOOD_SWORD: tier = 1; break;
        case A_MAKE_STONE_SWORD: tier = 2; break;
        case A_MAKE_IRON_SWORD: tier = 3; break;
        case A_MAKE_DIAMOND_SWORD: tier = 4; break;
        default: break;
    }
    if (tier != 0) {
        const int have = is_pickaxe ? opaque(h.pickaxe) : opaque(h.sword);
        const int diamonds = is_pickaxe ? 3 : 2;
        bool ok = have < tier && h.wood >= 1;
        if (tier == 2) ok = ok && h.stone >= 1;
        if (tier == 3) ok = ok && h.stone >= 1 && h.iron >= 1 && h.coal >= 1 && furnace;
        if (tier == 4) ok = ok && h.diamond >= diamonds;
        if (!ok) return;
        h.wood -= 1;
        if (tier == 2 || tier == 3) h.stone -= 1;
        if (tier == 3) {
            h.iron -= 1;
            h.coal -= 1;
        }
        if (tier == 4) h.diamond -= diamonds;
        if (is_pickaxe) h.pickaxe = tier; else h.sword = tier;
        return;
    }
    if (action == A_MAKE_IRON_ARMOUR) {
        const int slot = first_armour_below(h, 1);
        if (slot >= 0 && h.iron >= 3 && h.coal >= 3 && furnace) {
            h.iron -= 3;
            h.coal -= 3;
            put(h.armour, slot, 1);
            unlock(h, ACH_MAKE_IRON_ARMOUR);
        }
    } else if (action == A_MAKE_DIAMOND_ARMOUR) {
        const int slot = first_armour_below(h, 2);
        if (slot >= 0 && h.diamond >= 3) {
            h.diamond -= 3;
            put(h.armour, slot, 2);
            unlock(h, ACH_MAKE_DIAMOND_ARMOUR);
        }
    } else if (action == A_MAKE_ARROW) {
        if (h.stone >= 1 && h.wood >= 1 && h.arrows < 99) {
            h.wood -= 1;
            h.stone -= 1;
            h.arrows += 2;
        }
    } else if (action == A_MAKE_TORCH) {
        if (h.coal >= 1 && h.wood >= 1 && h.torches < 99) {
            h.wood -= 1;
            h.coal -= 1;
            h.torches += 4;
        }
    }
}

// damage of the player's own hit as (physical, fire, ice) (:5763-5783)
CFE_FN void player_damage(const Hot& h, float (&d)[3]) {
    const int tier = wrap_clamp(h.sword, 5);
    float phys = tier == 0 ? 1.0f : tier == 1 ? 2.0f : tier == 2 ? 3.0f : tier == 3 ? 5.0f : 8.0f;
    float fire = phys * (float)(h.sword_ench == 1) * 0.5f;
    float ice = phys * (float)(h.sword_ench == 2) * 0.5f;
    phys *= 1.0f + 0.25f * (float)(h.str - 1);
    const float magic = 1.0f + 0.05f * (float)(h.intel - 1);
    fire *= magic;
    ice *= magic;
    d[0] = phys;
    d[1] = fire;
    d[2] = ice;
}

struct Hit {
    bool attacked, killed;
};
// craftax_do_action_attack_mobs3 / _mobs2 (:5820-5920) on one pool of the current level.
// The reference refreshes the pool's masks on every level; on the other levels that is the
// identity as long as no masked mob has health <= 0 there, which holds for every state the
// game produces (health only falls in these two functions, and each refreshes).
template <class S>
CFE_FN Hit hit_pool(S& s, Hot& h, int pool, int slots, int mc, int r, int c, const float (&dmg)[3],
                    bool can_unlock) {
    int target = 0;
    bool attacked = false;
    for (int i = slots - 1; i >= 0; i--) {
        const bool here = s.m_mask(pool, i) && s.m_row(pool, i) == r && s.m_col(pool, i) == c;
        target = here ? i : target;
        attacked = attacked || here;
    }
    const int type = s.m_type(pool, target);
    float damage = 0.0f;
#pragma unroll
    for (int k = 0; k < 3; k++) damage += (1.0f - mob_defence(type, mc, k)) * dmg[k];
    const bool old_mask = s.m_mask(pool, target);
    s.set_m_hp(pool, target, s.m_hp(pool, target) - damage * (float)(int)attacked);
    for (int i = 0; i < slots; i++) s.set_m_mask(pool, i, s.m_mask(pool, i) && s.m_hp(pool, i) > 0.0f);
    const bool killed = old_mask && !s.m_mask(pool, target);
    unlock_if(h, kill_achievement(mc, type), killed && can_unlock);
    return Hit{attacked, killed};
}

// craftax_do_action_attack_mob / craftax_update_mobs_attack_mob_with_damage (:5962-6036,
// 6725-6797): melee, passive, ranged pools in that order, then the mob bitmap and the
// kill counter
template <class S>
CFE_FN Hit hit_cell(S& s, Hot& h, int r, int c, const float (&dmg)[3], bool can_eat) {
    const Hit melee = hit_pool(s, h, P_MELEE, 3, MC_MELEE, r, c, dmg, true);
    const Hit passive = hit_pool(s, h, P_PASSIVE, 3, MC_PASSIVE, r, c, dmg, can_eat);
    if (passive.killed && can_eat) {
        h.food = imin(max_food(h), h.food + 6);
        h.hunger = 0.0f;
    }
    const Hit ranged = hit_pool(s, h, P_RANGED, 2, MC_RANGED, r, c, dmg, true);
    const bool monster = melee.killed || ranged.killed;
    const bool killed = monster || passive.killed;
    int ur, uc;
    if (killed && wrap_drop(r, kMap, ur) && wrap_drop(c, kMap, uc)) {
        const int l = wrap_clamp(h.level, kLevels);
        (void)uc;
        s.put_mobrow(l, ur, movers_row(s, ur));
    }
    if (monster) {
        const int l = wrap_clamp(h.level, kLevels);
        s.set_kills(l, s.kills(l) + 1);
    }
    return Hit{melee.attacked || passive.attacked || ranged.attacked, killed};
}

// craftax_add_items_from_chest_native (:5519-5644).  The sixteen keys are consecutive LCG
// states after `key`; the wood draws are made and dropped as in the reference.
template <class S>
CFE_FN void loot_chest(S& s, Hot& h, uint64_t key) {
    uint64_t rng = key;
    (void)next_key(rng);  // wood chance
    (void)next_key(rng);  // wood amount
    const bool torch = draw_unit(next_key(rng)) < 0.6f;
    const int torch_n = draw_int(next_key(rng), 4, 8) * (int)torch;
    const bool ore = draw_unit(next_key(rng)) < 0.6f;
    const float ore_w[5] = {0.3f, 0.3f, 0.15f, 0.125f, 0.125f};
    const int ore_id = draw_weighted(next_key(rng), ore_w);
    const uint64_t amount_key = next_key(rng);
    const bool potion = draw_unit(next_key(rng)) < 0.5f;
    const int potion_idx = draw_int(next_key(rng), 0, 6);
    const int potion_n = draw_int(next_key(rng), 1, 3);
    const bool arrows = draw_unit(next_key(rng)) < 0.25f;
    const int arrows_n = draw_int(next_key(rng), 1, 5) * (int)arrows;
    const bool tool = draw_unit(next_key(rng)) < 0.2f;
    const int tool_id = draw_int(next_key(rng), 0, 2);
    const float tool_w[4] = {0.4f, 0.3f, 0.2f, 0.1f};
    const int pickaxe_tier = draw_weighted(next_key(rng), tool_w) + 1;
    const int sword_tier = draw_weighted(next_key(rng), tool_w) + 1;

    h.torches += torch_n;
    if (ore) {
        if (ore_id == 0) h.coal += draw_int(amount_key, 1, 4);
        if (ore_id == 1) h.iron += draw_int(amount_key, 1, 3);
        if (ore_id == 2) h.diamond += draw_int(amount_key, 1, 2);
        if (ore_id == 3) h.sapphire += draw_int(amount_key, 1, 2);
        if (ore_id == 4) h.ruby += draw_int(amount_key, 1, 2);
    }
    h.arrows += arrows_n;
    if (tool && tool_id == 0) h.pickaxe = imax(pickaxe_tier, h.pickaxe);
    if (tool && tool_id == 1) h.sword = imax(sword_tier, h.sword);
    if (potion) put(h.potions, potion_idx, pick(h.potions, potion_idx) + potion_n);
    const int l = wrap_clamp(h.level, kLevels);
    const bool first = !s.chest(l);
    if (h.level == 1 && first) h.bow = 1;
    if (first && (h.level == 3 || h.level == 4)) h.books += 1;
}

// craftax_do_action_native (:6083-6256)
template <class S>
CFE_FN void do_action(S& s, Hot& h, uint64_t key) {
    const Vec2 d = dir_vec(h.dir);
    const int tr = h.pr + d.r, tc = h.pc + d.c;
    float dmg[3];
    player_damage(h, dmg);
    const Hit hit = hit_cell(s, h, tr, tc, dmg, true);

    const int l = wrap_clamp(h.level, kLevels);
    // the target block is read at the wrapped-and-clamped cell even when the target is off
    // the map; a chest or the necromancer seen that way still counts below
    const int b = s.blk(l, wrap_clamp(tr, kMap), wrap_clamp(tc, kMap));
    uint64_t rng = key;
    const uint64_t sapling_key = next_key(rng);
    const uint64_t chest_key = next_key(rng);

    const bool opening_chest = b == B_CHEST;
    bool boss_vulnerable = false;
    if (b == B_NECROMANCER && at_boss(h)) {
        // craftax_do_action_boss_vulnerable (:6045-6063)
        int guards = 0;
        for (int i = 0; i < 3; i++) guards += (int)s.m_mask(P_MELEE, i);
        for (int i = 0; i < 2; i++) guards += (int)s.m_mask(P_RANGED, i);
        boss_vulnerable = guards == 0 && h.boss_timer <= 0;
    }
    const bool damaging_boss = boss_vulnerable;

    if (on_map(tr, tc) && !hit.attacked) {
        switch (b) {
            case B_TREE: set_block(s, l, tr, tc, B_GRASS); h.wood += 1; break;
            case B_FIRE_TREE: set_block(s, l, tr, tc, B_FIRE_GRASS); h.wood += 1; break;
            case B_ICE_SHRUB: set_block(s, l, tr, tc, B_ICE_GRASS); h.wood += 1; break;
            case B_STONE:
                if (h.pickaxe >= 1) { set_block(s, l, tr, tc, B_PATH); h.stone += 1; }
                break;
            case B_FURNACE:
            case B_TABLE: set_block(s, l, tr, tc, B_PATH); break;
            case B_COAL:
                if (h.pickaxe >= 1) { set_block(s, l, tr, tc, B_PATH); h.coal += 1; }
                break;
            case B_IRON:
                if (h.pickaxe >= 2) { set_block(s, l, tr, tc, B_PATH); h.iron += 1; }
                break;
            case B_DIAMOND:
                if (h.pickaxe >= 3) { set_block(s, l, tr, tc, B_PATH); h.diamond += 1; }
                break;
            case B_SAPPHIRE:
                if (h.pickaxe >= 4) { set_block(s, l, tr, tc, B_PATH); h.sapphire += 1; }
                break;
            case B_RUBY:
                if (h.pickaxe >= 4) { set_block(s, l, tr, tc, B_PATH); h.ruby += 1; }
                break;
            case B_GRASS: h.sapling += (int)(draw_unit(sapling_key) < 0.1f); break;
            case B_WATER:
            case B_FOUNTAIN:
                h.drink = imin(max_food(h), h.drink + 1);
                h.thirst = 0.0f;
                unlock(h, ACH_COLLECT_DRINK);
                break;
            case B_RIPE_PLANT: {
                set_block(s, l, tr, tc, B_PLANT);
                h.food = imin(max_food(h), h.food + 4);
                h.hunger = 0.0f;
                unlock(h, ACH_EAT_PLANT);
                // craftax_do_action_update_plants_with_eat (:6065-6081): the first slot at
                // this position, masked or not; slot 0 when none is
                int idx = 0;
                for (int i = kPlants - 1; i >= 0; i--)
                    idx = (s.plant_r(i) == tr && s.plant_c(i) == tc) ? i : idx;
                s.set_plant_age(idx, 0);
                break;
            }
            case B_STALAGMITE:
                if (h.pickaxe >= 1) { set_block(s, l, tr, tc, B_PATH); h.stone += 1; }
                break;
            case B_CHEST:
                set_block(s, l, tr, tc, B_PATH);
                loot_chest(s, h, chest_key);
                unlock(h, ACH_OPEN_CHEST);
                break;
            default: break;
        }
        if (damaging_boss) unlock(h, ACH_DAMAGE_NECROMANCER);
    }
    if (opening_chest) s.set_chest(l);
    if (damaging_boss) {
        h.boss_progress += 1;
        h.boss_timer = 7;  // CRAFTAX_DO_ACTION_BOSS_FIGHT_SPAWN_TURNS
    }
}

// craftax_crafting_add_torch_light (:5030-5052)
template <class S>
CFE_FN void add_torch_light(S& s, int l, int r, int c) {
    for (int dr = -4; dr <= 4; dr++) {
        const int rr = r + dr;
        if ((unsigned)rr >= (unsigned)kMap) continue;
        for (int dc = -4; dc <= 4; dc++) {
            const int cc = c + dc;
            if ((unsigned)cc >= (unsigned)kMap) continue;
            const float t = torch_light(dr, dc);
            if (t == 0.0f) continue;  // q / 255 * 255 truncates back to q for every byte q
            // product and sum rounded separately, as the reference's GPU port spells it
            // (craftax_full.cu:5163-5164, built with -fmad=false).  Its C build under gcc
            // -ffast-math fuses the two into one multiply-add where the CPU has one, which
            // gives a byte one higher for a third of the (byte, distance) pairs: that is
            // the toolchain's choice, not the game's.
            float v = (float)s.lum(l, rr, cc) * (1.0f / 255.0f) + t;
            v = v < 0.0f ? 0.0f : v;
            v = v > 1.0f ? 1.0f : v;
            s.put_lum(l, rr, cc, (int)(uint8_t)(v * 255.0f));
        }
    }
}

// craftax_place_block_native (:5078-5181)
template <class S>
CFE_FN void place_block(S& s, Hot& h, int action) {
    if (!(action == A_PLACE_STONE || action == A_PLACE_TABLE || action == A_PLACE_FURNACE ||
          action == A_PLACE_PLANT || action == A_PLACE_TORCH))
        return;
    const Vec2 d = dir_vec(h.dir);
    const int r = h.pr + d.r, c = h.pc + d.c;
    if (!on_map(r, c) || mob_or_player_at(s, h, r, c)) return;
    const int l = wrap_clamp(h.level, kLevels);
    const int b = s.blk(l, r, c);
    const int it = s.item(l, r, c);
    const bool occupied = is_solid(b) || it != I_NONE;
    if (action == A_PLACE_TABLE) {
        if (!occupied && h.wood >= 2) {
            set_block(s, l, r, c, B_TABLE);
            h.wood -= 2;
            unlock(h, ACH_PLACE_TABLE);
        }
    } else if (action == A_PLACE_FURNACE) {
        if (!occupied && h.stone > 0) {
            set_block(s, l, r, c, B_FURNACE);
            h.stone -= 1;
            unlock(h, ACH_PLACE_FURNACE);
        }
    } else if (action == A_PLACE_STONE) {
        if ((b == B_WATER || !occupied) && h.stone > 0) {
            set_block(s, l, r, c, B_STONE);
            h.stone -= 1;
            unlock(h, ACH_PLACE_STONE);
        }
    } else if (action == A_PLACE_TORCH) {
        if (in_set(kItemGround, b) && it == I_NONE && h.torches > 0) {
            s.put_item(l, r, c, I_TORCH);
            add_torch_light(s, l, r, c);
            h.torches -= 1;
            unlock(h, ACH_PLACE_TORCH);
        }
    } else {  // A_PLACE_PLANT
        if (b == B_GRASS && h.sapling > 0 && it == I_NONE) {
            set_block(s, l, r, c, B_PLANT);
            // craftax_add_new_growing_plant_native (:5054-5076): first free slot, if any
            int slot = -1;
            for (int i = kPlants - 1; i >= 0; i--) slot = ((h.plant_mask >> i) & 1u) ? slot : i;
            if (slot >= 0) {
                s.set_plant(slot, r, c);
                s.set_plant_age(slot, 0);
                h.plant_mask |= 1u << slot;
            }
            h.sapling -= 1;
            unlock(h, ACH_PLACE_PLANT);
        }
    }
}

// craftax_medium_spawn_player_projectile (:5231-5280)
template <class S>
CFE_FN bool launch_player_projectile(S& s, const Hot& h, int type) {
    int count = 0, slot = 0;
    for (int i = 2; i >= 0; i--) {
        const bool m = s.m_mask(P_PLAYER_PROJ, i);
        count += (int)m;
        slot = m ? slot : i;
    }
    if (count >= 3) return false;
    const Vec2 d = dir_vec(h.dir);
    s.set_m_pos(P_PLAYER_PROJ, slot, h.pr, h.pc);
    s.set_m_mask(P_PLAYER_PROJ, slot, true);
    s.set_m_type(P_PLAYER_PROJ, slot, type);
    s.set_pd(P_PLAYER_PROJ, slot, d.r, d.c);
    return true;
}

// craftax_shoot_projectile_native, craftax_cast_spell_native (:5305-5367)
template <class S>
CFE_FN void shoot_or_cast(S& s, Hot& h, int action) {
    if (action == A_SHOOT_ARROW) {
        if (h.bow >= 1 && h.arrows >= 1 && launch_player_projectile(s, h, 4 /* ARROW2 */)) {
            unlock(h, ACH_FIRE_BOW);
            h.arrows -= 1;
        }
    } else if (action == A_CAST_FIREBALL || action == A_CAST_ICEBALL) {
        const int which = action - A_CAST_FIREBALL;
        if (h.mana >= 2 && (which ? opaque(h.spell[1]) : opaque(h.spell[0])) && launch_player_projectile(s, h, 2 + which)) {
            unlock(h, which ? ACH_CAST_ICEBALL : ACH_CAST_FIREBALL);
            h.mana -= 2;
        }
    }
}

// craftax_drink_potion_native (:4656-4721)
template <class S>
CFE_FN void drink_potion(S& s, Hot& h, int action) {
    if (action < A_DRINK_POTION_RED || action > A_DRINK_POTION_YELLOW) return;
    const int colour = action - A_DRINK_POTION_RED;
    const int have = pick(h.potions, colour);
    if (have <= 0) return;
    const int effect = s.potion_effect(colour);
    if (effect == 0) h.health += 8.0f;
    if (effect == 1) h.health += -3.0f;
    if (effect == 2) h.mana += 8;
    if (effect == 3) h.mana -= 3;
    if (effect == 4) h.energy += 8;
    if (effect == 5) h.energy -= 3;
    unlock(h, ACH_DRINK_POTION);
    put(h.potions, colour, have - 1);
}

// craftax_read_book_native (:4723-4755)
CFE_FN void read_book(Hot& h, uint64_t key, int action) {
    if (!(action == A_READ_BOOK && h.books > 0)) return;
    const uint64_t choice_key = lcg(lcg(key));
    float p0 = h.spell[0] ? 0.0f : 1.0f;
    const float p1 = h.spell[1] ? 0.0f : 1.0f;
    const float sum = p0 + p1;
    int which = 0;
    if (sum != 0.0f) {
        p0 /= sum;
        which = (1.0f - draw_unit(choice_key)) <= p0 ? 0 : 1;
    }
    unlock(h, which ? ACH_LEARN_ICEBALL : ACH_LEARN_FIREBALL);
    h.books -= 1;
    if (which) h.spell[1] = 1; else h.spell[0] = 1;
}

// craftax_enchant_native (:5369-5458)
template <class S>
CFE_FN void enchant(S& s, Hot& h, int action, uint64_t key) {
    if (!(action == A_ENCHANT_SWORD || action == A_ENCHANT_ARMOUR || action == A_ENCHANT_BOW)) return;
    const Vec2 d = dir_vec(h.dir);
    const int b = s.blk(wrap_clamp(h.level, kLevels), wrap_clamp(h.pr + d.r, kMap), wrap_clamp(h.pc + d.c, kMap));
    const bool fire = b == B_ENCH_FIRE, ice = b == B_ENCH_ICE;
    const int kind = fire ? 1 : 2;
    const int gems = fire ? opaque(h.ruby) : opaque(h.sapphire);
    if (!(h.mana >= 9 && (fire || ice) && gems >= 1)) return;
    bool done = false;
    if (action == A_ENCHANT_BOW && h.bow > 0) {
        h.bow_ench = kind;
        done = true;
    } else if (action == A_ENCHANT_SWORD && h.sword > 0) {
        h.sword_ench = kind;
        unlock(h, ACH_ENCHANT_SWORD);
        done = true;
    } else if (action == A_ENCHANT_ARMOUR && h.armour[0] + h.armour[1] + h.armour[2] + h.armour[3] > 0) {
        uint64_t rng = key;
        const uint64_t armour_key = next_key(rng);
        int plain = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) plain += (int)(h.armour_ench[i] == 0);
        float w[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e = h.armour_ench[i];
            w[i] = (e == 0 || (plain == 0 && e != 0 && e != kind)) ? 1.0f : 0.0f;
        }
        put(h.armour_ench, draw_weighted(armour_key, w), kind);
        unlock(h, ACH_ENCHANT_ARMOUR);
        done = true;
    }
    if (done) {
        if (kind == 2) h.sapphire -= 1; else h.ruby -= 1;
        h.mana -= 9;
    }
}

// craftax_boss_logic_native, craftax_level_up_attributes_native (:4407-4438)
CFE_FN void boss_and_attributes(Hot& h, int action) {
    unlock_if(h, ACH_DEFEAT_NECROMANCER, h.boss_progress >= kLevels - 1);
    h.boss_timer -= (int)at_boss(h);
    if (h.xp >= 1) {
        if (action == A_LEVEL_UP_DEX && h.dex < 5) { h.dex += 1; h.xp -= 1; }
        if (action == A_LEVEL_UP_STR && h.str < 5) { h.str += 1; h.xp -= 1; }
        if (action == A_LEVEL_UP_INT && h.intel < 5) { h.intel += 1; h.xp -= 1; }
    }
}

// ---- mobs (craftax_update_mobs_native, :6269-7377) -----------------------------------------
// craftax_update_mobs_damage_done_to_player (:6659-6680)
CFE_FN float damage_to_player(const Hot& h, const float (&dmg)[3]) {
    float def[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        def[0] += (float)h.armour[i] * 0.1f;
        def[1] += (float)(int)(h.armour_ench[i] == 1) * 0.2f;
        def[2] += (float)(int)(h.armour_ench[i] == 2) * 0.2f;
    }
    const float boss = at_boss(h) ? 1.5f : 1.0f;
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < 3; k++) total += (1.0f - def[k]) * dmg[k] * boss;
    return total;
}

// A mob's move in two halves.  `plan_*` makes every draw of the mob and fixes the cell it
// wants to enter -- that needs the mob's own slot, the player's position and the key, nothing
// an earlier mob of the same step changes.  update_mobs plans all eight movers first and asks
// for the blocks under their targets together (one memory round trip for the eight instead
// of one each); `apply_*` then runs mob by mob in the reference's order with that block:
// damage to the player, the validity of the target against the mobs as they stand by then,
// the bitmap rows, the slot.
struct MoverPlan {
    bool active;      // the slot holds a mob
    int r1, c1;       // the cell the validity test looks at
    Vec2 to;          // ranged: the step towards the player (projectile direction, retreat)
};
// craftax_update_mobs_valid_position (:6625-6648) for target (r, c) with block b under it
CFE_FN bool can_stand(const MoverKeys& m, const Hot& h, int b, int r, int c, int collision) {
    const bool solid = is_solid(b), water = b == B_WATER, lava = b == B_LAVA;
    const bool ground = !solid && !water && !lava;
    const bool taken = keys_at(m, wrap_clamp(r, kMap), wrap_clamp(c, kMap)) || (h.pr == r && h.pc == c);
    bool ok = on_map(r, c) && !taken && !solid;
    ok = ok && (!(collision & 1) || !ground);
    ok = ok && (!(collision & 2) || !water);
    ok = ok && (!(collision & 4) || !lava);
    return ok;
}
// The mob of (pool, i) has left row r0 and stands -- if it is still alive -- where its slot
// says: the rows it left and entered go out as the slots have them
// (craftax_update_mobs_clear_old_map_entry / _enter_new_map_entry, :6389-6421).
template <class S>
CFE_FN void settle_in_bitmap(S& s, int l, MoverKeys& m, int k, int r0, int r1, int c1, bool alive) {
    m.key[k] = alive ? cell_key(r1, c1) : kNoCell;
    const int i_from = wrap_clamp(r0, kMap), i_to = wrap_clamp(r1, kMap);
    s.put_mobrow(l, i_from, keys_row(m, i_from));
    if (i_to != i_from) s.put_mobrow(l, i_to, keys_row(m, i_to));
}

// the step towards the player along the longer axis, drawn when both are equal
// (craftax_update_mobs_player_axis_choice, :6605-6623)
CFE_FN Vec2 step_towards_player(const Hot& h, uint64_t key, int r, int c) {
    const int dr = iabs(h.pr - r), dc = iabs(h.pc - c);
    const int longest = imax(dr, dc), total = dr + dc;
    int axis = 1;
    if (total != 0) {
        const float w[2] = {dr == longest ? 1.0f / (float)total : 0.0f, dc == longest ? 1.0f / (float)total : 0.0f};
        axis = draw_weighted(key, w);
    }
    return axis == 0 ? Vec2{isign(h.pr - r), 0} : Vec2{0, isign(h.pc - c)};
}
CFE_FN Vec2 random_step(uint64_t key, int choices) {  // craftax_update_mobs_direction_choice, :6575-6592
    const int k = draw_int(key, 0, choices);
    return Vec2{k == 2 ? -1 : (k == 3 ? 1 : 0), k == 0 ? -1 : (k == 1 ? 1 : 0)};
}

// craftax_update_mobs_move_melee (:6856-6987)
template <class S>
CFE_FN MoverPlan plan_melee(S& s, const Hot& h, uint64_t& rng, int i) {
    MoverPlan p{s.m_mask(P_MELEE, i), 0, 0, Vec2{0, 0}};
    if (!p.active) return p;
    const int r0 = s.m_row(P_MELEE, i), c0 = s.m_col(P_MELEE, i), cd = s.m_cd(P_MELEE, i);
    const Vec2 rnd = random_step(next_key(rng), 4);
    const Vec2 to = step_towards_player(h, next_key(rng), r0, c0);
    const int dist = iabs(h.pr - r0) + iabs(h.pc - c0);
    bool chase = dist < 10 || at_boss(h);
    chase = (draw_unit(next_key(rng)) < 0.75f) && chase;
    p.r1 = r0 + (chase ? to.r : rnd.r);
    p.c1 = c0 + (chase ? to.c : rnd.c);
    if (dist == 1 && cd <= 0) {   // attacking: it stays
        p.r1 = r0;
        p.c1 = c0;
    }
    rng = lcg(lcg(rng));
    return p;
}
template <class S>
CFE_FN void apply_melee(S& s, Hot& h, MoverKeys& m, const MoverPlan& p, int b, int i) {
    if (!p.active) return;
    const int l = wrap_clamp(h.level, kLevels);
    const int r0 = s.m_row(P_MELEE, i), c0 = s.m_col(P_MELEE, i), cd = s.m_cd(P_MELEE, i), type = s.m_type(P_MELEE, i);
    const int dist = iabs(h.pr - r0) + iabs(h.pc - c0);
    const bool attacking = dist == 1 && cd <= 0;
    int r1 = p.r1, c1 = p.c1;
    float base[3];
    mob_damage(type, MC_MELEE, base);
    const float asleep = 1.0f + 2.5f * (float)(int)(h.sleeping != 0);
#pragma unroll
    for (int k = 0; k < 3; k++) base[k] *= asleep;
    const float damage = damage_to_player(h, base);
    h.health -= damage * (float)(int)attacking;
    unlock_if(h, ACH_WAKE_UP, h.sleeping && attacking);
    if (attacking) h.sleeping = h.resting = 0;
    if (!can_stand(m, h, b, r1, c1, mob_collision(type, MC_MELEE))) {
        r1 = r0;
        c1 = c0;
    }
    const bool alive = dist < kDespawn || at_boss(h);
    s.set_m_pos(P_MELEE, i, r1, c1);
    s.set_m_cd(P_MELEE, i, attacking ? 5 : cd - 1);
    s.set_m_mask(P_MELEE, i, alive);
    settle_in_bitmap(s, l, m, i, r0, r1, c1, alive);
}

// craftax_update_mobs_move_passive (:6989-7052)
template <class S>
CFE_FN MoverPlan plan_passive(S& s, const Hot&, uint64_t& rng, int i) {
    MoverPlan p{s.m_mask(P_PASSIVE, i), 0, 0, Vec2{0, 0}};
    if (!p.active) return p;
    const Vec2 rnd = random_step(next_key(rng), 8);
    p.r1 = s.m_row(P_PASSIVE, i) + rnd.r;
    p.c1 = s.m_col(P_PASSIVE, i) + rnd.c;
    return p;
}
template <class S>
CFE_FN void apply_passive(S& s, Hot& h, MoverKeys& m, const MoverPlan& p, int b, int i) {
    if (!p.active) return;
    const int l = wrap_clamp(h.level, kLevels);
    const int r0 = s.m_row(P_PASSIVE, i), c0 = s.m_col(P_PASSIVE, i), type = s.m_type(P_PASSIVE, i);
    int r1 = p.r1, c1 = p.c1;
    if (!can_stand(m, h, b, r1, c1, mob_collision(type, MC_PASSIVE))) {
        r1 = r0;
        c1 = c0;
    }
    const bool alive = iabs(r0 - h.pr) + iabs(c0 - h.pc) < kDespawn;
    s.set_m_pos(P_PASSIVE, i, r1, c1);
    s.set_m_mask(P_PASSIVE, i, alive);
    settle_in_bitmap(s, l, m, 3 + i, r0, r1, c1, alive);
}

// craftax_update_mobs_move_ranged (:7054-7191)
template <class S>
CFE_FN MoverPlan plan_ranged(S& s, const Hot& h, uint64_t& rng, int i) {
    MoverPlan p{s.m_mask(P_RANGED, i), 0, 0, Vec2{0, 0}};
    if (!p.active) return p;
    const int r0 = s.m_row(P_RANGED, i), c0 = s.m_col(P_RANGED, i);
    const Vec2 rnd = random_step(next_key(rng), 4);
    const Vec2 to = step_towards_player(h, next_key(rng), r0, c0);
    const int dist = iabs(h.pr - r0) + iabs(h.pc - c0);
    const bool far = dist >= 6, close = dist <= 3;
    int r1 = r0 + (far ? to.r : rnd.r), c1 = c0 + (far ? to.c : rnd.c);
    if (close) {
        r1 = r0 - to.r;
        c1 = c0 - to.c;
    }
    if (!(draw_unit(next_key(rng)) > 0.85f)) {
        r1 = r0 + rnd.r;
        c1 = c0 + rnd.c;
    }
    p.r1 = r1;
    p.c1 = c1;
    p.to = to;
    return p;
}
template <class S>
CFE_FN void apply_ranged(S& s, Hot& h, MoverKeys& m, const MoverPlan& p, int b, int i) {
    if (!p.active) return;
    const int l = wrap_clamp(h.level, kLevels);
    const int r0 = s.m_row(P_RANGED, i), c0 = s.m_col(P_RANGED, i), cd = s.m_cd(P_RANGED, i), type = s.m_type(P_RANGED, i);
    const int dist = iabs(h.pr - r0) + iabs(h.pc - c0);
    const bool close = dist <= 3;
    int r1 = p.r1, c1 = p.c1;
    // the target's validity is read once: the reference asks for it up to twice (here and
    // below), for this target or -- when the mob attacks and stays -- for its own cell, which
    // it occupies itself, so that answer never changes where the mob ends up
    const bool can = can_stand(m, h, b, r1, c1, mob_collision(type, MC_RANGED));
    bool attacking = dist >= 4 && dist <= 5;
    attacking = attacking || (close && !can);
    attacking = attacking && cd <= 0;
    if (attacking) {
        // craftax_update_mobs_spawn_mob_projectile (:6682-6723)
        int count = 0, slot = 0;
        for (int k = 2; k >= 0; k--) {
            const bool m = s.m_mask(P_MOB_PROJ, k);
            count += (int)m;
            slot = m ? slot : k;
        }
        if (count < 3) {
            s.set_m_pos(P_MOB_PROJ, slot, r0, c0);
            s.set_m_mask(P_MOB_PROJ, slot, true);
            s.set_m_type(P_MOB_PROJ, slot, ranged_projectile(type));
            s.set_pd(P_MOB_PROJ, slot, p.to.r, p.to.c);
        }
        r1 = r0;
        c1 = c0;
    }
    if (!can) {
        r1 = r0;
        c1 = c0;
    }
    const bool alive = dist < kDespawn || at_boss(h);
    s.set_m_pos(P_RANGED, i, r1, c1);
    s.set_m_cd(P_RANGED, i, attacking ? 4 : cd - 1);
    s.set_m_mask(P_RANGED, i, alive);
    settle_in_bitmap(s, l, m, 6 + i, r0, r1, c1, alive);
}

// craftax_update_mobs_move_mob_projectile (:7193-7268); b = the block under its next cell.
// Returns true when it destroyed that block (a crafting table or furnace in the way).
template <class S>
CFE_FN bool move_mob_projectile(S& s, Hot& h, const MoverKeys& m, int b, int i) {
    if (!s.m_mask(P_MOB_PROJ, i)) return false;
    const int l = wrap_clamp(h.level, kLevels);
    const int r0 = s.m_row(P_MOB_PROJ, i), c0 = s.m_col(P_MOB_PROJ, i);
    const int r1 = r0 + s.pd_r(P_MOB_PROJ, i), c1 = c0 + s.pd_c(P_MOB_PROJ, i);
    const bool hit = (r0 == h.pr && c0 == h.pc) || (r1 == h.pr && c1 == h.pc);
    const bool taken = keys_at(m, wrap_clamp(r1, kMap), wrap_clamp(c1, kMap)) || (h.pr == r1 && h.pc == c1);
    const bool flying = on_map(r1, c1) && !is_solid(b) && !taken && !hit;
    float dmg[3];
    mob_damage(s.m_type(P_MOB_PROJ, i), MC_PROJECTILE, dmg);
    const float damage = damage_to_player(h, dmg);
    s.set_m_pos(P_MOB_PROJ, i, r1, c1);
    s.set_m_mask(P_MOB_PROJ, i, flying);
    h.health -= damage * (float)(int)hit;
    if (hit) h.sleeping = h.resting = 0;
    // a crafting table or furnace in the way is destroyed; the write goes through the
    // scatter index (negative wraps, 48 and beyond is dropped) while the read was clamped
    int wl, wr, wc;
    if ((b == B_FURNACE || b == B_TABLE) && wrap_drop(l, kLevels, wl) && wrap_drop(r1, kMap, wr) && wrap_drop(c1, kMap, wc)) {
        set_block(s, wl, wr, wc, B_PATH);
        return true;
    }
    return false;
}

// craftax_update_mobs_move_player_projectile (:6799-6854, 7270-7346); b as above
template <class S>
CFE_FN void move_player_projectile(S& s, Hot& h, int b, int i) {
    if (!s.m_mask(P_PLAYER_PROJ, i)) return;
    const int r0 = s.m_row(P_PLAYER_PROJ, i), c0 = s.m_col(P_PLAYER_PROJ, i);
    const int r1 = r0 + s.pd_r(P_PLAYER_PROJ, i), c1 = c0 + s.pd_c(P_PLAYER_PROJ, i);
    const int type = s.m_type(P_PLAYER_PROJ, i);
    float dmg[3];
    mob_damage(type, MC_PROJECTILE, dmg);
    if (type == 0 || type == 4) {  // arrows: the bow's enchantment adds half the physical part
        float add[3] = {0.0f, 0.0f, 0.0f};
        int e;
        if (wrap_drop(h.bow_ench, 3, e)) {
            const float half = dmg[0] * (1.0f / 2.0f);
            add[1] = e == 1 ? half : 0.0f;
            add[2] = e == 2 ? half : 0.0f;
        }
        const float coeff = 1.0f + 0.2f * (float)(h.dex - 1);
#pragma unroll
        for (int k = 0; k < 3; k++) dmg[k] = (dmg[k] + add[k]) * coeff;
    }
    if (type == 2 || type == 3) {  // fireball, iceball
        const float coeff = 1.0f + 0.5f * (float)(h.intel - 1);
#pragma unroll
        for (int k = 0; k < 3; k++) dmg[k] *= coeff;
    }
    const Hit first = hit_cell(s, h, r0, c0, dmg, false);
    float second[3];
#pragma unroll
    for (int k = 0; k < 3; k++) second[k] = dmg[k] * (float)(int)(!first.attacked);
    const Hit next = hit_cell(s, h, r1, c1, second, false);
    const bool flying = on_map(r1, c1) && !is_solid(b) && !(first.attacked || next.attacked);
    s.set_m_pos(P_PLAYER_PROJ, i, r1, c1);
    s.set_m_mask(P_PLAYER_PROJ, i, flying);
}

template <class S>
CFE_FN void update_mobs(S& s, Hot& h, uint64_t rng) {
    const int l = wrap_clamp(h.level, kLevels);
    MoverPlan plan[8];
    rng = lcg(rng);
#pragma unroll
    for (int i = 0; i < 3; i++) plan[i] = plan_melee(s, h, rng, i);
    rng = lcg(rng);
#pragma unroll
    for (int i = 0; i < 3; i++) plan[3 + i] = plan_passive(s, h, rng, i);
    rng = lcg(rng);
#pragma unroll
    for (int i = 0; i < 2; i++) plan[6 + i] = plan_ranged(s, h, rng, i);
    // the eight blocks, asked for together (an empty slot reads the block under cell (0, 0))
    int b[8];
#pragma unroll
    for (int k = 0; k < 8; k++) b[k] = s.blk(l, wrap_clamp(plan[k].r1, kMap), wrap_clamp(plan[k].c1, kMap));
    MoverKeys m = load_mover_keys(s);
#pragma unroll
    for (int i = 0; i < 3; i++) apply_melee(s, h, m, plan[i], b[i], i);
#pragma unroll
    for (int i = 0; i < 3; i++) apply_passive(s, h, m, plan[3 + i], b[3 + i], i);
#pragma unroll
    for (int i = 0; i < 2; i++) apply_ranged(s, h, m, plan[6 + i], b[6 + i], i);
    // the six projectiles -- those the ranged mobs just launched among them -- likewise.  A
    // mob projectile that destroys the block under its next cell changes what a later
    // projectile with the same next cell finds there.
    int pr1[6], pc1[6], pb[6];
#pragma unroll
    for (int k = 0; k < 6; k++) {
        const int pool = k < 3 ? P_MOB_PROJ : P_PLAYER_PROJ, i = k % 3;
        pr1[k] = wrap_clamp(s.m_row(pool, i) + s.pd_r(pool, i), kMap);
        pc1[k] = wrap_clamp(s.m_col(pool, i) + s.pd_c(pool, i), kMap);
        pb[k] = s.blk(l, pr1[k], pc1[k]);
    }
#pragma unroll
    for (int i = 0; i < 3; i++) {
        if (move_mob_projectile(s, h, m, pb[i], i)) {
#pragma unroll
            for (int k = i + 1; k < 6; k++)
                if (pr1[k] == pr1[i] && pc1[k] == pc1[i]) pb[k] = B_PATH;
        }
    }
#pragma unroll
    for (int i = 0; i < 3; i++) move_player_projectile(s, h, pb[3 + i], i);
}

// ---- spawning (craftax_spawn_mobs_native, :7397-8225) ---------------------------------------
// Rings around the player a mob may appear in, as the set of column offsets -13..13 (bit
// dc + 13) allowed in the row |dr| away: passive 9 < d^2 < 196, hostile 81 < d^2 < 196,
// boss fight d^2 < 37 (craftax_spawn_init_offsets_once, :7459-7509).
enum Ring : int { RING_PASSIVE = 0, RING_HOSTILE = 1, RING_BOSS = 2 };
constexpr uint32_t ring_row_const(int ring, int adr) {
    const int lo = ring == RING_PASSIVE ? 9 : ring == RING_HOSTILE ? 81 : -1;
    const int hi = ring == RING_BOSS ? 37 : kDespawn * kDespawn;
    uint32_t m = 0;
    for (int dc = -(kDespawn - 1); dc <= kDespawn - 1; dc++) {
        const int d2 = adr * adr + dc * dc;
        m |= (uint32_t)(d2 > lo && d2 < hi) << (dc + kDespawn - 1);
    }
    return m;
}
// The allowed offsets of a ring row are a centred run minus a centred run: half-widths + 1 (0 =
// empty), one nibble per |dr|, derived from ring_row_const at compile time.
constexpr int run_half_width(uint32_t m) {   // widest w with bits 13-w .. 13+w all set, +1; 0 if bit 13 is clear
    int w = 0;
    while (w <= kDespawn - 1 && ((m >> (kDespawn - 1 - w)) & 1u) && ((m >> (kDespawn - 1 + w)) & 1u)) w++;
    return w;
}
constexpr uint32_t centred_run(int w1) { return w1 ? ((1u << (2 * w1 - 1)) - 1u) << (kDespawn - w1) : 0u; }
constexpr uint64_t pack_outer(int ring) {
    uint64_t t = 0;
    for (int a = 0; a < kDespawn; a++) {
        const uint32_t m = ring_row_const(ring, a);
        int w = 0;   // the row's extent: widest set offset + 1
        for (int dc = 0; dc < kDespawn; dc++)
            if ((m >> (kDespawn - 1 + dc)) & 1u) w = dc + 1;
        t |= (uint64_t)w << (4 * a);
    }
    return t;
}
constexpr uint64_t pack_inner(int ring, uint64_t outer_table) {   // the hole around dc = 0, as a centred run
    uint64_t t = 0;
    for (int a = 0; a < kDespawn; a++) {
        const uint32_t outer = centred_run((int)((outer_table >> (4 * a)) & 15));
        t |= (uint64_t)run_half_width(outer & ~ring_row_const(ring, a)) << (4 * a);
    }
    return t;
}
constexpr uint64_t kRingOuter[3] = {pack_outer(RING_PASSIVE), pack_outer(RING_HOSTILE), pack_outer(RING_BOSS)};
constexpr uint64_t kRingInner[3] = {pack_inner(RING_PASSIVE, kRingOuter[0]), pack_inner(RING_HOSTILE, kRingOuter[1]),
                                    pack_inner(RING_BOSS, kRingOuter[2])};
constexpr bool ring_table_holds(int ring) {
    for (int a = 0; a < kDespawn; a++)
        if (ring_row_const(ring, a) != (centred_run((int)((kRingOuter[ring] >> (4 * a)) & 15)) &
                                        ~centred_run((int)((kRingInner[ring] >> (4 * a)) & 15))))
            return false;
    return true;
}
static_assert(ring_table_holds(0) && ring_table_holds(1) && ring_table_holds(2),
              "ring rows are a centred run minus a centred run");
CFE_FN uint32_t ring_row(int ring, int adr) {
    constexpr uint64_t o0 = kRingOuter[0], o1 = kRingOuter[1], o2 = kRingOuter[2];
    constexpr uint64_t i0 = kRingInner[0], i1 = kRingInner[1], i2 = kRingInner[2];
    const uint64_t outer = ring == RING_PASSIVE ? o0 : (ring == RING_HOSTILE ? o1 : o2);
    const uint64_t inner = ring == RING_PASSIVE ? i0 : (ring == RING_HOSTILE ? i1 : i2);
    const int w = (int)((outer >> (4 * adr)) & 15), v = (int)((inner >> (4 * adr)) & 15);
    const uint32_t a = w ? ((1u << (2 * w - 1)) - 1u) << (kDespawn - w) : 0u;
    const uint32_t b = v ? ((1u << (2 * v - 1)) - 1u) << (kDespawn - v) : 0u;
    return a & ~b;
}
// open cells of map row pr + dr in the ring: the terrain plane, minus mobs, inside the map
template <class S>
CFE_FN uint64_t spawn_candidates(S& s, const Hot& h, int l, int ring, int kind, int dr) {
    // no branch around the two loads: a row off the map reads row 0 and is masked out, so that
    // a caller that unrolls over the rows gets all its loads in flight together
    const int r = h.pr + dr;
    const bool live = (unsigned)r < (unsigned)kMap;
    const int rr = live ? r : 0;
    const uint64_t shape = ring_row(ring, iabs(dr));
    const int sh = h.pc - (kDespawn - 1);
    const uint64_t cols = live ? ((sh >= 0 ? shape << sh : shape >> -sh) & kRowMask) : 0ull;
    return s.spawnrow(kind, l, rr) & ~s.mobrow(l, rr) & cols;
}
// craftax_spawn_pick_kth (:7694-7704): the smallest k with k + 1 >= n * (1 - u)
CFE_FN int pick_index(int n, uint64_t key) {
    const float draw = (float)n * (1.0f - draw_unit(key));
    // the reference counts cum = 1, 2, ... until cum >= draw; integers up to 729 are exact
    int k = (int)__builtin_ceilf(draw) - 1;
    k = k < 0 ? 0 : k;
    return k > n - 1 ? n - 1 : k;
}
// craftax_spawn_scan_spans (:7717-7770) without the coordinate list: count, draw, find
template <class S>
CFE_FN bool spawn_site(S& s, const Hot& h, int l, int ring, int kind, uint64_t key, int& row, int& col) {
    int n = 0;
    for (int dr = -(kDespawn - 1); dr <= kDespawn - 1; dr++) n += __builtin_popcountll(spawn_candidates(s, h, l, ring, kind, dr));
    if (n == 0) return false;
    int k = pick_index(n, key);
    for (int dr = -(kDespawn - 1); dr <= kDespawn - 1; dr++) {
        uint64_t m = spawn_candidates(s, h, l, ring, kind, dr);
        const int cnt = __builtin_popcountll(m);
        if (k >= cnt) {
            k -= cnt;
            continue;
        }
        for (; k > 0; k--) m &= m - 1;
        row = h.pr + dr;
        col = __builtin_ctzll(m);
        return true;
    }
    return false;
}

struct SpawnPlan {  // what the per-env prologue decides; the scans may run later
    uint64_t key[3];    // position keys: passive, melee, ranged
    int8_t slot[3];
    int8_t type[3];
    int8_t ring[3];
    int8_t kind[3];
    uint8_t tries;      // bit 0 passive, 1 melee, 2 ranged
};
CFE_FN int spawn_pool(int which) { return which == 0 ? P_PASSIVE : which == 1 ? P_MELEE : P_RANGED; }
CFE_FN int spawn_class(int which) { return which == 0 ? MC_PASSIVE : which == 1 ? MC_MELEE : MC_RANGED; }

// first half of craftax_spawn_mobs_native (:8065-8131): counts, keys, the unconditional
// type_id writes, the three chance rolls
template <class S>
CFE_FN SpawnPlan plan_spawns(S& s, const Hot& h, uint64_t rng) {
    SpawnPlan p;
    const int l = wrap_clamp(h.level, kLevels);
    const bool boss = at_boss(h);
    int coeff = 1 + (int)(s.kills(l) < kKillsToClear) * 2;
    if (boss) coeff *= (int)(h.boss_timer >= 1) * 1000;
    // level:                              8     7     6     5     4     3     2     1     0
    // chances (:7556-7573): passive 0.1 except level 7 (0); melee 0.06 (level 0: 0.02); ranged
    // 0.05; night term 0.1 on level 0 only
    const float passive_chance = l == 7 ? 0.0f : 0.1f;
    const float melee_base = l == 0 ? 0.02f : 0.06f;
    const float night_gain = l == 0 ? 0.1f : 0.0f;
    int count[3], slot[3];
#pragma unroll
    for (int w = 0; w < 3; w++) {
        const int pool = spawn_pool(w), slots = w == 2 ? 2 : 3;
        int n = 0, first = 0;
#pragma unroll
        for (int i = slots - 1; i >= 0; i--) {
            const bool m = s.m_mask(pool, i);
            n += (int)m;
            first = m ? first : i;
        }
        count[w] = n;
        slot[w] = first;
        p.slot[w] = (int8_t)first;
    }
    const uint64_t passive_prob = next_key(rng);
    p.key[0] = next_key(rng);
    p.type[0] = (int8_t)floor_mob_type(l, MC_PASSIVE);
    s.set_m_type(P_PASSIVE, slot[0], p.type[0]);

    p.type[1] = (int8_t)floor_mob_type(boss ? (int)h.boss_progress : (int)l, MC_MELEE);
    const uint64_t melee_prob = next_key(rng);
    const float night = 1.0f - h.light_level;
    const float melee_chance = melee_base + night_gain * night * night;
    p.key[1] = next_key(rng);
    s.set_m_type(P_MELEE, slot[1], p.type[1]);

    p.type[2] = (int8_t)floor_mob_type(boss ? (int)h.boss_progress : (int)l, MC_RANGED);
    const uint64_t ranged_prob = next_key(rng);
    p.key[2] = next_key(rng);
    s.set_m_type(P_RANGED, slot[2], p.type[2]);

    const bool try_passive = !boss && count[0] < 3 && draw_unit(passive_prob) < passive_chance;
    const bool try_melee = count[1] < 3 && draw_unit(melee_prob) < melee_chance * (float)coeff;
    const bool try_ranged = count[2] < 2 && draw_unit(ranged_prob) < 0.05f * (float)coeff;
    p.tries = (uint8_t)((int)try_passive | (int)try_melee << 1 | (int)try_ranged << 2);
    p.ring[0] = RING_PASSIVE;
    p.kind[0] = SK_ALL;
    p.ring[1] = p.ring[2] = (int8_t)(boss ? RING_BOSS : RING_HOSTILE);
    p.kind[1] = (int8_t)(boss ? SK_GRAVE : SK_ALL);
    p.kind[2] = (int8_t)(boss ? SK_GRAVE : (p.type[2] == 5 ? SK_WATER : SK_ALL));
    return p;
}
// a mob appears (:7989-7994 and the like)
template <class S>
CFE_FN void place_spawn(S& s, int l, int which, const SpawnPlan& p, int row, int col) {
    const int pool = spawn_pool(which);
    s.set_m_pos(pool, p.slot[which], row, col);
    s.set_m_hp(pool, p.slot[which], mob_health(p.type[which], spawn_class(which)));
    s.set_m_mask(pool, p.slot[which], true);
    s.put_mobrow(l, row, movers_row(s, row));
}
// second half (:8133-8224): passive, melee, ranged in that order.  The reference scans all
// three against the bitmap as it was and then excludes the cells just taken; scanning in
// order against the bitmap as it becomes is the same selection.
template <class S>
CFE_FN void run_spawns(S& s, const Hot& h, const SpawnPlan& p) {
    const int l = wrap_clamp(h.level, kLevels);
#pragma unroll
    for (int w = 0; w < 3; w++) {
        if (!((p.tries >> w) & 1)) continue;
        int row, col;
        if (spawn_site(s, h, l, p.ring[w], p.kind[w], p.key[w], row, col)) place_spawn(s, l, w, p, row, col);
    }
}

// ---- plants, intrinsics, clipping, inventory achievements -----------------------------------
// craftax_update_plants_native (:4381-4405); unmasked slots keep age 0
template <class S>
CFE_FN void grow_plants(S& s, Hot& h) {
    for (uint32_t m = h.plant_mask; m != 0; m &= m - 1) {
        const int i = __builtin_ctz(m);
        const int age = s.plant_age(i) + 1;
        s.set_plant_age(i, age);
        if (age >= 600) set_block(s, 0, wrap_clamp(s.plant_r(i), kMap), wrap_clamp(s.plant_c(i), kMap), B_RIPE_PLANT);
    }
}

CFE_FN float fmin_(float a, float b) { return a < b ? a : b; }
CFE_FN float fmax_(float a, float b) { return a > b ? a : b; }

// craftax_update_player_intrinsics_native (:4549-4654)
CFE_FN void update_intrinsics(Hot& h, int action) {
    const int cap = max_food(h);
    if (action == A_SLEEP && h.energy < cap) h.sleeping = 1;
    const bool waking = h.energy >= cap && h.sleeping;
    if (waking) h.sleeping = 0;
    unlock_if(h, ACH_WAKE_UP, waking);
    const float hp_cap = (float)max_health(h);
    if (action == A_REST && h.health < hp_cap) h.resting = 1;
    if (h.resting && (h.health >= hp_cap || h.food <= 0 || h.drink <= 0)) h.resting = 0;

    const int not_boss = (int)!at_boss(h);
    const float decay = 1.0f - (0.125f * (float)(h.dex - 1));
    const float pace = h.sleeping ? 0.5f : 1.0f;

    float hunger = h.hunger + pace * decay;
    if (hunger > 25.0f) {
        h.food = imax(h.food - not_boss, 0);
        hunger = 0.0f;
    }
    h.hunger = hunger;

    float thirst = h.thirst + pace * decay;
    if (thirst > 20.0f) {
        h.drink = imax(h.drink - not_boss, 0);
        thirst = 0.0f;
    }
    h.thirst = thirst;

    float fatigue = h.sleeping ? fmin_(h.fatigue - 1.0f, 0.0f) : h.fatigue + decay;
    int energy = h.energy;
    if (fatigue > 30.0f) {
        energy = imax(h.energy - not_boss, 0);
        fatigue = 0.0f;
    }
    if (fatigue < -10.0f) {
        energy = imin(h.energy + 1, cap);
        fatigue = 0.0f;
    }
    h.fatigue = fatigue;
    h.energy = energy;

    const bool provided = h.food > 0 && h.drink > 0 && (h.energy > 0 || h.sleeping);
    const float gain = provided ? (h.sleeping ? 2.0f : 1.0f) : (h.sleeping ? -0.5f : -1.0f) * (float)not_boss;
    float recover = h.recover + gain;
    float health = h.health;
    if (recover > 25.0f) {
        health = fmin_(h.health + 1.0f, hp_cap);
        recover = 0.0f;
    }
    if (recover < -15.0f) {
        health = h.health - 1.0f;
        recover = 0.0f;
    }
    h.recover = recover;
    h.health = health;

    const float mana_pace = 1.0f + 0.25f * (float)(h.intel - 1);
    float rm = (h.sleeping ? h.recover_mana + 2.0f : h.recover_mana + 1.0f) * mana_pace;
    if (rm > 30.0f) {
        h.mana += 1;
        rm = 0.0f;
    }
    h.recover_mana = rm;
}

// craftax_clip_inventory_and_intrinsics_native, craftax_calculate_inventory_achievements_native
// (:4440-4547)
CFE_FN void clip_and_count(Hot& h) {
    h.wood = imin(h.wood, 99);
    h.stone = imin(h.stone, 99);
    h.coal = imin(h.coal, 99);
    h.iron = imin(h.iron, 99);
    h.diamond = imin(h.diamond, 99);
    h.sapling = imin(h.sapling, 99);
    h.pickaxe = imin(h.pickaxe, 99);
    h.sword = imin(h.sword, 99);
    h.bow = imin(h.bow, 99);
    h.arrows = imin(h.arrows, 99);
    h.torches = imin(h.torches, 99);
    h.ruby = imin(h.ruby, 99);
    h.sapphire = imin(h.sapphire, 99);
    h.books = imin(h.books, 99);
#pragma unroll
    for (int i = 0; i < 4; i++) h.armour[i] = imin(h.armour[i], 99);
#pragma unroll
    for (int i = 0; i < 6; i++) h.potions[i] = imin(h.potions[i], 99);
    h.health = fmin_(fmax_(h.health, 0.0f), (float)max_health(h));
    const int cap = max_food(h);
    h.food = imin(imax(h.food, 0), cap);
    h.drink = imin(imax(h.drink, 0), cap);
    h.energy = imin(imax(h.energy, 0), cap);
    h.mana = imin(imax(h.mana, 0), max_mana(h));

    unlock_if(h, ACH_COLLECT_WOOD, h.wood > 0);
    unlock_if(h, ACH_COLLECT_STONE, h.stone > 0);
    unlock_if(h, ACH_COLLECT_COAL, h.coal > 0);
    unlock_if(h, ACH_COLLECT_IRON, h.iron > 0);
    unlock_if(h, ACH_COLLECT_DIAMOND, h.diamond > 0);
    unlock_if(h, ACH_COLLECT_RUBY, h.ruby > 0);
    unlock_if(h, ACH_COLLECT_SAPPHIRE, h.sapphire > 0);
    unlock_if(h, ACH_COLLECT_SAPLING, h.sapling > 0);
    unlock_if(h, ACH_FIND_BOW, h.bow > 0);
    unlock_if(h, ACH_MAKE_ARROW, h.arrows > 0);
    unlock_if(h, ACH_MAKE_TORCH, h.torches > 0);
    unlock_if(h, ACH_MAKE_WOOD_PICKAXE, h.pickaxe >= 1);
    unlock_if(h, ACH_MAKE_STONE_PICKAXE, h.pickaxe >= 2);
    unlock_if(h, ACH_MAKE_IRON_PICKAXE, h.pickaxe >= 3);
    unlock_if(h, ACH_MAKE_DIAMOND_PICKAXE, h.pickaxe >= 4);
    unlock_if(h, ACH_MAKE_WOOD_SWORD, h.sword >= 1);
    unlock_if(h, ACH_MAKE_STONE_SWORD, h.sword >= 2);
    unlock_if(h, ACH_MAKE_IRON_SWORD, h.sword >= 3);
    unlock_if(h, ACH_MAKE_DIAMOND_SWORD, h.sword >= 4);
}

// ---- the step (craftax_gameplay_step_native, :3798-3878) ---------------------------------------
struct StepOut {
    float reward;
    bool done;
    uint64_t state_rng;   // CraftaxState.state_rng after the step
};

// Everything of the step up to and including the spawn rolls; the scans the rolls ask for
// are returned in `plan` and run by run_spawns, at once (host) or cooperatively by the
// wavefront once every lane is through (kernel).  Nothing after the rolls reads what a
// spawn writes.
template <class S>
CFE_FN StepOut step(S& s, Hot& h, int action, uint64_t rng, SpawnPlan& plan) {
    const uint32_t ach0[3] = {h.ach[0], h.ach[1], h.ach[2]};
    const float health0 = h.health;
    if (h.sleeping || h.resting) action = A_NOOP;

    change_floor(s, h, action);
    s.open_level(wrap_clamp(h.level, kLevels));
    s.stamp(2);
    craft(s, h, action);
    uint64_t key = next_key(rng);
    if (action == A_DO) do_action(s, h, key);
    s.stamp(3);
    place_block(s, h, action);
    shoot_or_cast(s, h, action);
    drink_potion(s, h, action);
    key = next_key(rng);
    read_book(h, key, action);
    key = next_key(rng);
    enchant(s, h, action, key);
    boss_and_attributes(h, action);
    move_player(s, h, action);
    s.stamp(4);
    key = next_key(rng);
    update_mobs(s, h, key);
    s.stamp(5);
    key = next_key(rng);
    plan = plan_spawns(s, h, key);
    grow_plants(s, h);
    update_intrinsics(h, action);
    clip_and_count(h);
    s.stamp(6);

    float reward = 0.0f;
#pragma unroll
    for (int w = 0; w < 3; w++)
        for (uint32_t fresh = h.ach[w] & ~ach0[w]; fresh != 0; fresh &= fresh - 1)
            reward += achievement_reward(32 * w + __builtin_ctz(fresh));
    reward += (h.health - health0) * 0.1f;

    StepOut out;
    out.state_rng = next_key(rng);
    h.timestep += 1;
    h.light_level = s.light_at(h.timestep);
    out.reward = reward;
    out.done = h.timestep >= kMaxTimesteps || h.health <= 0.0f;  // craftax_is_game_over_native, :3769
    return out;
}

// c_step_gameplay's key schedule (:3989-3993): the env key advances one LCG state, the
// step's own generator is two states further, the reset key three
struct StepKeys {
    uint64_t env_key, step_rng, reset_key;
};
CFE_FN StepKeys split_env_key(uint64_t env_key) {
    StepKeys k;
    k.env_key = lcg(env_key);
    k.step_rng = lcg(lcg(k.env_key));
    k.reset_key = lcg(k.step_rng);
    return k;
}
CFE_FN int clamp_action(float a) {  // :3985-3987
    int v = (int)a;
    return v < 0 ? 0 : (v >= kNumActions ? kNumActions - 1 : v);
}
CFE_FN uint32_t xorshift32(uint32_t x) {  // cf_xorshift32, :8238-8245
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x ? x : 0xdeadbeefu;
}

}  // namespace cfenv
