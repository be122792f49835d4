// World generation for a reset (craftax_generate_world_from_key, craftax_full.c:2050-2142):
// nine floors -- six "smooth" ones from four Perlin fields each (:209-300, 443-503,
// 1248-1359, 1577-1700) and three dungeons of rooms and corridors (:1733-1944) -- plus the
// player's starting scalars.  Written once for a cooperating group of threads: the gfx950
// reset kernel runs it with one workgroup of 256 or 512 threads per (env, floor) and the floor's
// working set (four 48x48 float fields, the byte planes, the dungeon's padded canvas) in
// LDS; the host build runs the same text with a group of one.  `G` supplies the group:
//   int tid(), nt(); void sync(); void gminmax4(float (&)[4], float (&)[4]); int gmaxi(int);
//   int gscan(int v, int& total)   exclusive prefix sum over the threads in tid order
//   float cosine(float), sine(float)
// Every per-cell draw is a pure function of (key, cell), so the split of cells over
// threads does not change a value; reductions are min / max / integer sums (exact).
//
// Floating point follows the reference's GPU port (strict per-operation fp32, division by
// a literal constant as multiplication by its rounded reciprocal, craftax_full.cu:1196,
// 1254): compile with contraction off.  The gradient table's cos / sin are the group's:
// the C library's on the host, a double-precision evaluation rounded to float on the GPU,
// which can differ from the C library's in the last bit for a small fraction of arguments
// (a cell of a map changes only if a noise value lies within that bit of a threshold).
#pragma once

#include "env_logic.h"

namespace cfenv {

constexpr int kCells = kMap * kMap;     // 2304
constexpr int kPad = 10;                // max room size: the dungeon canvas is padded by it
constexpr int kCanvas = kMap + 2 * kPad;  // 68

// CRAFTAX_SMOOTHGEN_CONFIGS (craftax_full.c:852-1015), one row per smooth floor
// (floors 0, 2, 5, 6, 7, 8).
struct SmoothCfg {
    uint8_t base, sea, coast, mountain, path, inner;
    uint8_t ore_on[5], ore[5];
    float ore_chance[5];
    uint8_t tree_on, tree, lava, spawn, ladder_on;
    bool ladder_up, ladder_down;
    float water_strength, water_max, mountain_strength, mountain_max, light;
    float water_thr, sand_thr, tree_thr_uniform, tree_thr_perlin;
};
CFE_FN SmoothCfg smooth_cfg(int ci) {
    SmoothCfg c;
    // members that are the same on every smooth floor
    c.sea = B_WATER;
    c.mountain = B_STONE;
    c.path = B_STONE;
    c.inner = B_STONE;
    for (int i = 0; i < 5; i++) c.ore_on[i] = B_STONE;
    c.ore[0] = B_COAL; c.ore[1] = B_IRON; c.ore[2] = B_DIAMOND; c.ore[3] = B_SAPPHIRE; c.ore[4] = B_RUBY;
    c.lava = B_LAVA;
    c.ladder_up = c.ladder_down = true;
    c.water_strength = 5.0f; c.water_max = 1.0f; c.mountain_strength = 17.0f; c.mountain_max = 1.5f;
    c.light = 0.0f;
    c.water_thr = 0.7f; c.sand_thr = 0.6f; c.tree_thr_uniform = 0.8f; c.tree_thr_perlin = 0.5f;
    if (ci == 0) {          // overworld
        c.base = B_GRASS; c.coast = B_SAND; c.path = B_PATH; c.inner = B_PATH;
        c.ore[3] = c.ore[4] = B_OOB;
        c.ore_chance[0] = 0.03f; c.ore_chance[1] = 0.02f; c.ore_chance[2] = 0.001f; c.ore_chance[3] = c.ore_chance[4] = 0.0f;
        c.tree_on = B_GRASS; c.tree = B_TREE; c.spawn = B_GRASS; c.ladder_on = B_PATH;
        c.ladder_up = false;
        c.mountain_strength = 5.0f; c.mountain_max = 1.0f; c.light = 1.0f;
    } else if (ci == 1 || ci == 2) {   // gnomish mines, troll mines
        c.base = B_PATH; c.coast = B_PATH;
        const bool deep = ci == 2;
        c.ore_chance[0] = 0.04f; c.ore_chance[1] = deep ? 0.03f : 0.02f; c.ore_chance[2] = deep ? 0.01f : 0.005f;
        c.ore_chance[3] = c.ore_chance[4] = deep ? 0.01f : 0.0025f;
        c.tree_on = B_PATH; c.tree = B_STALAGMITE; c.spawn = B_PATH; c.ladder_on = B_PATH;
    } else if (ci == 3) {   // fire realm
        c.base = B_FIRE_GRASS; c.sea = B_LAVA; c.coast = B_SAND;
        c.ore_chance[0] = 0.05f; c.ore_chance[1] = c.ore_chance[2] = c.ore_chance[3] = 0.0f; c.ore_chance[4] = 0.025f;
        c.tree_on = B_FIRE_GRASS; c.tree = B_FIRE_TREE; c.spawn = B_FIRE_GRASS; c.ladder_on = B_FIRE_GRASS;
        c.mountain_strength = 5.0f; c.mountain_max = 1.0f; c.light = 1.0f; c.water_thr = 0.5f;
    } else if (ci == 4) {   // ice realm
        c.base = B_ICE_GRASS; c.coast = B_ICE_GRASS;
        c.ore_chance[0] = c.ore_chance[1] = 0.0f; c.ore_chance[2] = 0.005f; c.ore_chance[3] = 0.02f; c.ore_chance[4] = 0.0f;
        c.tree_on = B_ICE_GRASS; c.tree = B_ICE_SHRUB; c.lava = B_WATER; c.spawn = B_ICE_GRASS; c.ladder_on = B_ICE_GRASS;
        c.water_thr = 0.5f; c.tree_thr_uniform = 0.4f;
    } else {                // graveyard
        c.base = B_PATH; c.sea = B_PATH; c.coast = B_PATH; c.mountain = B_WALL; c.path = B_WALL; c.inner = B_WALL;
        c.ore_on[1] = c.ore_on[2] = B_GRAVE;
        c.ore_on[0] = c.ore_on[3] = c.ore_on[4] = B_WALL;
        c.ore[0] = B_WALL_MOSS; c.ore[1] = B_GRAVE2; c.ore[2] = B_GRAVE3;
        c.ore_chance[0] = 0.1f; c.ore_chance[1] = 0.333f; c.ore_chance[2] = 0.5f; c.ore_chance[3] = c.ore_chance[4] = 0.0f;
        c.tree_on = B_PATH; c.tree = B_GRAVE; c.lava = B_WALL; c.spawn = B_NECROMANCER; c.ladder_on = B_PATH;
        c.ladder_up = c.ladder_down = false;
        c.mountain_strength = 10.0f; c.mountain_max = 10.0f;
        c.tree_thr_uniform = 0.95f; c.tree_thr_perlin = -1.0f;
    }
    return c;
}

// what the dungeon's eight rooms and eight corridors are, as numbers (canvas coordinates)
struct DungeonPlan {
    int8_t size_r[8], size_c[8], pos_r[8], pos_c[8];
    int8_t chest_r[8], chest_c[8];
    int8_t fountain_r[8], fountain_c[8];   // row -1: this room has no fountain
    int8_t h_row[8], h_c0[8], h_c1[8];     // corridor k: cells (h_row, h_c0..h_c1) ...
    int8_t v_col[8], v_r0[8], v_r1[8];     // ... and (v_r0..v_r1, v_col); an empty leg has end -1
};
// corners of the four noise fields of a smooth floor: 4 x 4, 4 x 4, 7 x 25, 13 x 13
constexpr int kGradTotal = 16 + 16 + 175 + 169;
// per-floor working set (LDS on the GPU)
struct alignas(16) FloorScratch {
    float field[4][kCells];     // water, mountain, path, tree noise
    uint8_t map[kCells], item[kCells], light[kCells], lava[kCells];
    float gx[kGradTotal], gy[kGradTotal];   // gradient tables of the four fields, one after the other
    int32_t ladder_down[2], ladder_up[2];
    DungeonPlan plan;
};
// the dungeon's padded canvas lives where the noise fields are (a dungeon floor has none)
static_assert(2 * kCanvas * kCanvas <= 4 * (int)sizeof(float) * kCells, "canvas fits in the noise fields");

CFE_FN uint64_t hash_at(uint64_t key, uint64_t index) { return fmix64(key ^ index); }
CFE_FN uint32_t u32_at(uint64_t key, uint64_t index) {
    const uint64_t h = hash_at(key, index);
    return (uint32_t)h ^ (uint32_t)(h >> 32);
}
CFE_FN float unit_at(uint64_t key, uint64_t index) { return bits_to_float((u32_at(key, index) >> 9) | 0x3F800000u) - 1.0f; }
CFE_FN int int_at(uint64_t key, uint64_t index, int lo, int hi) {   // craftax_randint_i32_at, :1079-1108
    const uint32_t span = (uint32_t)hi > (uint32_t)lo ? (uint32_t)hi - (uint32_t)lo : 1u;
    if ((span & (span - 1)) == 0) return (int)((uint32_t)lo + (u32_at(key, index) & (span - 1)));
    return (int)((uint32_t)lo + (uint32_t)(((hash_at(key, index) >> 32) * (uint64_t)span) >> 32));
}

// this thread's contiguous share of the floor's cells
template <class G>
CFE_FN void my_cells(G& g, int& lo, int& hi) {
    const int per = (kCells + g.nt() - 1) / g.nt();
    lo = g.tid() * per;
    hi = lo + per < kCells ? lo + per : kCells;
    if (lo > kCells) lo = kCells;
}

// craftax_choice_bool_flat (:1110-1138) over the floor's cells: the ceil(n * (1 - u))-th cell
// with flag set (0 when none is).  `flag(i)` is evaluated by the thread that owns cell i.
template <class G, class F>
CFE_FN int choose_cell(G& g, uint64_t key, F flag) {
    int lo, hi;
    my_cells(g, lo, hi);
    int mine = 0;
    for (int i = lo; i < hi; i++) mine += (int)flag(i);
    int total;
    const int before = g.gscan(mine, total);
    if (total == 0) return 0;
    const float draw = (float)total * (1.0f - draw_unit(key));
    int want = (int)__builtin_ceilf(draw);      // 1-based rank; counts up to 2304 are exact floats
    want = want < 1 ? 1 : (want > total ? total : want);
    int found = -1;
    if (want > before && want <= before + mine) {
        int seen = before;
        for (int i = lo; i < hi; i++)
            if (flag(i) && ++seen == want) {
                found = i;
                break;
            }
    }
    return g.gmaxi(found);
}

// The four normalised Perlin fields of a smooth floor (each craftax_generate_fractal_noise_2d
// with one octave, :443-503; craftax_generate_perlin_noise_2d_scalar, :209-300), made together:
// one pass over the gradient corners of all four, one over the cells, one group reduction for
// the eight extrema.  Field f: subkey[f], res_r[f] x res_c[f] periods, result in sc.field[f].
template <class G>
CFE_FN void noise_fields(G& g, FloorScratch& sc, const uint64_t (&subkey)[4], const int (&res_r)[4],
                         const int (&res_c)[4]) {
    int base[4];
    int corners = 0;
#pragma unroll
    for (int f = 0; f < 4; f++) {
        base[f] = corners;
        corners += (res_r[f] + 1) * (res_c[f] + 1);
    }
    for (int k = g.tid(); k < corners; k += g.nt()) {
        // (selects, not indexing: the small tables stay in registers)
        uint64_t sk = subkey[0];
        int first = 0;
#pragma unroll
        for (int f = 1; f < 4; f++)
            if (k >= base[f]) {
                sk = subkey[f];
                first = base[f];
            }
        const uint64_t angle_key = lcg(lcg(lcg(lcg(sk))));   // two splits, the right key each time
        const float angle = 6.28318530717958647692f * unit_at(angle_key, (uint64_t)(k - first));
        sc.gx[k] = g.cosine(angle);
        sc.gy[k] = g.sine(angle);
    }
    g.sync();
    int lo, hi;
    my_cells(g, lo, hi);
    float vmin[4], vmax[4];
#pragma unroll
    for (int f = 0; f < 4; f++) {
        vmin[f] = 3.0e38f;
        vmax[f] = -3.0e38f;
    }
    for (int i = lo; i < hi; i++) {
        const int row = i / kMap, col = i - row * kMap;
#pragma unroll
        for (int f = 0; f < 4; f++) {
            const int gw = res_c[f] + 1;
            const int cr = kMap / res_r[f], cc = kMap / res_c[f];
            const float* gx = sc.gx + base[f];
            const float* gy = sc.gy + base[f];
            const int gr = row / cr, gc = col / cc;
            const float lr = (float)(row - gr * cr) / (float)cr, lc = (float)(col - gc * cc) / (float)cc;
            const float ir = lr * lr * lr * (lr * (lr * 6.0f - 15.0f) + 10.0f);
            const float ic = lc * lc * lc * (lc * (lc * 6.0f - 15.0f) + 10.0f);
            const int i00 = gr * gw + gc, i10 = i00 + gw;
            float n00 = lr * gx[i00];
            n00 += lc * gy[i00];
            float n10 = (lr - 1.0f) * gx[i10];
            n10 += lc * gy[i10];
            float n01 = lr * gx[i00 + 1];
            n01 += (lc - 1.0f) * gy[i00 + 1];
            float n11 = (lr - 1.0f) * gx[i10 + 1];
            n11 += (lc - 1.0f) * gy[i10 + 1];
            const float n0 = n00 * (1.0f - ir) + ir * n10;
            const float n1 = n01 * (1.0f - ir) + ir * n11;
            float v = 1.41421356237309504880f * ((1.0f - ic) * n0 + ic * n1);
            v = 0.0f + 1.0f * v;     // the octave accumulation: out = 0; out += amplitude * perlin
            sc.field[f][i] = v;
            vmin[f] = v < vmin[f] ? v : vmin[f];
            vmax[f] = v > vmax[f] ? v : vmax[f];
        }
    }
    g.gminmax4(vmin, vmax);
#pragma unroll
    for (int f = 0; f < 4; f++) {
        const float scale = vmax[f] - vmin[f];
        for (int i = lo; i < hi; i++) sc.field[f][i] = (sc.field[f][i] - vmin[f]) / scale;
    }
    g.sync();
}

// craftax_generate_smoothworld_config (:1577-1700)
template <class G>
CFE_FN void smooth_floor(G& g, FloorScratch& sc, uint64_t rng, int ci) {
    const SmoothCfg c = smooth_cfg(ci);
    float* water = sc.field[0];
    float* mountain = sc.field[1];
    float* path = sc.field[2];
    float* tree = sc.field[3];
    uint64_t sub[4];
    sub[0] = next_key(rng);
    (void)next_key(rng);
    sub[1] = next_key(rng);
    sub[2] = next_key(rng);
    (void)next_key(rng);
    sub[3] = next_key(rng);
    const uint64_t tree_key = rng;
    const int res_r[4] = {3, 3, 6, 12}, res_c[4] = {3, 3, 24, 12};
    noise_fields(g, sc, sub, res_r, res_c);
    g.stamp(1);

    uint64_t ore_rng = next_key(rng);
    uint64_t ore_key[5];
    for (int k = 0; k < 5; k++) ore_key[k] = next_key(ore_rng);

    int lo, hi;
    my_cells(g, lo, hi);
    const uint8_t default_light = (uint8_t)(c.light * 255.0f);
    for (int i = lo; i < hi; i++) {
        // craftax_smoothworld_classify_scalar (:1248-1321)
        const int row = i / kMap, col = i - row * kMap;
        const int dr = iabs(row - kMap / 2), dc = iabs(col - kMap / 2);
        const float dist = __builtin_sqrtf((float)(dr * dr + dc * dc));
        float pw = dist / c.water_strength;
        pw = pw < 0.0f ? 0.0f : (pw > c.water_max ? c.water_max : pw);
        float pm = dist / c.mountain_strength;
        pm = pm < 0.0f ? 0.0f : (pm > c.mountain_max ? c.mountain_max : pm);
        const float w = water[i] + pw - 1.0f;
        int b = w > c.water_thr ? c.sea : c.base;
        if (w > c.sand_thr && b != c.sea) b = c.coast;
        const float m = mountain[i] + 0.05f + pm - 1.0f;
        if (m > 0.7f) b = c.mountain;
        if (m > 0.7f && path[i] > 0.8f) b = c.path;
        if (m > 0.7f && path[col * kMap + row] > 0.8f) b = c.path;
        if (m > 0.85f && w > 0.4f) b = c.inner;
        const float t = tree[i];
        if (t > c.tree_thr_perlin && unit_at(tree_key, (uint64_t)i) > c.tree_thr_uniform && b == c.tree_on) b = c.tree;
        // craftax_smoothworld_ore_scalar x 5 (:1323-1340), craftax_smoothworld_lava_scalar (:1342-1359)
        for (int k = 0; k < 5; k++)
            if (b == c.ore_on[k] && unit_at(ore_key[k], (uint64_t)i) < c.ore_chance[k]) b = c.ore[k];
        const bool lava = m > 0.85f && t > 0.7f;
        if (lava) b = c.lava;
        sc.map[i] = (uint8_t)b;
        sc.item[i] = I_NONE;
        sc.light[i] = default_light;
        sc.lava[i] = lava;
    }
    g.sync();
    g.stamp(2);

    // the diamond draw (:1662-1670) rewrites a stone cell with stone -- or cell 0 when the
    // floor has no stone at all
    uint64_t key = next_key(rng);
    const int diamond = choose_cell(g, key, [&](int i) { return sc.map[i] == B_STONE; });
    if (g.tid() == 0) {
        sc.map[diamond] = B_STONE;
        sc.map[(kMap / 2) * kMap + kMap / 2] = c.spawn;
    }
    g.sync();
    key = next_key(rng);
    const int down = choose_cell(g, key, [&](int i) { return sc.map[i] == c.ladder_on; });
    key = next_key(rng);
    const int up = choose_cell(g, key, [&](int i) { return sc.map[i] == c.ladder_on; });
    if (g.tid() == 0) {
        sc.ladder_down[0] = down / kMap;
        sc.ladder_down[1] = down % kMap;
        sc.ladder_up[0] = up / kMap;
        sc.ladder_up[1] = up % kMap;
        if (c.ladder_down) sc.item[down] = I_LADDER_DOWN;
    }
    g.stamp(3);
    // craftax_apply_ladder_light (:1148-1169): a 9x9 torch pattern around the up ladder
    int r0 = up / kMap - 4, c0 = up % kMap - 4;
    if (r0 < 0) r0 += kMap;
    if (c0 < 0) c0 += kMap;
    r0 = r0 > kMap - 9 ? kMap - 9 : r0;
    c0 = c0 > kMap - 9 ? kMap - 9 : c0;
    for (int k = g.tid(); k < 81; k += g.nt()) {
        const int row = k / 9, col = k - row * 9;
        const float fr = (float)(row - 4), fc = (float)(col - 4);
        const float dist = __builtin_sqrtf(fr * fr + fc * fc);
        float torch = 1.0f - dist * (1.0f / 5.0f);
        torch = torch < 0.0f ? 0.0f : (torch > 1.0f ? 1.0f : torch);
        const float v = torch * (1.0f - c.light) + c.light;
        sc.light[(r0 + row) * kMap + c0 + col] = (uint8_t)(v * 255.0f);
    }
    g.sync();
    // craftax_add_lava_light (:1171-1206)
    if (c.lava == B_LAVA) {
        for (int i = lo; i < hi; i++) {
            const int row = i / kMap, col = i - row * kMap;
            float add = 0.0f;
            for (int kr = -1; kr <= 1; kr++) {
                if ((unsigned)(row + kr) >= (unsigned)kMap) continue;
                for (int kc = -1; kc <= 1; kc++) {
                    if ((unsigned)(col + kc) >= (unsigned)kMap) continue;
                    const float k = (kr == 0 && kc == 0) ? 1.0f : ((kr == 0 || kc == 0) ? 0.7f : 0.2f);
                    add += sc.lava[(row + kr) * kMap + col + kc] ? k : 0.0f;
                }
            }
            float v = (float)sc.light[i] * (1.0f / 255.0f) + add;
            v = v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v);
            sc.light[i] = (uint8_t)(v * 255.0f);
        }
    }
    g.sync();
    if (g.tid() == 0 && c.ladder_up) sc.item[up] = I_LADDER_UP;
    g.sync();
    g.stamp(4);
}

// craftax_generate_dungeon_config (:1733-1944).  Rooms and corridors are a few hundred
// dependent byte writes: one thread lays them out, the group does the per-cell passes.
template <class G>
CFE_FN void dungeon_floor(G& g, FloorScratch& sc, uint64_t rng, int ci) {
    const uint8_t special = ci == 0 ? B_PATH : (ci == 1 ? B_ENCH_ICE : B_ENCH_FIRE);
    const uint8_t fountain = ci == 1 ? B_WATER : B_FOUNTAIN;
    const uint8_t rare_path = ci == 1 ? B_WATER : B_PATH;
    uint8_t* canvas = reinterpret_cast<uint8_t*>(sc.field[0]);
    uint8_t* items = canvas + kCanvas * kCanvas;
    // key schedule: split3 -> (rng, ignored, room sizes); split -> room_rng; later path_rng, rare, ladders
    const uint64_t size_key = lcg(lcg(lcg(rng)));
    rng = lcg(rng);
    uint64_t room_rng = next_key(rng);
    uint64_t path_rng = next_key(rng);
    // The reference draws eight rooms and eight corridors one after the other onto the canvas
    // (a few hundred dependent byte writes).  Here one thread only draws the numbers -- the
    // plan below, arithmetic and no memory -- and the group paints from it: the rooms in
    // order, a cell a thread; then the corridors, which only ever turn wall into path and so
    // need no order among themselves; then the special block of room 0.
    DungeonPlan& plan = sc.plan;
    if (g.tid() == 0) {
        for (int k = 0; k < 8; k++) {
            plan.size_r[k] = (int8_t)int_at(size_key, 2 * k, 5, 10);
            plan.size_c[k] = (int8_t)int_at(size_key, 2 * k + 1, 5, 10);
        }
        uint32_t free_chunks = 0x1ff;
        for (int k = 0; k < 8; k++) {
            // craftax_choice_bool_flat over the nine 16x16 chunks still free
            uint64_t key = next_key(room_rng);
            const int nfree = __builtin_popcount(free_chunks);
            int want = (int)__builtin_ceilf((float)nfree * (1.0f - draw_unit(key)));
            want = want < 1 ? 1 : (want > nfree ? nfree : want);
            uint32_t m = free_chunks;
            for (int j = 1; j < want; j++) m &= m - 1;
            const int chunk = __builtin_ctz(m);
            free_chunks &= ~(1u << chunk);
            key = next_key(room_rng);
            const int rr = (chunk % 3) * 16 + kPad + int_at(key, 0, 0, 11);
            const int rc = (chunk / 3) * 16 + kPad + int_at(key, 1, 0, 11);
            plan.pos_r[k] = (int8_t)rr;
            plan.pos_c[k] = (int8_t)rc;
            key = next_key(room_rng);
            plan.chest_r[k] = (int8_t)(rr + int_at(key, 0, 1, plan.size_r[k] - 1));
            plan.chest_c[k] = (int8_t)(rc + int_at(key, 1, 1, plan.size_c[k] - 1));
            // split3: (room_rng, fountain position, fountain coin)
            const uint64_t fkey = lcg(lcg(room_rng)), coin = lcg(fkey);
            room_rng = lcg(room_rng);
            const int fr = int_at(fkey, 0, 1, plan.size_r[k] - 1), fc = int_at(fkey, 1, 1, plan.size_c[k] - 1);
            const bool has = draw_unit(coin) > 0.5f;
            plan.fountain_r[k] = (int8_t)(has ? rr + fr : -1);
            plan.fountain_c[k] = (int8_t)(rc + fc);
        }
        uint32_t linked = 0x80;   // room 7 is the first sink
        for (int k = 0; k < 8; k++) {
            const uint64_t key = next_key(path_rng);
            const int nlinked = __builtin_popcount(linked);
            int want = (int)__builtin_ceilf((float)nlinked * (1.0f - draw_unit(key)));
            want = want < 1 ? 1 : (want > nlinked ? nlinked : want);
            uint32_t m = linked;
            for (int j = 1; j < want; j++) m &= m - 1;
            const int sink = __builtin_ctz(m);
            // the corridor runs along room k's row to the sink's column, then along that column
            const int ck = plan.pos_c[k], cs = plan.pos_c[sink], rk = plan.pos_r[k], rs = plan.pos_r[sink];
            plan.h_row[k] = (int8_t)rk;
            plan.h_c0[k] = (int8_t)(ck < cs ? ck : cs);
            plan.h_c1[k] = (int8_t)(ck == cs ? -1 : (ck < cs ? cs : ck));   // empty when the columns agree
            plan.v_col[k] = (int8_t)cs;
            plan.v_r0[k] = (int8_t)(rk < rs ? rk : rs);
            plan.v_r1[k] = (int8_t)(rk == rs ? -1 : (rk < rs ? rs : rk));
            path_rng = lcg(lcg(path_rng));
            linked |= 1u << k;
        }
    }
    g.sync();
    g.stamp(1);
    for (int k = g.tid(); k < kCanvas * kCanvas; k += g.nt()) {
        const int row = k / kCanvas, col = k - row * kCanvas;
        const bool inner = row >= kPad && row < kPad + kMap && col >= kPad && col < kPad + kMap;
        canvas[k] = inner ? B_WALL : 0;
        items[k] = I_NONE;
    }
    g.sync();
    // rooms one after the other (a later room's floor covers what an earlier one put where
    // they overlap), each cell of a room written once by its own thread: floor, or the chest,
    // or the fountain, which is drawn after the chest
    for (int q = 0; q < 8; q++) {
        const int rr = plan.pos_r[q], rc = plan.pos_c[q], sr = plan.size_r[q], sz = plan.size_c[q];
        for (int k = g.tid(); k < sr * sz; k += g.nt()) {
            const int a = k / sz, b = k - a * sz;
            const int row = rr + a, col = rc + b;
            int v = B_PATH;
            if (row == plan.chest_r[q] && col == plan.chest_c[q]) v = B_CHEST;
            if (row == plan.fountain_r[q] && col == plan.fountain_c[q]) v = fountain;
            canvas[row * kCanvas + col] = (uint8_t)v;
            if ((a == 0 || a == sr - 1) && (b == 0 || b == sz - 1)) items[row * kCanvas + col] = I_TORCH;
        }
        g.sync();
    }
    // the sixteen corridor legs together: each only turns wall into path
    for (int k = g.tid(); k < 16 * 64; k += g.nt()) {
        const int leg = k >> 6, i = k & 63, q = leg & 7;
        int row, col;
        bool on;
        if (leg < 8) {
            row = plan.h_row[q];
            col = plan.h_c0[q] + i;
            on = col <= plan.h_c1[q];
        } else {
            col = plan.v_col[q];
            row = plan.v_r0[q] + i;
            on = row <= plan.v_r1[q];
        }
        if (on && canvas[row * kCanvas + col] == B_WALL) canvas[row * kCanvas + col] = B_PATH;
    }
    g.sync();
    if (g.tid() == 0) canvas[(plan.pos_r[0] + 2) * kCanvas + plan.pos_c[0] + 2] = special;
    g.sync();
    g.stamp(2);
    const uint64_t rare_key = next_key(rng);
    int lo, hi;
    my_cells(g, lo, hi);
    for (int i = lo; i < hi; i++) {
        const int row = i / kMap, col = i - row * kMap;
        const uint8_t* p = canvas + (row + kPad) * kCanvas + col + kPad;
        const int b = p[0], it = items[(row + kPad) * kCanvas + col + kPad];
        // a wall cell with no open neighbour inside the map is darkness; the canvas border is 0
        bool open = b != B_WALL;
        open = open || (row > 0 && p[-kCanvas] != B_WALL) || (row + 1 < kMap && p[kCanvas] != B_WALL);
        open = open || (col > 0 && p[-1] != B_WALL) || (col + 1 < kMap && p[1] != B_WALL);
        const bool rare = (1.0f - unit_at(rare_key, (uint64_t)i)) > 0.9f;
        int out = b;
        if (!open) out = B_DARKNESS;
        else if (b == B_WALL) out = rare ? B_WALL_MOSS : B_WALL;
        else if (rare && b == B_PATH && it == I_NONE) out = rare_path;
        sc.map[i] = (uint8_t)out;
        sc.item[i] = (uint8_t)it;
        sc.light[i] = 255;
        sc.lava[i] = 0;
    }
    g.sync();
    g.stamp(3);
    uint64_t key = next_key(rng);
    const int down = choose_cell(g, key, [&](int i) { return sc.map[i] == B_PATH; });
    key = next_key(rng);
    const int up = choose_cell(g, key, [&](int i) { return sc.map[i] == B_PATH; });
    if (g.tid() == 0) {
        sc.ladder_down[0] = down / kMap;
        sc.ladder_down[1] = down % kMap;
        sc.ladder_up[0] = up / kMap;
        sc.ladder_up[1] = up % kMap;
        sc.item[down] = I_LADDER_DOWN;
        sc.item[up] = I_LADDER_UP;   // written second: wins when both land on one cell
    }
    g.sync();
    g.stamp(4);
}

// The key of each floor and of the two trailing draws (craftax_generate_world_from_key_lazy,
// :2057-2125): with s_k = the k-th LCG state after the world key, the smooth floors 0, 2, 5, 6,
// 7, 8 take s_2 .. s_7, the dungeons 1, 3, 4 take s_3, s_4, s_5, the potion permutation s_4
// and the state key s_5.
CFE_FN uint64_t lcg_n(uint64_t s, int n) {
    for (int i = 0; i < n; i++) s = lcg(s);
    return s;
}
CFE_FN uint64_t floor_key(uint64_t world_key, int level) {
    const int steps = level == 0 ? 2 : level == 2 ? 3 : level == 5 ? 4 : level == 6 ? 5 : level == 7 ? 6
                    : level == 8 ? 7 : level == 1 ? 3 : level == 3 ? 4 : 5;
    return lcg_n(world_key, steps);
}
CFE_FN bool floor_is_dungeon(int level) { return level == 1 || level == 3 || level == 4; }
CFE_FN int floor_config(int level) {   // index into the smooth / dungeon configs
    return level == 0 ? 0 : level == 2 ? 1 : level == 5 ? 2 : level == 6 ? 3 : level == 7 ? 4 : level == 8 ? 5
         : level == 1 ? 0 : level == 3 ? 1 : 2;
}
template <class G>
CFE_FN void generate_floor(G& g, FloorScratch& sc, uint64_t world_key, int level) {
    if (floor_is_dungeon(level)) dungeon_floor(g, sc, floor_key(world_key, level), floor_config(level));
    else smooth_floor(g, sc, floor_key(world_key, level), floor_config(level));
}
// craftax_permutation_6 (:1977-2001): stable ascending order of six 32-bit draws
CFE_FN void potion_permutation(uint64_t world_key, int32_t (&out)[6]) {
    const uint64_t sort_key = lcg(lcg(lcg_n(world_key, 4)));
    uint32_t k[6];
    for (int i = 0; i < 6; i++) {
        k[i] = u32_at(sort_key, (uint64_t)i);
        out[i] = i;
    }
    for (int i = 1; i < 6; i++)
        for (int j = i; j > 0 && k[j - 1] > k[j]; j--) {
            const uint32_t tk = k[j]; k[j] = k[j - 1]; k[j - 1] = tk;
            const int32_t tv = out[j]; out[j] = out[j - 1]; out[j - 1] = tv;
        }
}
CFE_FN uint64_t world_state_key(uint64_t world_key) { return lcg_n(world_key, 5); }
// keys of an env created from `seed` (craftax_reset_state_from_seed, :3601-3614): the env's
// own key and the key of its first world; and of a world from a reset key (:3545-3553)
CFE_FN uint64_t seed_key(uint32_t seed) { return (uint64_t)(seed ^ 0x9E3779B9u) << 32 | seed; }
CFE_FN uint64_t world_key_of_reset(uint64_t reset_key) { return lcg(lcg(reset_key)); }

}  // namespace cfenv
